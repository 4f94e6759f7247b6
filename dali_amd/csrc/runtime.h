// Internals shared by the translation units of libdali_hip.so.
#ifndef DALI_HIP_RUNTIME_H
#define DALI_HIP_RUNTIME_H

#include <hip/hip_runtime.h>

#include <string>

#include "../../include/dali_hip.h"

namespace dali_hip {

// Workspace of the two-stage reductions: kWorkspaceCounters uint32 counters
// (zero at creation, reset to zero by the block that consumes them) followed by
// kWorkspacePartialBytes of partial results.
constexpr int kWorkspaceCounters = 16384;
constexpr size_t kWorkspaceCounterBytes = (size_t)kWorkspaceCounters * 4;
constexpr size_t kWorkspacePartialBytes = (size_t)32 << 20;
constexpr size_t kWorkspaceBytes = kWorkspaceCounterBytes + kWorkspacePartialBytes;

int fail(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
int fail_str(const std::string& s);
int ensure_init();
hipStream_t stream();
char* workspace();
// device the library is bound to, -1 before dali_hip_init
int bound_device();
// sort.hip: looks up the device address of its built-in scratch array; called by dali_hip_init with `device` current
int sort_scratch_init(int device);
// sgemm_skinny.hip: row-major C[M, N] = alpha * A[M, K] . B[K, N] + beta * C for M <= 64 by streaming B once
// (tb: B stored as [N][K]). 1: launched; 0: not a case for it (take the tiled kernels); -1: failure (message set)
int sgemm_skinny(bool tb, int M, int N, int K, float alpha, const float* A, int lda, const float* B, int ldb, float beta, float* C, int ldc);
// sgemv.hip: y[M] = alpha * A[M, K] . x[K] + beta * y for row-major A, strides in elements; 1 = launched, 0 = not taken, -1 = error
int sgemv_rows(int M, int K, float alpha, const float* A, int lda, const float* x, int incx, float beta, float* y, int incy);
// the same for an inner extent of at most 64 against a large C (ta: A stored as [K][M]): bound by writing C once
int sgemm_smallk(bool ta, bool tb, int M, int N, int K, float alpha, const float* A, int lda, const float* B, int ldb, float beta, float* C, int ldc);
// sgemm_dma.hip: row-major C[M, N] = alpha * sum_s A_s . B_s + beta * C for one or two terms of whole 64-deep slabs through
// the kernel whose operand slabs are written into LDS by the loads themselves (ta: A_s stored as [K][M], tb: B_s stored as
// [N][K]; leading dimensions per term). With `bias` the sums go through the LSTM gate arithmetic instead of into C
// (N = 4 H, columns gathered per hidden unit). 1: launched; 0: not a case for it; -1: failure (message set)
int sgemm_dma(bool ta, bool tb, int M, int N, int nseg, const int* K, const float* const* A, const float* const* B, const int* lda, const int* ldb,
              float alpha, float beta, float* C, int ldc, const float* bias, const float* c_prev, float* c_out, float* h_out, int H);
// The same pipeline over a stream of work items per workgroup (one workgroup per compute unit walks many tiles, its loads
// running ahead across tile boundaries); `shares` > 1 cuts every tile's inner extent into that many contiguous shares that meet
// in the library workspace (single products only). `cus`: compute units of the bound device. Same return values.
// With `bias` the sums go through the LSTM gate arithmetic instead of into C, as in sgemm_dma.
int sgemm_dma_stream(bool ta, bool tb, int M, int N, int nseg, const int* K, const float* const* A, const float* const* B, const int* lda, const int* ldb,
                     float alpha, float beta, float* C, int ldc, int shares, int cus, const float* bias = nullptr, const float* c_prev = nullptr,
                     float* c_out = nullptr, float* h_out = nullptr, int H = 0);
// sgemm_dma128.hip: row-major C[M, N] = alpha * A . B + beta * C over whole 32-deep slabs with 128x128 tiles, one workgroup per
// compute unit walking a list of tiles (ta: A stored as [K][M]; tb: B stored as [N][K]). Same return values.
int sgemm_dma128(bool ta, bool tb, int M, int N, int K, const float* A, int lda, const float* B, int ldb, float alpha, float beta, float* C, int ldc, int cus);
// hipFuncSetAttribute(MaxDynamicSharedMemorySize) once per kernel: later launches of that kernel, which may be recorded into a
// graph, are launches only. Keyed on the kernel's address (kernels of one signature share a function type, so a flag inside a
// generic lambda or template would be shared among them).
hipError_t reserve_dynamic_lds(const void* kernel, size_t bytes);
// recurrent_phased.hip: the recurrent half of a sequence in one launch for up to 128 rows and hidden sizes that are multiples of
// 64 up to 2048 (weights in registers, two row blocks taking turns at the grid barrier). `status` is the host-visible word that a
// workgroup sets when a wait gives up; `cus` the number of compute units of the bound device.
int recurrent_phased_supported(int batch, int hidden, int cus);
int lstm_recurrent_phased(int steps, int batch, int hidden, const float* pre, const float* U, int ldu, const float* h0, const float* c0, float* hs,
                          float* c_out, int* status, int cus);
int gru_recurrent_phased(int steps, int batch, int hidden, const float* pre, const float* U, int ldu, const float* h0, float* hs, float* scratch,
                         int* status, int cus);
// lstm_persistent.hip: 1 when a persistent kernel's grid barrier gave up since the last call (and clears that)
int persistent_status_take();

}  // namespace dali_hip

#endif
