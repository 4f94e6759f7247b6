/*
 * dali_hip.h — C ABI of the MI355X (gfx950) execution backend for Dali's
 * JIT-fused array expressions.
 *
 * Every entry point returns 0 on success and a non-zero status on failure; the
 * message for the calling thread's last failure is dali_hip_last_error(). The
 * library never calls exit() and never frees caller memory. All device work is
 * issued on ONE non-blocking HIP stream owned by the library, so launches are
 * ordered among themselves; host-visible copies synchronise that stream.
 *
 * Each declaration cites the interface of the reference (bzcheeseman/Dali,
 * paths relative to its repository root) that it replaces.
 */
#ifndef DALI_HIP_H
#define DALI_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DALI_HIP_OK 0
#define DALI_HIP_ERROR 1

/* scalar / element types; numbering follows dali/array/dtype.h:6-10 */
#define DALI_HIP_FLOAT 0
#define DALI_HIP_DOUBLE 1
#define DALI_HIP_INT32 2

/* ---------------------------------------------------------------- errors */

/* Message of the last failed call on this thread ("" when none). Replaces the
 * ASSERT2 -> std::runtime_error text of dali/utils/assert2.h:12 and the
 * exit(EXIT_FAILURE) paths of dali/utils/compiler.h:81-88. */
const char* dali_hip_last_error(void);

/* ------------------------------------------------ device and placement */

/* Number of HIP devices. Replaces memory::Device::num_gpus,
 * dali/array/memory/device.cu.cpp:89-129. */
int dali_hip_device_count(int* count);

/* Select the device all later calls act on and create the library stream for
 * it. Replaces Device::set_cuda_device, dali/array/memory/device.cu.cpp:89-129. */
int dali_hip_init(int device);

/* Device marketing name and gcn arch string. Replaces Device::gpu_name,
 * dali/array/memory/device.cu.cpp:89-129. */
int dali_hip_device_name(int device, char* name, size_t name_len, char* arch, size_t arch_len);

/* Free and total device memory in bytes. Replaces memory::cuda_available_memory,
 * dali/array/memory/memory_ops.cu.cpp:134-138. */
int dali_hip_mem_info(size_t* free_bytes, size_t* total_bytes);

/* Block until everything issued on the library stream has finished. The
 * reference relies on NULL-stream ordering plus blocking cudaMemcpy
 * (dali/array/jit/jit.cpp:752, dali/array/memory/memory_ops.cu.cpp:109-126). */
int dali_hip_sync(void);

/* The library stream as an opaque hipStream_t, for callers that record their own events. */
void* dali_hip_stream(void);

/* -------------------------------------------------------------- memory */

/* Raw allocation / release. Replace memory::allocate and memory::free,
 * dali/array/memory/memory_ops.cu.cpp:58-95 (cudaMallocPitch / cudaFree);
 * byte counts are size_t instead of the reference's int. */
int dali_hip_malloc(void** ptr, size_t bytes);
int dali_hip_free(void* ptr);

/* Free-list reuse of device blocks. Replace memory::bank::allocate, deposit and clear,
 * dali/array/memory/memory_bank.cpp:40-81: a deposited block is handed to the next request of its size.
 * Here sizes are rounded up to classes (four per power of two, at most 25% slack) so that nearly equal
 * requests share blocks, and blocks of up to 2 MiB are carved out of 64 MiB slabs instead of costing a driver
 * allocation each. dali_hip_bank_clear returns the parked driver allocations; slab blocks stay parked.
 * Same-stream ordering makes immediate reuse safe. */
/* (dali_hip_malloc, dali_hip_bank_allocate and dali_hip_memset_async fail while the library stream is being captured) */
int dali_hip_bank_allocate(void** ptr, size_t bytes);
int dali_hip_bank_deposit(void* ptr, size_t bytes);
int dali_hip_bank_clear(void);
/* bytes currently parked in the bank / handed out by it and not yet deposited */
int dali_hip_bank_stats(size_t* parked_bytes, size_t* live_bytes);

/* Zero-fill on the library stream. Replaces memory::clear,
 * dali/array/memory/memory_ops.cu.cpp:97-107 (cudaMemset). */
int dali_hip_memset_async(void* ptr, int value, size_t bytes);

/* Copies. Replace memory::copy, dali/array/memory/memory_ops.cu.cpp:109-126
 * (blocking cudaMemcpy). h2d and d2h return after the data has arrived (they
 * synchronise the library stream); d2d is asynchronous on the library stream. */
int dali_hip_memcpy_h2d(void* dst_device, const void* src_host, size_t bytes);
int dali_hip_memcpy_d2h(void* dst_host, const void* src_device, size_t bytes);
int dali_hip_memcpy_d2d(void* dst_device, const void* src_device, size_t bytes);

/* Pinned host memory and migrations that do not block the caller: the alternative to the blocking cudaMemcpy of
 * memory::copy (dali/array/memory/memory_ops.cu.cpp:109-126) for a caller whose host side lives in memory from
 * dali_hip_host_alloc. The copy runs on a second stream of the library. It starts after everything already issued
 * on the compute stream (so kernels that still use the device block are not overtaken) and records `done_event`
 * (from dali_hip_event_create, may be NULL) when the bytes have arrived. Work issued afterwards on the compute
 * stream does not wait for the copy unless dali_hip_stream_wait_event(done_event) is called; the host waits with
 * dali_hip_event_synchronize or polls with dali_hip_event_query. The host block must stay untouched (h2d) or
 * unread (d2h) until the event has fired. Not allowed during a capture. */
int dali_hip_host_alloc(void** ptr, size_t bytes);
int dali_hip_host_free(void* ptr);
int dali_hip_memcpy_h2d_async(void* dst_device, const void* src_pinned, size_t bytes, void* done_event);
int dali_hip_memcpy_d2h_async(void* dst_pinned, const void* src_device, size_t bytes, void* done_event);

/* ------------------------------------------- runtime-compiled kernels */

/* How the launcher turns the six argument arrays into a grid. */
#define DALI_HIP_GRID_ELEMS 0  /* 1-D: blocks over prod(iv[work_begin..+work_count)) / work_per_block */
#define DALI_HIP_GRID_ROWS 1   /* 1-D: one block per work_per_block rows; rows = prod(iv[work_begin..+work_count)) */
#define DALI_HIP_GRID_COLS 2   /* 2-D: x over kept columns, y splits the reduced rows; partials in the workspace */
#define DALI_HIP_GRID_ALL 3    /* 1-D: bounded grid, one partial per block in the workspace */

/*
 * Launch plan of one generated kernel. The generated kernel has the signature
 *     extern "C" __global__ void <kernel_name>(KArgs args)
 * where KArgs is laid out by the launcher as
 *     void*  ws;                   library workspace (partials and counters)
 *     void*  p[n_arrays];          array_data[i] + offsets[i] * array_elsize[i]
 *     slot   s[max(1,n_scalars)];  8-byte slots holding *scalar_arguments[j]
 *     int    iv[...];              per array: sizes[i][0..nd) then, if the array is
 *                                  declared strided, strides[i][0..nd); then per
 *                                  shape k: shapes[k][0..shape_ndim[k])
 * with nd = array_ndim[i]. The grid is computed from iv by grid_kind.
 */
typedef struct dali_hip_launch_plan {
    int32_t n_arrays;
    int32_t n_scalars;
    int32_t n_shapes;
    const int32_t* array_ndim;    /* [n_arrays] max(1, ndim) of each buffer (dali/array/jit/jit.cpp:281-285) */
    const int32_t* array_strided; /* [n_arrays] 1 when strides[i] is valid (dali/array/jit/jit.cpp:216-232) */
    const int32_t* array_elsize;  /* [n_arrays] bytes per element */
    const int32_t* scalar_dtype;  /* [n_scalars] DALI_HIP_FLOAT / DOUBLE / INT32 (dali/array/jit/scalar_view.cpp:39-66) */
    const int32_t* shape_ndim;    /* [n_shapes] ints read from shapes[k] */
    int32_t block_threads;        /* workgroup size */
    int32_t grid_kind;            /* DALI_HIP_GRID_* */
    int32_t work_begin;           /* first iv index of the extent product (x dimension) */
    int32_t work_count;           /* number of iv entries multiplied (0 => 1) */
    int32_t work_per_block;       /* elements / rows / columns covered by one block in x */
    int32_t max_blocks;           /* upper bound of grid.x (0 => unbounded); GRID_COLS: of grid.x * grid.y, met by shrinking grid.y */
    int32_t work2_begin;          /* GRID_COLS: iv index of the reduced extent */
    int32_t work2_per_block;      /* GRID_COLS: reduced rows per y-block */
    int32_t max_blocks2;          /* GRID_COLS: upper bound of grid.y */
    int32_t ws_elsize;            /* GRID_COLS / GRID_ALL: bytes of one partial result (0 = no workspace) */
} dali_hip_launch_plan;

/*
 * Make the kernel for `hash` launchable: in-process map, else the on-disk code
 * object cache (<cache>/<hash>.hsaco), else hipRTC for gfx950. `*was_cached`
 * (may be NULL) receives 2 for an in-process hit, 1 for a disk hit, 0 after a
 * compile. Replaces Compiler::load / Compiler::compile / dlopen / dlsym("maker"),
 * dali/utils/compiler.h:91-173 and dali/utils/compiler.cpp:36-49,86-103,123-227.
 * The cache directory is $DALI_HIP_CACHE_DIR, else ~/.dali/cache_hip
 * (dali/utils/compiler.cpp:234-238); DALI_JIT_ALWAYS_RECOMPILE=true forces one
 * rebuild per hash per process (dali/array/jit/jit.cpp:27-47,1023-1024).
 */
int dali_hip_module_load(uint64_t hash, const char* hip_source, const char* kernel_name,
                         const dali_hip_launch_plan* plan, int* was_cached);

/* 1 when `hash` is already loaded in this process, else 0 (no compile, no disk access). */
int dali_hip_module_is_loaded(uint64_t hash);

/*
 * Launch the kernel of `hash` with the reference's six argument arrays, same
 * order and meaning as `maker(void** array_data, const int* offsets, const int**
 * sizes, const int** strides, const void** scalar_arguments, const int** shapes)`
 * (dali/utils/compiler.cpp:190-197, called from dali/array/jit/jit.cpp:1216-1223):
 * array_data[i] are device pointers, offsets in elements, scalars are host
 * pointers read at call time.
 */
int dali_hip_launch(uint64_t hash, void** array_data, const int* offsets, const int** sizes,
                    const int** strides, const void** scalar_arguments, const int** shapes);

/* Compile only (no device needed): hipRTC `hip_source` for gfx950 and return the
 * code object size; used to check generated source on machines without a GPU. */
int dali_hip_compile_only(const char* hip_source, size_t* code_size);

/* The hipRTC options (besides the target) every generated kernel is compiled with, space-separated: part of what a
 * caller must fold into `hash` so that code objects built under other options are not taken from the disk cache. */
const char* dali_hip_rtc_options(void);

/* Counters: modules compiled by hipRTC, loaded from disk, and launches so far. */
int dali_hip_jit_stats(uint64_t* compiled, uint64_t* disk_hits, uint64_t* launches);

/* Set the code-object cache directory (overrides the environment). Replaces
 * Compiler::set_output_path, dali/utils/compiler.cpp:115-117. */
int dali_hip_set_cache_dir(const char* path);
/* Load every code object of the cache directory into the device ahead of its first use (the counterpart of
 * shipping ~/.dali/cache/<hash>.so files and having dlopen done before the first request,
 * dali/utils/compiler.cpp:86-103): dali_hip_module_load then only attaches the launch plan. Files that do not
 * load are skipped and rebuilt from source when their expression is first evaluated. `loaded` (may be NULL)
 * receives the number of code objects taken in by this call. */
int dali_hip_cache_warm(int* loaded);

/* ---------------------------------------------------------------- GEMM */

/*
 * fp32 GEMM on the matrix cores, column-major convention of the call it
 * replaces: cublasSgemm(handle, transB, transA, m, n, k, &alpha, B, ldb, A, lda,
 * &beta, C, ldc) in dali/array/gemm/cublas_gemm.cu:153-166 (and cblas_sgemm in
 * dali/array/gemm/cpu_gemm.cpp:59-68): C(m x n, column-major, ldc) =
 * alpha * op(B)(m x k) * op(A)(k x n) + beta * C, i.e. in row-major terms
 * C[n, m] = alpha * A[n, k] * B[k, m] + beta * C. trans flags: 0 = no transpose,
 * 1 = transpose. With n <= 64 (a few rows of A against a wide B, transA = 0, k a multiple of 4) B is streamed once,
 * straight from memory into the matrix instruction, instead of being tiled through LDS; the sums are then formed in
 * another order than the tiled kernels form them (DALI_HIP_GEMM_SKINNY=0 switches this off). With k <= 64 against a
 * large C (transB = 0) the rows of A stay in registers and C is written once (DALI_HIP_GEMM_SMALLK=0 switches that off).
 */
int dali_hip_sgemm(int transB, int transA, int m, int n, int k, float alpha, const float* B, int ldb,
                   const float* A, int lda, float beta, float* C, int ldc);

/*
 * fp64 GEMM on the matrix cores, same conventions as dali_hip_sgemm: replaces
 * cublasDgemm(handle, transB, transA, m, n, k, &alpha, B, ldb, A, lda, &beta, C, ldc)
 * in dali/array/gemm/cublas_gemm.cu:167-178 (and cblas_dgemm in
 * dali/array/gemm/cpu_gemm.cpp). Any leading dimensions and alignments; k == 0
 * scales C by beta.
 */
int dali_hip_dgemm(int transB, int transA, int m, int n, int k, double alpha, const double* B, int ldb,
                   const double* A, int lda, double beta, double* C, int ldc);

/*
 * Two products accumulated into one destination in a single launch:
 * C = alpha * (op(B1) * op(A1) + op(B2) * op(A2)) + beta * C with the same
 * conventions as dali_hip_sgemm (k1 and k2 are the two inner extents). This is
 * the shape `dst = X.W; dst += H.U` of StackedInputLayer::activate,
 * dali/layers/layers.cpp:159-161 via dali/tensor/op/composite.cpp:18-53.
 */
int dali_hip_sgemm_pair(int transB1, int transA1, int transB2, int transA2, int m, int n, int k1, int k2,
                        float alpha, const float* B1, int ldb1, const float* A1, int lda1, const float* B2,
                        int ldb2, const float* A2, int lda2, float beta, float* C, int ldc);

/* Row-major sum of up to 8 products into one accumulator: C[M, N] = alpha * sum_t op(A_t) . op(B_t) + beta * C, all A_t with
 * the leading dimension lda and all B_t with ldb (transA: A_t stored [K_t][M]; transB: B_t stored [N][K_t]). Without
 * transA the rows of A_t may overlap (lda < K_t). That is a stride-1 convolution without a patch matrix: over a
 * zero-padded channels-last image X[N, Hp, Wp, C], filter row kh is the term A = X + kh * Wp * C, lda = C, K = filter_w * C
 * against rows [kh * filter_w * C, ...) of the filter matrix, evaluated at every padded position (M = N * Hp * Wp); the image
 * needs (filter_h - 1) * Wp + filter_w pixels of readable slack behind it. row_map (NULL, or {Hp, Wp, out_h, out_w}) keeps
 * only the positions i < out_h, j < out_w of each [Hp, Wp] grid and stores them densely, as rows (n * out_h + i) * out_w + j.
 * Replaces im2col + op::dot in op::conv2d (dali/array/op/conv.cpp:253-272) for the NHWC, stride-1 case. */
int dali_hip_sgemm_terms(int nterms, int transA, int transB, int M, int N, const int* K, const float* const* A, int lda,
                         const float* const* B, int ldb, float alpha, float beta, float* C, int ldc, const int* row_map);

/*
 * One LSTM cell step in a single launch: pre = X[batch, input] . W[input, 4 hidden] + Hprev[batch, hidden] .
 * U[hidden, 4 hidden] (row-major, gates packed i, f, o, g along the columns), then per element
 * i, f, o = sigmoid(pre + bias), g = tanh(pre + bias), Cout = f * Cprev + i * g, Hout = o * tanh(Cout)
 * (dali/layers/lstm.cpp:226-261 with StackedInputLayer::activate, dali/layers/layers.cpp:159-161). The MFMA tile of
 * a workgroup gathers the four gate columns of sixteen hidden units, so the pre-activations never leave the chip;
 * every operation is rounded as in the two-launch form (dali_hip_sgemm_pair followed by the generated gate
 * kernel). Needs input and hidden to be multiples of 64 and 16-byte aligned operands whose leading dimensions are
 * multiples of 4 (X and Hprev, W and U may differ in theirs: the input size need not equal the hidden size);
 * otherwise it fails and the caller uses the two-launch form. Cprev, Cout, Hout are dense [batch, hidden].
 */
int dali_hip_lstm_step(int batch, int input, int hidden, const float* X, int ldx, const float* Hprev, int ldh,
                       const float* Cprev, const float* W, int ldw, const float* U, int ldu, const float* bias,
                       float* Cout, float* Hout);

/*
 * The same step for batches of up to 64 rows (a decoder that feeds each output back through the host): 16-row tiles on
 * the matrix cores and about one workgroup per compute unit, each streaming its own 64 columns of one gate of W and U over
 * a share of the inner extent (whole cache lines, 16-byte loads straight into the matrix operand), instead of the 64-row
 * tiles of dali_hip_lstm_step, whose time does not fall with the batch. Same arguments and gate arithmetic
 * (dali/layers/lstm.cpp:226-261); the products are summed in another order, so results agree with dali_hip_lstm_step to
 * rounding, not bit for bit. hidden must be 256, 512, 768 or 1024, input a multiple of 16 with input + hidden a multiple of
 * 64; all matrices 16-byte aligned with leading dimensions that are multiples of 4. Partial sums and tickets live in
 * the library workspace.
 */
int dali_hip_lstm_step_small(int batch, int input, int hidden, const float* X, int ldx, const float* Hprev, int ldh,
                             const float* Cprev, const float* W, int ldw, const float* U, int ldu, const float* bias,
                             float* Cout, float* Hout);

/*
 * The recurrent half of an LSTM over a whole sequence in one launch, for batches of at most 128 rows: the loop of
 * dali/layers/lstm.cpp:294-303 (one cell activation per time step), whose hidden-to-hidden product the reference meant to
 * hand to a persistent kernel (third_party/nervana_kernels/sass/persistent_rnn_fprop.sass). pre [steps, batch, 4 hidden]
 * holds the input half of the pre-activations for every step, x(t).W + bias, gates packed i, f, o, g along the columns (one
 * large product computed beforehand); U [hidden, 4 hidden] (row stride ldu >= 4 hidden) stays on the chip for the whole
 * sequence, every workgroup holding the gate columns of its hidden units; per step a workgroup forms h(t-1).U for those
 * columns, finishes the cell (same arithmetic as dali_hip_lstm_step) and meets the others at a grid barrier.
 * hs [steps, batch, hidden] receives every hidden state, c_out [batch, hidden] the last cell state.
 * Accepted sizes: hidden a multiple of 64 up to 2048 and at most 128 rows (dali_hip_lstm_recurrent_persistent_supported
 * answers for the bound device; anything else is refused with an error). Up to 64 rows with hidden = 256, 512, 768 or 1024
 * the weights sit in LDS (up to 32 rows a step waits for the values of h(t-1) themselves: hs is first filled with a "not
 * written yet" bit pattern); otherwise the weights sit in registers and the batch is cut into row blocks that take turns,
 * so that one block's barrier runs while the others are multiplied. h0 and hs must be 16-byte aligned. hs must not overlap h0, c0
 * or pre (a call where it does is refused) and must not be read by anybody else while the launch runs.
 * The grid has at most one workgroup per compute unit, so all are resident; a workgroup that still does not see the others
 * arrive within 2^20 polls (DALI_HIP_PERSISTENT_SPIN_LIMIT) raises a flag, every workgroup leaves, and the next
 * dali_hip_sync or dali_hip_memcpy_d2h fails with that message instead of the device hanging. Until that error has been
 * collected, further persistent launches are refused (they would leave at their first wait).
 */
int dali_hip_lstm_recurrent_persistent(int steps, int batch, int hidden, const float* pre, const float* U, int ldu, const float* h0,
                                       const float* c0, float* hs, float* c_out);
/* Whether dali_hip_lstm_recurrent_persistent serves this batch and hidden size on the bound device: 0 no (the call would be refused), 1 yes,
 * 2 yes and it is expected to beat one launch of dali_hip_lstm_step per step (up to 32 rows; up to 48 from 1024 hidden units on). No error is set. */
int dali_hip_lstm_recurrent_persistent_supported(int batch, int hidden);

/*
 * The recurrent half of a GRU over a whole sequence in one launch: the loop of dali/layers/gru.cpp:59-64 over
 * GRU::activate (gru.cpp:27-44). pre [steps, batch, 3 hidden] holds x(t).W + bias for the reset, update and candidate
 * layers (packed in that order along the columns, one product computed beforehand), U [hidden, 3 hidden] (row stride ldu)
 * the recurrent weights in the same packing. Per step every workgroup forms (r, z) = sigmoid(pre + h(t-1).U) for its hidden
 * units, writes r * h(t-1) into scratch [steps, batch, hidden], meets the others at a grid barrier, forms the candidate
 * tanh(pre + (r * h(t-1)).U) and h(t) = h(t-1) * (1 - z) + candidate * z, and meets them again; hs [steps, batch, hidden]
 * receives every state. Same sizes, row blocks that take turns at the barriers, bounded waits and error reporting as
 * dali_hip_lstm_recurrent_persistent (weights in registers). h0, hs and scratch 16-byte aligned; hs and scratch must not
 * overlap each other or an input, and must not be touched by anybody else while the launch runs.
 */
int dali_hip_gru_recurrent_persistent(int steps, int batch, int hidden, const float* pre, const float* U, int ldu, const float* h0, float* hs,
                                      float* scratch);
/* 0: not served; 1: served; 2: served and expected to beat the launch-per-step form */
int dali_hip_gru_recurrent_persistent_supported(int batch, int hidden);

/* ------------------------------------------------------------- softmax along an inner axis */
/*
 * out = softmax(x) along the middle axis of a contiguous fp32 array seen as [outer, extent, inner]
 * (reference: op::softmax(logits, axis), dali/array/op/softmax.cpp:5-8, for an axis other than the last; outer = 1 is the
 * leading axis of a matrix). One pass over memory: a workgroup keeps a strip of the reduced axis in registers. inner must be
 * a multiple of 4 and at least 16, extent at most 2048 (at most 512 for the widest strips), both arrays 16-byte aligned;
 * x and out may be the same array. dali_hip_softmax_axis_supported returns 1 for the sizes the kernel takes (the generated
 * three-pass form serves the others).
 */
int dali_hip_softmax_axis(const float* x, float* out, long long outer, int extent, long long inner);
int dali_hip_softmax_axis_supported(long long outer, int extent, long long inner);

/* ------------------------------------------------------------- scatter */
/*
 * Stable ordering of n int32 keys held in device memory: sorted_keys[p] is the p-th smallest key and
 * perm[p] its position in `keys`; equal keys keep their input order. key_limit > 0 promises that every
 * key lies in [0, key_limit) (fewer bits to sort); pass 0 for arbitrary keys. Runs on the library stream.
 * It serves assignment through a gather (`dest[indices] += values`, dali/array/op/gather.cpp:89-97,
 * 126-143): the reference's GPU code adds duplicates with atomicAdd in arrival order (gather.cpp:14-28);
 * the generated scatter kernel instead walks each destination row's contributions in input order,
 * the order of the reference's sequential CPU loop, so the result does not depend on scheduling.
 * Up to 16384 keys are ordered by one kernel that allocates nothing (it may be captured); longer inputs take a
 * least-significant-digit radix sort (eight bits per pass; histogram, per-digit scan and ranked move per pass) whose temporary block comes from
 * the bank, so they fail during a capture. With key_limit > 0, keys outside the promised range come out behind
 * every key inside it (among themselves in an unspecified but stable order) and never between two equal valid
 * keys; perm is a permutation for any input. keys, sorted_keys and perm must not overlap (the outputs are written
 * while the keys are still being read): a call with overlapping arrays is refused.
 */
int dali_hip_argsort_i32(const int32_t* keys, int64_t n, int32_t key_limit, int32_t* sorted_keys, int32_t* perm);

/*
 * dali_hip_argsort_i32 for callers that cannot allocate: code under HIP graph capture, tight serving loops and
 * harnesses that forbid hipMalloc. It has no counterpart in the reference. Same arguments and same result as
 * dali_hip_argsort_i32, for at most 16384 keys (more is an error, nothing is launched). The tickets and counts of the
 * ordering kernel live in a 2 MiB + 256 B device array that is part of the library's code object (each device that the
 * library runs on holds it until the process ends); the call allocates and frees nothing, neither from the driver nor
 * from the bank. dali_hip_init must have been called before (it allocates; this call does not initialise). All calls
 * on a device share that array: calls that overlap on one device (from two threads, or on streams other than the
 * library stream) race; calls issued one after the other are ordered by the library stream.
 */
int dali_hip_argsort_i32_noalloc(const int32_t* keys, int64_t n, int32_t key_limit, int32_t* sorted_keys, int32_t* perm);

/*
 * The column numbers of the k best entries of every row of a dense row-major [rows, cols] matrix, best first, into
 * out[rows, k]. Replaces the reference's CPU-only CpuTopKImpl (dali/array/op/top_k.cpp:36-196; "add gpu impl of topk"
 * is a TODO there, :198). dtype: 0 = float, 1 = double, 2 = int32. largest != 0 orders by descending value (top_k),
 * else ascending (bottom_k, argsort). Equal values come out in ascending column order, or in descending column order
 * with ties_by_descending_column != 0 (what the reference's heap gives bottom_k for k < cols, top_k.cpp:118-123).
 * -0.0 and +0.0 are equal; the place of NaNs is unspecified. Rows of at least 1024 entries with k <= 64 take a one-pass
 * selection kernel that allocates nothing; everything else stable radix passes over the whole matrix (by key, then by
 * row) on the library stream whose buffers (four times the input) come from the bank, so that form fails during a capture.
 */
int dali_hip_topk_rows(const void* x, int dtype, int64_t rows, int32_t cols, int32_t k, int largest, int ties_by_descending_column,
                       int32_t* out);

/* ---------------------------------------------------------- HIP graphs */

/*
 * Capture the launches issued on the library stream between begin and end into
 * a HIP graph and replay it with one call; for launch-bound steady-state loops
 * (the reference has no counterpart: it launches every kernel eagerly from
 * dali/array/jit/jit.cpp:1216-1223). Only kernel launches and device-to-device
 * copies may be issued while capturing: allocation, host copies and
 * dali_hip_sync are errors until dali_hip_capture_end.
 */
int dali_hip_capture_begin(void);
int dali_hip_capture_end(void** graph_exec);
int dali_hip_graph_launch(void* graph_exec);
int dali_hip_graph_destroy(void* graph_exec);

/* --------------------------------------------------------------- timing */

/* hipEvent wrappers bound to the library stream (the reference times host-side
 * only, dali/utils/performance_report.cpp:22-149). */
int dali_hip_event_create(void** event);
int dali_hip_event_record(void* event);
int dali_hip_event_elapsed_ms(void* start, void* stop, float* ms); /* waits for `stop` */
int dali_hip_event_destroy(void* event);
/* the compute stream waits (on the device) for an event recorded by an asynchronous copy or by dali_hip_event_record */
int dali_hip_stream_wait_event(void* event);
/* the host waits for / polls an event */
int dali_hip_event_synchronize(void* event);
int dali_hip_event_query(void* event, int* done);

#ifdef __cplusplus
}
#endif
#endif /* DALI_HIP_H */
