// fp32 matrix-vector product: y[M] = alpha * A[M, K] . x[K] + beta * y, A row-major
// (op::dot of a matrix with a column, dali/array/op/dot.cpp:49-67 with b.shape[1] == 1; the reference hands it to the
// same sgemm call as every other product, dali/array/gemm/cublas_gemm.cu:153-166 with m == 1).
//
// The tiled product kernels compute a 64-column tile for the one column that exists and read A through LDS for a single
// use ([4096,4096] . [4096]: 40 us, 0.2 of the memory peak). Here A is streamed once: a row belongs to one wave (many
// rows) or to the four waves of a workgroup (few rows), a lane takes 16-byte pieces of the row, 64 pieces apart, multiplies
// them with the matching piece of x (16 KiB for K = 4096: it stays in the caches) and the lanes' sums meet through
// cross-lane shuffles, the waves' through LDS. Rows need no alignment beyond their elements: global memory takes 16-byte
// accesses at any 4-byte address; the K % 4 elements behind a row's last piece go one to a lane.
#include <cstdint>

#include "runtime.h"

namespace dali_hip {
namespace {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef f4 f4u __attribute__((aligned(4)));

struct GemvArgs {
    int M, K;
    const float* A;
    long lda;
    const float* x;
    long incx;
    float* y;
    long incy;
    float alpha, beta;
};

// WPR: waves per row (1 or 4); UNIT: x has unit stride
template <int WPR, bool UNIT>
__global__ __launch_bounds__(256) void sgemv_rows_kernel(GemvArgs a) {
    __shared__ float part[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const long row = WPR == 1 ? (long)blockIdx.x * 4 + wave : (long)blockIdx.x;
    const bool row_ok = row < a.M;  // (WPR == 4: always)
    const float* ar = a.A + (row_ok ? row : 0) * a.lda;
    const int pieces = a.K / 4;
    const int first = WPR == 1 ? lane : tid, step = WPR == 1 ? 64 : 256;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    int p = first;
    // four pieces of the row in flight per lane
    for (; p + 3 * step < pieces; p += 4 * step) {
        f4 av[4], xv[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const long k = 4L * (p + u * step);
            av[u] = __builtin_nontemporal_load(reinterpret_cast<const f4u*>(ar + k));
            if (UNIT) {
                xv[u] = *reinterpret_cast<const f4u*>(a.x + k);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) xv[u][j] = a.x[(k + j) * a.incx];
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            s0 = __builtin_fmaf(av[u][0], xv[u][0], s0);
            s1 = __builtin_fmaf(av[u][1], xv[u][1], s1);
            s2 = __builtin_fmaf(av[u][2], xv[u][2], s2);
            s3 = __builtin_fmaf(av[u][3], xv[u][3], s3);
        }
    }
    for (; p < pieces; p += step) {
        const long k = 4L * p;
        const f4 av = *reinterpret_cast<const f4u*>(ar + k);
        f4 xv;
        if (UNIT) {
            xv = *reinterpret_cast<const f4u*>(a.x + k);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) xv[j] = a.x[(k + j) * a.incx];
        }
        s0 = __builtin_fmaf(av[0], xv[0], s0);
        s1 = __builtin_fmaf(av[1], xv[1], s1);
        s2 = __builtin_fmaf(av[2], xv[2], s2);
        s3 = __builtin_fmaf(av[3], xv[3], s3);
    }
    // the K % 4 elements behind the last piece
    const int rest = a.K - 4 * pieces;
    if (first < rest) {
        const long k = 4L * pieces + first;
        s0 = __builtin_fmaf(ar[k], a.x[k * a.incx], s0);
    }
    float s = (s0 + s1) + (s2 + s3);
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) s += __shfl_xor(s, d, 64);
    if (WPR == 4) {
        if (lane == 0) part[wave] = s;
        __syncthreads();
        s = (part[0] + part[1]) + (part[2] + part[3]);
        if (tid != 0) return;
    } else if (lane != 0 || !row_ok) {
        return;
    }
    float* out = a.y + row * a.incy;
    // (beta == 0: y is not read, whatever it holds, as in the product kernels)
    *out = a.beta == 0.0f ? a.alpha * s : __builtin_fmaf(a.alpha, s, a.beta * *out);
}

}  // namespace

// 1 = launched, 0 = not this kernel's case, -1 = error (message set)
int sgemv_rows(int M, int K, float alpha, const float* A, int lda, const float* x, int incx, float beta, float* y, int incy) {
    if (M < 1 || K < 1 || lda < K || incx < 1 || incy < 1) return 0;
    GemvArgs a;
    a.M = M;
    a.K = K;
    a.A = A;
    a.lda = lda;
    a.x = x;
    a.incx = incx;
    a.y = y;
    a.incy = incy;
    a.alpha = alpha;
    a.beta = beta;
    // few rows: a workgroup per row, so that the rows still spread over the device
    const bool wide = M < 2048;
    const dim3 grid((unsigned)(wide ? M : (M + 3) / 4));
    if (wide) {
        if (incx == 1)
            hipLaunchKernelGGL((sgemv_rows_kernel<4, true>), grid, dim3(256), 0, stream(), a);
        else
            hipLaunchKernelGGL((sgemv_rows_kernel<4, false>), grid, dim3(256), 0, stream(), a);
    } else {
        if (incx == 1)
            hipLaunchKernelGGL((sgemv_rows_kernel<1, true>), grid, dim3(256), 0, stream(), a);
        else
            hipLaunchKernelGGL((sgemv_rows_kernel<1, false>), grid, dim3(256), 0, stream(), a);
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        fail("sgemv launch failed: %s", hipGetErrorString(e));
        return -1;
    }
    return 1;
}

}  // namespace dali_hip
