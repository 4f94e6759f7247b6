// fp32 GEMM on the CDNA4 matrix cores (v_mfma_f32_32x32x2_f32), LDS-staged and
// software-pipelined, for dali_hip_sgemm / dali_hip_sgemm_pair.
//
// Row-major view used inside this file: C[M,N] = alpha * sum_s A_s[M,K_s] * B_s[K_s,N] + beta * C
// for one or two (A_s, B_s) segments. The column-major entry points map onto it
// by swapping the operands (C^T = B^T A^T), exactly as the reference does when it
// calls a column-major BLAS (dali/array/gemm/cpu_gemm.cpp:43-68).
//
// Work decomposition: a 256-thread workgroup (4 waves, 2x2) owns a BM x BN tile
// of C; each wave owns (BM/2) x (BN/2), built from 32x32 MFMA accumulators.
// Operand tiles are staged as As[k][m] and Bs[k][n] so that the MFMA operand
// fetch (lane l reads element l%32 of row k + l/32) is a conflict-free 32-float
// row read. The next K-slab is fetched from global memory into registers while
// the current one is consumed from LDS (two LDS buffers, one barrier per slab).
#include "runtime.h"

#include <cstring>

namespace dali_hip {

typedef float floatx16 __attribute__((ext_vector_type(16)));

struct GemmSeg {
    const float* A;
    const float* B;
    int lda, ldb, K;
};

struct GemmArgs {
    GemmSeg seg[2];
    int nseg;
    int M, N;
    float* C;
    int ldc;
    float alpha, beta;
};

constexpr int BK = 16;

template <int BM, int BN, bool TA, bool TB, bool VEC>
__global__ __launch_bounds__(256) void sgemm_kernel(GemmArgs g) {
    constexpr int PAD = 4;
    constexpr int WTM = BM / 2, WTN = BN / 2;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int A_F4 = BM * BK / 4 / 256;  // float4 fetches per thread for the A slab
    constexpr int B_F4 = BN * BK / 4 / 256;
    static_assert(A_F4 >= 1 && B_F4 >= 1, "tile too small for 256 threads");

    __shared__ float As[2][BK][BM + PAD];
    __shared__ float Bs[2][BK][BN + PAD];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, h = lane >> 5;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int M = g.M, N = g.N;

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    float4 ra[A_F4], rb[B_F4];

    // fetch one BK-deep slab of segment s starting at k0 into registers
    auto fetch = [&](const GemmSeg& s, int k0) {
#pragma unroll
        for (int t = 0; t < A_F4; ++t) {
            int idx = tid + t * 256;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (!TA) {
                // A[m][k], k contiguous: 4 consecutive k of one row
                int m = m0 + idx / (BK / 4), k = k0 + (idx % (BK / 4)) * 4;
                if (m < M) {
                    const float* p = s.A + (size_t)m * s.lda + k;
                    if (VEC && k + 3 < s.K) {
                        v = *(const float4*)p;
                    } else {
                        if (k + 0 < s.K) v.x = p[0];
                        if (k + 1 < s.K) v.y = p[1];
                        if (k + 2 < s.K) v.z = p[2];
                        if (k + 3 < s.K) v.w = p[3];
                    }
                }
            } else {
                // A stored as [K][M], m contiguous: 4 consecutive m of one k
                int k = k0 + idx / (BM / 4), m = m0 + (idx % (BM / 4)) * 4;
                if (k < s.K) {
                    const float* p = s.A + (size_t)k * s.lda + m;
                    if (VEC && m + 3 < M) {
                        v = *(const float4*)p;
                    } else {
                        if (m + 0 < M) v.x = p[0];
                        if (m + 1 < M) v.y = p[1];
                        if (m + 2 < M) v.z = p[2];
                        if (m + 3 < M) v.w = p[3];
                    }
                }
            }
            ra[t] = v;
        }
#pragma unroll
        for (int t = 0; t < B_F4; ++t) {
            int idx = tid + t * 256;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (!TB) {
                // B[k][n], n contiguous
                int k = k0 + idx / (BN / 4), n = n0 + (idx % (BN / 4)) * 4;
                if (k < s.K) {
                    const float* p = s.B + (size_t)k * s.ldb + n;
                    if (VEC && n + 3 < N) {
                        v = *(const float4*)p;
                    } else {
                        if (n + 0 < N) v.x = p[0];
                        if (n + 1 < N) v.y = p[1];
                        if (n + 2 < N) v.z = p[2];
                        if (n + 3 < N) v.w = p[3];
                    }
                }
            } else {
                // B stored as [N][K], k contiguous
                int n = n0 + idx / (BK / 4), k = k0 + (idx % (BK / 4)) * 4;
                if (n < N) {
                    const float* p = s.B + (size_t)n * s.ldb + k;
                    if (VEC && k + 3 < s.K) {
                        v = *(const float4*)p;
                    } else {
                        if (k + 0 < s.K) v.x = p[0];
                        if (k + 1 < s.K) v.y = p[1];
                        if (k + 2 < s.K) v.z = p[2];
                        if (k + 3 < s.K) v.w = p[3];
                    }
                }
            }
            rb[t] = v;
        }
    };

    auto stage = [&](int buf) {
#pragma unroll
        for (int t = 0; t < A_F4; ++t) {
            int idx = tid + t * 256;
            if (!TA) {
                int m = idx / (BK / 4), k = (idx % (BK / 4)) * 4;
                As[buf][k + 0][m] = ra[t].x;
                As[buf][k + 1][m] = ra[t].y;
                As[buf][k + 2][m] = ra[t].z;
                As[buf][k + 3][m] = ra[t].w;
            } else {
                int k = idx / (BM / 4), m = (idx % (BM / 4)) * 4;
                *(float4*)&As[buf][k][m] = ra[t];
            }
        }
#pragma unroll
        for (int t = 0; t < B_F4; ++t) {
            int idx = tid + t * 256;
            if (!TB) {
                int k = idx / (BN / 4), n = (idx % (BN / 4)) * 4;
                *(float4*)&Bs[buf][k][n] = rb[t];
            } else {
                int n = idx / (BK / 4), k = (idx % (BK / 4)) * 4;
                Bs[buf][k + 0][n] = rb[t].x;
                Bs[buf][k + 1][n] = rb[t].y;
                Bs[buf][k + 2][n] = rb[t].z;
                Bs[buf][k + 3][n] = rb[t].w;
            }
        }
    };

    // flat list of slabs over the segments
    int slabs0 = (g.seg[0].K + BK - 1) / BK;
    int slabs1 = g.nseg > 1 ? (g.seg[1].K + BK - 1) / BK : 0;
    int nslab = slabs0 + slabs1;
    auto fetch_slab = [&](int i) {
        if (i < slabs0)
            fetch(g.seg[0], i * BK);
        else
            fetch(g.seg[1], (i - slabs0) * BK);
    };

    if (nslab > 0) {
        fetch_slab(0);
        stage(0);
    }
    __syncthreads();
    for (int i = 0; i < nslab; ++i) {
        int cur = i & 1;
        if (i + 1 < nslab) fetch_slab(i + 1);
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
            float a[TM], b[TN];
#pragma unroll
            for (int ii = 0; ii < TM; ++ii) a[ii] = As[cur][kk + h][wm * WTM + ii * 32 + l32];
#pragma unroll
            for (int jj = 0; jj < TN; ++jj) b[jj] = Bs[cur][kk + h][wn * WTN + jj * 32 + l32];
#pragma unroll
            for (int ii = 0; ii < TM; ++ii)
#pragma unroll
                for (int jj = 0; jj < TN; ++jj)
                    acc[ii][jj] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ii], b[jj], acc[ii][jj], 0, 0, 0);
        }
        if (i + 1 < nslab) stage(cur ^ 1);
        __syncthreads();
    }

    // epilogue: lane holds column l32 and rows 8*(v/4) + 4*h + v%4 of each 32x32 tile
    const float alpha = g.alpha, beta = g.beta;
#pragma unroll
    for (int ii = 0; ii < TM; ++ii)
#pragma unroll
        for (int jj = 0; jj < TN; ++jj) {
            int n = n0 + wn * WTN + jj * 32 + l32;
            if (n >= N) continue;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                int m = m0 + wm * WTM + ii * 32 + 8 * (v / 4) + 4 * h + (v % 4);
                if (m < M) {
                    float* c = g.C + (size_t)m * g.ldc + n;
                    float r = alpha * acc[ii][jj][v];
                    if (beta != 0.f) r += beta * *c;
                    *c = r;
                }
            }
        }
}

template <int BM, int BN>
static int launch_tile(const GemmArgs& g, bool ta, bool tb, bool vec) {
    dim3 grid((g.N + BN - 1) / BN, (g.M + BM - 1) / BM);
    dim3 block(256);
    hipStream_t st = stream();
#define DALI_GEMM_CASE(TA_, TB_, V_)                                                   \
    if (ta == TA_ && tb == TB_ && vec == V_) {                                         \
        hipLaunchKernelGGL((sgemm_kernel<BM, BN, TA_, TB_, V_>), grid, block, 0, st, g); \
    }
    DALI_GEMM_CASE(false, false, true)
    DALI_GEMM_CASE(false, false, false)
    DALI_GEMM_CASE(false, true, true)
    DALI_GEMM_CASE(false, true, false)
    DALI_GEMM_CASE(true, false, true)
    DALI_GEMM_CASE(true, false, false)
    DALI_GEMM_CASE(true, true, true)
    DALI_GEMM_CASE(true, true, false)
#undef DALI_GEMM_CASE
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("sgemm launch failed: %s", hipGetErrorString(e));
    return DALI_HIP_OK;
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// Row-major driver: C[M,N] = alpha * sum_s opA_s * opB_s + beta * C.
// ta: A_s is stored as [K][M]; tb: B_s is stored as [N][K].
static int sgemm_rowmajor(int nseg, bool ta, bool tb, int M, int N, const int* K, const float* const* A,
                          const int* lda, const float* const* B, const int* ldb, float alpha, float beta, float* C,
                          int ldc) {
    if (ensure_init()) return DALI_HIP_ERROR;
    if (M < 0 || N < 0) return fail("sgemm: negative extent (M=%d, N=%d)", M, N);
    if (M == 0 || N == 0) return DALI_HIP_OK;
    if (!C) return fail("sgemm: C is NULL");
    if (ldc < N) return fail("sgemm: ldc=%d smaller than row length %d", ldc, N);
    GemmArgs g = {};
    g.nseg = 0;
    bool vec = true;
    for (int s = 0; s < nseg; ++s) {
        if (K[s] < 0) return fail("sgemm: negative inner extent %d", K[s]);
        if (K[s] == 0) continue;
        if (!A[s] || !B[s]) return fail("sgemm: operand %d is NULL", s);
        int a_row = ta ? M : K[s], b_row = tb ? K[s] : N;
        if (lda[s] < a_row) return fail("sgemm: leading dimension %d of the left operand is smaller than its row length %d", lda[s], a_row);
        if (ldb[s] < b_row) return fail("sgemm: leading dimension %d of the right operand is smaller than its row length %d", ldb[s], b_row);
        GemmSeg& sg = g.seg[g.nseg++];
        sg.A = A[s];
        sg.B = B[s];
        sg.lda = lda[s];
        sg.ldb = ldb[s];
        sg.K = K[s];
        vec = vec && aligned16(A[s]) && aligned16(B[s]) && lda[s] % 4 == 0 && ldb[s] % 4 == 0;
    }
    g.M = M;
    g.N = N;
    g.C = C;
    g.ldc = ldc;
    g.alpha = alpha;
    g.beta = beta;
    if (g.nseg == 0) {
        // empty inner extent: C = beta * C
        g.nseg = 1;
        g.seg[0].K = 0;
        vec = false;
    }
    long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128);
    if (tiles128 >= 192) return launch_tile<128, 128>(g, ta, tb, vec);
    return launch_tile<64, 64>(g, ta, tb, vec);
}

}  // namespace dali_hip

using namespace dali_hip;

extern "C" {

// Column-major C(m x n) = alpha * op(B)(m x k) * op(A)(k x n) + beta * C is the
// row-major product C[n, m] = alpha * A'[n, k] * B'[k, m] + beta * C where the
// row-major left operand A' is the column-major second operand `A` and vice
// versa. A column-major, non-transposed k x n matrix with leading dimension lda
// is, read row-major, an [n][k] array with row length lda: exactly A'[n, k]
// "not transposed". A column-major transposed operand (stored n x k) reads
// row-major as [k][n], i.e. the transposed storage of A'.
int dali_hip_sgemm(int transB, int transA, int m, int n, int k, float alpha, const float* B, int ldb,
                   const float* A, int lda, float beta, float* C, int ldc) {
    const float* As[1] = {A};
    const float* Bs[1] = {B};
    int Ks[1] = {k}, ldas[1] = {lda}, ldbs[1] = {ldb};
    return sgemm_rowmajor(1, transA != 0, transB != 0, n, m, Ks, As, ldas, Bs, ldbs, alpha, beta, C, ldc);
}

int dali_hip_sgemm_pair(int transB1, int transA1, int transB2, int transA2, int m, int n, int k1, int k2,
                        float alpha, const float* B1, int ldb1, const float* A1, int lda1, const float* B2,
                        int ldb2, const float* A2, int lda2, float beta, float* C, int ldc) {
    if ((transA1 != 0) != (transA2 != 0) || (transB1 != 0) != (transB2 != 0)) {
        // mixed layouts: two accumulating launches
        int st = dali_hip_sgemm(transB1, transA1, m, n, k1, alpha, B1, ldb1, A1, lda1, beta, C, ldc);
        if (st) return st;
        return dali_hip_sgemm(transB2, transA2, m, n, k2, alpha, B2, ldb2, A2, lda2, 1.0f, C, ldc);
    }
    const float* As[2] = {A1, A2};
    const float* Bs[2] = {B1, B2};
    int Ks[2] = {k1, k2}, ldas[2] = {lda1, lda2}, ldbs[2] = {ldb1, ldb2};
    return sgemm_rowmajor(2, transA1 != 0, transB1 != 0, n, m, Ks, As, ldas, Bs, ldbs, alpha, beta, C, ldc);
}

}  // extern "C"
