// fp64 GEMM on the matrix cores of gfx950 (v_mfma_f64_16x16x4f64): the double-precision branch of op::dot, which the
// reference hands to cublasDgemm (dali/array/gemm/cublas_gemm.cu:167-178, cblas_dgemm in dali/array/gemm/cpu_gemm.cpp).
//
// A workgroup of four waves owns a 64 x 64 or a 128 x 128 tile of C; each wave a quarter of it as 2 x 2 or 4 x 4
// accumulators of 16 x 16. A slab of 16 values of k is staged in LDS k-major ([k][row] and [k][column]), so that a lane's
// operand of the instruction (row or column = lane % 16, k = lane / 16) is one 8-byte read and sixteen lanes read sixteen
// neighbours. Global loads of the next slab are issued before the products of the current one and land in the other LDS
// buffer: one barrier per slab. The instruction takes 16 passes (64 cycles), so the loads, the LDS traffic and the
// address arithmetic of a slab hide behind the sixteen to sixty-four instructions each wave issues for it. Operands are
// addressed through (row stride, k stride) pairs, which covers the four transposition cases; the lane-to-element map of
// the global loads follows whichever stride is 1.
#include <cstdint>

#include "runtime.h"

namespace dali_hip {
namespace {

typedef double d4 __attribute__((ext_vector_type(4)));

constexpr int BK = 16;

struct DgemmArgs {
    int M, N, K;              // row-major problem: C[M, N] = alpha * A[M, K] * B[K, N] + beta * C
    const double* A;
    long ai, ak;              // element (i, k) of A at A[i * ai + k * ak]
    const double* B;
    long bk, bj;              // element (k, j) of B at B[k * bk + j * bj]
    double* C;
    long ldc;
    double alpha, beta;
};

// T: 16 x 16 accumulators per wave and dimension. T = 2: the workgroup's tile of C is 64 x 64 (many workgroups for a small
// C); T = 4: 128 x 128, which halves the operand traffic per product and leaves four times the matrix instructions between
// two barriers (chosen when that still gives every compute unit a tile).
// CHECKED: the tile hangs over an edge of C or the last slab of K is short: every load is bounds-tested. Otherwise a
// thread's loads are a wave-uniform slab pointer plus a constant 32-bit offset, with no vector arithmetic in the loop
// (vector-ALU instructions between matrix instructions hold the matrix pipe back).
template <bool CHECKED, int T>
__device__ __forceinline__ void dgemm_tile(const DgemmArgs& a, double* lds, int m0, int n0) {
    constexpr int BM = 32 * T, BN = 32 * T;
    constexpr int PITCH = BM + 2;        // doubles per LDS row: the four k-groups of an operand read start 4 banks apart
    constexpr int LOADS = BM * BK / 256;  // elements of each operand tile a thread fetches per slab
    double (*As)[BK][PITCH] = reinterpret_cast<double (*)[BK][PITCH]>(lds);
    double (*Bs)[BK][PITCH] = reinterpret_cast<double (*)[BK][PITCH]>(lds + 2 * BK * PITCH);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // which element of a BM x 16 tile a thread fetches in its c-th load: along k when k is the unit stride, along the rows
    // otherwise
    const bool a_k_fast = a.ak == 1, b_k_fast = a.bk == 1;
    int ar[LOADS], akk[LOADS], bc[LOADS], bkk[LOADS];
    int aoff[LOADS], boff[LOADS];
#pragma unroll
    for (int c = 0; c < LOADS; ++c) {
        ar[c] = a_k_fast ? tid / 16 + 16 * c : tid % BM;
        akk[c] = a_k_fast ? tid % 16 : tid / BM + (256 / BM) * c;
        bc[c] = b_k_fast ? tid / 16 + 16 * c : tid % BN;
        bkk[c] = b_k_fast ? tid % 16 : tid / BN + (256 / BN) * c;
        aoff[c] = CHECKED ? 0 : (int)((long)ar[c] * a.ai + (long)akk[c] * a.ak);
        boff[c] = CHECKED ? 0 : (int)((long)bkk[c] * a.bk + (long)bc[c] * a.bj);
    }
    const double* Atile = a.A + (long)m0 * a.ai;
    const double* Btile = a.B + (long)n0 * a.bj;
    double ra[LOADS], rb[LOADS];
    auto fetch = [&](int k0) {
        if (CHECKED) {
#pragma unroll
            for (int c = 0; c < LOADS; ++c) {
                const int i = m0 + ar[c], k = k0 + akk[c];
                ra[c] = (i < a.M && k < a.K) ? a.A[(long)i * a.ai + (long)k * a.ak] : 0.0;
                const int j = n0 + bc[c], kb = k0 + bkk[c];
                rb[c] = (j < a.N && kb < a.K) ? a.B[(long)kb * a.bk + (long)j * a.bj] : 0.0;
            }
        } else {
            const double* As0 = Atile + (long)k0 * a.ak;  // wave-uniform
            const double* Bs0 = Btile + (long)k0 * a.bk;
#pragma unroll
            for (int c = 0; c < LOADS; ++c) {
                ra[c] = As0[aoff[c]];
                rb[c] = Bs0[boff[c]];
            }
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int c = 0; c < LOADS; ++c) {
            As[buf][akk[c]][ar[c]] = ra[c];
            Bs[buf][bkk[c]][bc[c]] = rb[c];
        }
    };
    const int wm = (wave >> 1) * 16 * T, wn = (wave & 1) * 16 * T;
    const int r = lane & 15, kg = lane >> 4;
    d4 acc[T][T];
#pragma unroll
    for (int i = 0; i < T; ++i)
#pragma unroll
        for (int j = 0; j < T; ++j) acc[i][j] = (d4){0.0, 0.0, 0.0, 0.0};
    fetch(0);
    stage(0);
    __syncthreads();
    const int slabs = (a.K + BK - 1) / BK;
    for (int s = 0; s < slabs; ++s) {
        const int buf = s & 1;
        if (s + 1 < slabs) fetch((s + 1) * BK);
#pragma unroll
        for (int ks = 0; ks < BK; ks += 4) {
            double av[T], bv[T];
#pragma unroll
            for (int i = 0; i < T; ++i) av[i] = As[buf][ks + kg][wm + 16 * i + r];
#pragma unroll
            for (int j = 0; j < T; ++j) bv[j] = Bs[buf][ks + kg][wn + 16 * j + r];
#pragma unroll
            for (int i = 0; i < T; ++i)
#pragma unroll
                for (int j = 0; j < T; ++j) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(av[i], bv[j], acc[i][j], 0, 0, 0);
        }
        if (s + 1 < slabs) stage(buf ^ 1);  // the other buffer: last read before the previous barrier
        __syncthreads();
    }
    // a lane holds column lane % 16 and rows 4 * v + lane / 16 of each 16 x 16 accumulator
#pragma unroll
    for (int i = 0; i < T; ++i)
#pragma unroll
        for (int j = 0; j < T; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int row = m0 + wm + 16 * i + 4 * v + kg, col = n0 + wn + 16 * j + r;
                if (!CHECKED || (row < a.M && col < a.N)) {
                    double* p = a.C + (long)row * a.ldc + col;
                    const double prod = a.alpha * acc[i][j][v];
                    *p = a.beta == 0.0 ? prod : prod + a.beta * *p;
                }
            }
}

template <int T>
__global__ __launch_bounds__(256, T == 4 ? 2 : 4) void dgemm_kernel(DgemmArgs a, int offsets_fit) {
    extern __shared__ double dgemm_lds[];  // [A, B][2 buffers][BK][32 T + 2]
    constexpr int BM = 32 * T, BN = 32 * T;
    const int tiles_n = (a.N + BN - 1) / BN;
    const int tm = blockIdx.x / tiles_n, tn = blockIdx.x % tiles_n;
    const int m0 = tm * BM, n0 = tn * BN;
    const bool interior = offsets_fit && m0 + BM <= a.M && n0 + BN <= a.N && a.K % BK == 0 && a.K > 0;  // workgroup-uniform
    if (interior) dgemm_tile<false, T>(a, dgemm_lds, m0, n0);
    else dgemm_tile<true, T>(a, dgemm_lds, m0, n0);
}

}  // namespace
}  // namespace dali_hip

using namespace dali_hip;

extern "C" int dali_hip_dgemm(int transB, int transA, int m, int n, int k, double alpha, const double* B, int ldb, const double* A, int lda,
                              double beta, double* C, int ldc) {
    if (ensure_init()) return DALI_HIP_ERROR;
    if (m < 0 || n < 0 || k < 0) return fail("dali_hip_dgemm: negative extent (m=%d n=%d k=%d)", m, n, k);
    if (m == 0 || n == 0) return DALI_HIP_OK;
    if (!C || (k > 0 && (!A || !B))) return fail("dali_hip_dgemm: NULL operand");
    // row-major view of the column-major call: C[n, m] = alpha * A[n, k] * B[k, m] + beta * C
    const int rows = n, cols = m;
    if (ldc < cols) return fail("dali_hip_dgemm: ldc %d is smaller than the row length %d", ldc, cols);
    if (k > 0) {
        if (lda < (transA ? rows : k)) return fail("dali_hip_dgemm: lda %d is too small", lda);
        if (ldb < (transB ? k : cols)) return fail("dali_hip_dgemm: ldb %d is too small", ldb);
    }
    DgemmArgs a;
    a.M = rows; a.N = cols; a.K = k;
    a.A = A; a.ai = transA ? 1 : lda; a.ak = transA ? lda : 1;
    a.B = B; a.bk = transB ? 1 : ldb; a.bj = transB ? ldb : 1;
    a.C = C; a.ldc = ldc; a.alpha = alpha; a.beta = beta;
    // 128 x 128 tiles when they still give every compute unit one, 64 x 64 otherwise
    static int cus = 0;
    if (cus == 0) {
        hipDeviceProp_t prop;
        cus = hipGetDeviceProperties(&prop, bound_device()) == hipSuccess ? prop.multiProcessorCount : 256;
    }
    const long tiles128 = (long)((rows + 127) / 128) * ((cols + 127) / 128);
    const int T = tiles128 >= cus ? 4 : 2;
    const int BM = 32 * T;
    const long tiles = (long)((rows + BM - 1) / BM) * ((cols + BM - 1) / BM);
    if (tiles > 0x7fffffffL) return fail("dali_hip_dgemm: too many tiles");
    // a thread's offset inside a BM x 16 operand tile as a 32-bit number of elements
    const long span_a = (BM - 1) * (a.ai > 0 ? a.ai : -a.ai) + 15 * (a.ak > 0 ? a.ak : -a.ak);
    const long span_b = 15 * (a.bk > 0 ? a.bk : -a.bk) + (BM - 1) * (a.bj > 0 ? a.bj : -a.bj);
    const int offsets_fit = span_a < (1L << 28) && span_b < (1L << 28);
    const size_t lds_bytes = (size_t)2 * 2 * BK * (BM + 2) * sizeof(double);
    if (T == 4) {
        // more than the 64 KiB a kernel may use without asking; once (later calls may be recorded into a graph)
        static bool attribute_set = false;
        if (!attribute_set) {
            if (hipFuncSetAttribute((const void*)dgemm_kernel<4>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess)
                return fail("dali_hip_dgemm: cannot reserve %zu bytes of LDS", lds_bytes);
            attribute_set = true;
        }
        hipLaunchKernelGGL(dgemm_kernel<4>, dim3((unsigned)tiles), dim3(256), lds_bytes, stream(), a, offsets_fit);
    } else {
        hipLaunchKernelGGL(dgemm_kernel<2>, dim3((unsigned)tiles), dim3(256), lds_bytes, stream(), a, offsets_fit);
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("dali_hip_dgemm launch failed: %s", hipGetErrorString(e));
    return DALI_HIP_OK;
}
