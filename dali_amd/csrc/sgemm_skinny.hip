// fp32 product with at most 64 rows on the left: C[M, N] = alpha * A[M, K] . B[K, N] + beta * C, A row-major, B row-major
// or stored transposed
// (the output projection of a decoder step, dot(h [batch, hidden], W [hidden, vocabulary]); the call of
// dali/array/gemm/cublas_gemm.cu:153-166 at small n).
//
// The tiles of the general kernel are 64 rows high and hold their operands in LDS: with 8 rows it does the matrix work
// of 64 and, more to the point, B passes through LDS for one use. Such a product has to stream B once (131 MB at
// 1024 x 32000: 16 us at 8 TB/s, against 78 us through the general kernel; here 20 us up to 16 rows, 26 at 32, 46 at 64
// rows, where the product is bound by the matrix pipe as much as by memory). Here B goes straight from memory into the B
// operand of the matrix instruction: a workgroup owns 64 consecutive columns, 256 bytes of every row of B, over a 1 / KS
// share of K, the share split over its four waves. A lane loads four consecutive columns of row k with one 16-byte load
// and feeds them to four instructions (v_mfma_f32_16x16x4_f32), whose 16-column tiles are therefore the columns
// congruent to 0, 1, 2 and 3 modulo 4. The four waves' partial tiles meet in LDS; with KS > 1 the workgroups of a column
// block publish their sums in the library workspace and the last to take a ticket adds them in k order.
// Rows of A past M, and the rows of both operands past K, lie outside the buffers' ranges and read as zero; what a tile
// computes for columns past N is never stored.
#include <cstdint>
#include <cstdlib>

#include "runtime.h"

namespace dali_hip {
namespace {

typedef float f4 __attribute__((ext_vector_type(4)));
constexpr int kCoherentLoad = 16;       // cache policy of a buffer load: device scope
constexpr int kOutside = 0x7ffffff0;    // an offset beyond every buffer range: the load returns zero
constexpr int kCols = 64;               // columns of a workgroup
constexpr int kMaxShares = 16;

struct SkinnyArgs {
    int M, N, K, KS, KP;  // KP: the K range of a workgroup, a multiple of 64
    const float* A;
    const float* B;
    float* C;
    int lda, ldb, ldc;
    float alpha, beta;
    unsigned int* tickets;  // one per column block, zero at rest
    float* partials;        // [column blocks][KS][M][64]
};

// MT: 16-row tiles of A; G: trips of 16 values of k whose loads are issued together
// TB: B is stored transposed, [N][K] with row length ldb (the weights of a layer kept as [outputs, inputs]). A lane then
// loads four consecutive k of its column, as it does for its row of A, and a 16-column tile is 16 consecutive columns.
template <int MT, int G, bool TB>
__global__ __launch_bounds__(256, 2) void sgemm_skinny_kernel(SkinnyArgs a) {
    extern __shared__ float red_flat[];  // [4 waves][4 column tiles][MT][16][16]
    float (*red)[4][MT][16][16] = reinterpret_cast<float (*)[4][MT][16][16]>(red_flat);
    __shared__ int is_last;
    const int M = a.M, N = a.N, K = a.K, KS = a.KS;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ks = blockIdx.x % KS, cb = blockIdx.x / KS;
    const int col0 = cb * kCols;
    const int arow = lane & 15, kgrp = lane >> 4;
    const int KW = a.KP / 4;  // K range of a wave, a multiple of 16
    const __amdgpu_buffer_rsrc_t arows = __builtin_amdgcn_make_buffer_rsrc((void*)a.A, 0, ((M - 1) * a.lda + K) * 4, 0x00027000);
    const __amdgpu_buffer_rsrc_t brows = __builtin_amdgcn_make_buffer_rsrc((void*)a.B, 0, TB ? ((N - 1) * a.ldb + K) * 4 : ((K - 1) * a.ldb + N) * 4, 0x00027000);
    f4 acc[4][MT];
#pragma unroll
    for (int ct = 0; ct < 4; ++ct)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[ct][m] = (f4){0.f, 0.f, 0.f, 0.f};
    const int kbase = ks * a.KP + wave * KW;
    const int bcol = (col0 + 4 * arow) * 4;  // byte offset of this lane's four columns inside a row of B
    const int trips = KW / 16;
    for (int q0 = 0; q0 < trips; q0 += G) {
        f4 av[G][MT];
        f4 bv[G][4];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const int kk = kbase + 16 * (q0 + g) + 4 * kgrp;  // this lane's four values of k
            const bool valid = q0 + g < trips && kk < K;      // (K is a multiple of 4: the four are inside or outside together)
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                // TB: c counts column tiles and the vector runs along k; otherwise c counts the lane's four rows of B and the
                // vector runs along the columns
                const int col = col0 + 16 * c + arow;
                const int off = TB ? (col < N && valid ? (col * a.ldb + kk) * 4 : kOutside) : (valid ? (kk + c) * a.ldb * 4 + bcol : kOutside);
                bv[g][c] = __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(brows, off, 0, 0));
            }
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const int row = 16 * m + arow;
                av[g][m] = __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(arows, row < M && valid ? (row * a.lda + kk) * 4 : kOutside, 0, 0));
            }
        }
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int ct = 0; ct < 4; ++ct)
#pragma unroll
                    for (int m = 0; m < MT; ++m)
                        acc[ct][m] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[g][m][c], TB ? bv[g][ct][c] : bv[g][c][ct], acc[ct][m], 0, 0, 0);
    }
    // a lane holds column lane % 16 of tile ct (column 4 * (lane % 16) + ct of the block, or 16 * ct + lane % 16 when B is
    // stored transposed) and rows 4 * (lane / 16) + v
#pragma unroll
    for (int ct = 0; ct < 4; ++ct)
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[wave][ct][m][4 * kgrp + v][arow] = acc[ct][m][v];
    __syncthreads();
    auto waves_sum = [&](int row, int u) {
        float s = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) s += TB ? red[w][u >> 4][row / 16][row & 15][u & 15] : red[w][u & 3][row / 16][row & 15][u >> 2];
        return s;
    };
    if (KS == 1) {
        for (int e = tid; e < M * kCols; e += 256) {
            const int row = e / kCols, u = e % kCols, col = col0 + u;
            if (col < N) {
                float* p = a.C + (size_t)row * a.ldc + col;
                const float s = a.alpha * waves_sum(row, u);
                *p = a.beta == 0.0f ? s : s + a.beta * *p;
            }
        }
        return;
    }
    float* mine = a.partials + ((size_t)cb * KS + ks) * (size_t)M * kCols;
    for (int e = tid; e < M * kCols; e += 256)
        __hip_atomic_store(mine + e, waves_sum(e / kCols, e % kCols), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // the shares are acknowledged by memory before the ticket is drawn; the clobber keeps the compiler from moving them
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        const unsigned int ticket = __hip_atomic_fetch_add(a.tickets + cb, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        is_last = ticket == (unsigned int)(KS - 1);
    }
    __syncthreads();
    if (!is_last) return;
    // the fold: four neighbouring columns of a row per thread; every share is asked for (device-coherent loads) before the
    // first is awaited, then they are added in k order
    const float* blockp = a.partials + (size_t)cb * KS * (size_t)M * kCols;
    const __amdgpu_buffer_rsrc_t shares = __builtin_amdgcn_make_buffer_rsrc((void*)blockp, 0, KS * M * kCols * 4, 0x00027000);
    for (int quad = tid; quad < M * (kCols / 4); quad += 256) {
        const int row = quad / (kCols / 4), u = (quad % (kCols / 4)) * 4, col = col0 + u;
        f4 pv[kMaxShares];
#pragma unroll
        for (int k = 0; k < kMaxShares; ++k)
            pv[k] = k < KS ? __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(shares, ((k * M + row) * kCols + u) * 4, 0, kCoherentLoad)) : (f4){0.f, 0.f, 0.f, 0.f};
        f4 sum = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < kMaxShares; ++k)
            if (k < KS) sum += pv[k];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (col + j < N) {
                float* p = a.C + (size_t)row * a.ldc + col + j;
                const float s = a.alpha * sum[j];
                *p = a.beta == 0.0f ? s : s + a.beta * *p;
            }
    }
    if (tid == 0) __hip_atomic_store(a.tickets + cb, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---------------------------------------------------------------------------------------------- short inner extent
// C[M, N] = alpha * A . B + beta * C with K <= 64, B row-major [K][N], A stored as [K][M] or [M][K]: the weight gradient of
// a layer, dot(h^T [hidden, batch], g [batch, outputs]), at a small batch, or a layer with few inputs. Such a product is bound by writing C once; the tiled
// kernel spends a whole 64-deep slab, its prologue and its epilogue on every 64 x 64 tile (1024 x 32000 at K = 8:
// 51 us for 131 MB). Here a workgroup keeps its 64 columns of A (64 rows of C) in registers in the layout of the
// instruction's A operand for all of K and walks along a strip of C; per 64 columns a wave loads K/4 16-byte pieces of B
// (four consecutive columns of row k, feeding the four column tiles congruent to 0..3 modulo 4, as above) and stores its
// 64 x 64 results as 16-byte pieces: the four tiles' values of a lane are four consecutive columns of one row.
struct SmallKArgs {
    int M, N, K, CB;  // CB: 64-column blocks per wave
    const float* A;
    const float* B;
    float* C;
    int a_row, a_k, a_extent;  // element (row, k) of A at A[row * a_row + k * a_k]; a_extent: elements up to its last one
    int ldb, ldc;
    float alpha, beta;
};

// S: steps of 4 values of k (K <= 4 S)
template <int S>
__global__ __launch_bounds__(256, 2) void sgemm_smallk_kernel(SmallKArgs a) {
    const int M = a.M, N = a.N, K = a.K;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int arow = lane & 15, kgrp = lane >> 4;
    const int row0 = blockIdx.x * 64;
    // rows of both operands past K lie outside the ranges and read as zero
    const __amdgpu_buffer_rsrc_t arows = __builtin_amdgcn_make_buffer_rsrc((void*)a.A, 0, a.a_extent * 4, 0x00027000);
    const __amdgpu_buffer_rsrc_t brows = __builtin_amdgcn_make_buffer_rsrc((void*)a.B, 0, ((K - 1) * a.ldb + N) * 4, 0x00027000);
    float av[S][4];
#pragma unroll
    for (int s = 0; s < S; ++s)
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            const int k = 4 * s + kgrp, row = row0 + 16 * m + arow;
            av[s][m] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(arows, k < K && row < M ? (k * a.a_k + row * a.a_row) * 4 : kOutside, 0, 0));
        }
    const int first = (blockIdx.y * 4 + wave) * a.CB;
    for (int cb = first; cb < first + a.CB; ++cb) {
        const int col0 = cb * kCols;
        if (col0 >= N) break;  // (wave-uniform)
        const int col = col0 + 4 * arow;
        f4 bv[S];
#pragma unroll
        for (int s = 0; s < S; ++s) {
            const int k = 4 * s + kgrp;
            bv[s] = __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(brows, k < K ? (k * a.ldb + col) * 4 : kOutside, 0, 0));
        }
        f4 acc[4][4];
#pragma unroll
        for (int ct = 0; ct < 4; ++ct)
#pragma unroll
            for (int m = 0; m < 4; ++m) acc[ct][m] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < S; ++s)
#pragma unroll
            for (int ct = 0; ct < 4; ++ct)
#pragma unroll
                for (int m = 0; m < 4; ++m) acc[ct][m] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[s][m], bv[s][ct], acc[ct][m], 0, 0, 0);
        // a lane holds, of tile ct, column 4 * (lane % 16) + ct of the block and rows 16 m + 4 * (lane / 16) + v
#pragma unroll
        for (int m = 0; m < 4; ++m)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int row = row0 + 16 * m + 4 * kgrp + v;
                if (row >= M || col >= N) continue;
                float* p = a.C + (size_t)row * a.ldc + col;
                f4 r = (f4){a.alpha * acc[0][m][v], a.alpha * acc[1][m][v], a.alpha * acc[2][m][v], a.alpha * acc[3][m][v]};
                typedef f4 f4u __attribute__((aligned(4)));
                if (col + 3 < N) {
                    if (a.beta != 0.0f) {
                        const f4 old = *reinterpret_cast<const f4u*>(p);
                        r += a.beta * old;
                    }
                    *reinterpret_cast<f4u*>(p) = r;
                } else {
                    for (int j = 0; j < 4 && col + j < N; ++j) p[j] = a.beta == 0.0f ? r[j] : r[j] + a.beta * p[j];
                }
            }
    }
}

}  // namespace

// 1: the product was launched; 0: not a case for this kernel (the caller takes the general path); -1: failure
int sgemm_skinny(bool tb, int M, int N, int K, float alpha, const float* A, int lda, const float* B, int ldb, float beta, float* C, int ldc) {
    static const bool enabled = !(getenv("DALI_HIP_GEMM_SKINNY") && atoi(getenv("DALI_HIP_GEMM_SKINNY")) == 0);
    if (!enabled || M < 1 || M > 64 || K < 64 || K % 4 != 0 || N < 64) return 0;
    // 32-bit byte offsets into both operands
    if ((size_t)(tb ? N : K) * ldb * 4 + 4096 >= ((size_t)1 << 31) || (size_t)M * lda * 4 + 4096 >= ((size_t)1 << 31)) return 0;
    if (((uintptr_t)A | (uintptr_t)B) % 4 != 0) return 0;
    const int blocks = (N + kCols - 1) / kCols;
    // K is split until there are about two workgroups per compute unit (each with at least 256 values of k): a split
    // costs its workgroups a publication, a ticket and a fold, three memory round trips during which their matrix pipes
    // idle, so 500 column blocks (32000 columns) stay whole
    int KS = 1;
    while (blocks * KS < 384 && KS < kMaxShares && K / (KS * 2) >= 256) KS *= 2;
    // a narrow B: shares down to 128 values of k until there are 128 workgroups ([8,1024].[1024,1024]: 7.1 us against 15.4
    // through the tiled kernel, which walks its sixteen slabs one after the other whatever the number of rows)
    while (blocks * KS < 128 && KS < kMaxShares && K / (KS * 2) >= 128) KS *= 2;
    if (blocks * KS < 32) return 0;
    // 33 to 64 rows with a split of K: the tiled kernel is as fast or faster unless the shares are long
    // (64 x 4096 over K = 1024: 16.4 against 22.9 us here; 64 x 1024 over K = 32000: 71 against 58 us)
    if (KS > 1 && M > 32 && K / KS < (M > 48 ? 1536 : 1024)) return 0;
    if (KS > 1 && ((size_t)blocks * KS * M * kCols * sizeof(float) > kWorkspacePartialBytes || blocks > kWorkspaceCounters - 2)) KS = 1;
    SkinnyArgs a;
    a.M = M; a.N = N; a.K = K; a.KS = KS;
    a.KP = ((K + 64 * KS - 1) / (64 * KS)) * 64;
    a.A = A; a.B = B; a.C = C;
    a.lda = lda; a.ldb = ldb; a.ldc = ldc;
    a.alpha = alpha; a.beta = beta;
    a.tickets = (unsigned int*)workspace();
    a.partials = (float*)(workspace() + kWorkspaceCounterBytes);
    const int MT = (M + 15) / 16;
    const size_t lds_bytes = (size_t)4 * 4 * MT * 256 * sizeof(float);
    const unsigned grid = (unsigned)blocks * KS;
    hipError_t e = hipSuccess;
    auto launch = [&](auto kernel) {
        e = reserve_dynamic_lds((const void*)kernel, lds_bytes);
        if (e == hipSuccess) hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), lds_bytes, stream(), a);
    };
    // (trips issued together: 1 to 8 measured alike, the compiler pipelines the loop; 4 is the best of them on short K shares)
#define SKINNY_CASE(mt)                                           \
    if (tb) launch(sgemm_skinny_kernel<mt, 4, true>);             \
    else launch(sgemm_skinny_kernel<mt, 4, false>);               \
    break;
    switch (MT) {
        case 1: SKINNY_CASE(1)
        case 2: SKINNY_CASE(2)
        case 3: SKINNY_CASE(3)
        default: SKINNY_CASE(4)
    }
#undef SKINNY_CASE
    if (e == hipSuccess) e = hipGetLastError();
    if (e != hipSuccess) {
        fail("sgemm (at most 64 rows) launch failed: %s", hipGetErrorString(e));
        return -1;
    }
    return 1;
}


// the same convention of results as sgemm_skinny; ta: A is stored as [K][M]
int sgemm_smallk(bool ta, bool tb, int M, int N, int K, float alpha, const float* A, int lda, const float* B, int ldb, float beta, float* C, int ldc) {
    static const bool enabled = !(getenv("DALI_HIP_GEMM_SMALLK") && atoi(getenv("DALI_HIP_GEMM_SMALLK")) == 0);
    if (!enabled || tb || K < 1 || K > 64 || M < 64 || N < 256) return 0;
    if ((size_t)K * ldb * 4 + 4096 >= ((size_t)1 << 31) || (size_t)(ta ? K : M) * lda * 4 + 4096 >= ((size_t)1 << 31)) return 0;
    if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) % 4 != 0) return 0;
    const int row_blocks = (M + 63) / 64, col_blocks = (N + kCols - 1) / kCols;
    // blocks per wave: long strips amortise the registers of A, but keep a few thousand workgroups
    if ((long)row_blocks * ((col_blocks + 3) / 4) < 256) return 0;  // a small C: the tiled kernel ([1024,1024] at K = 64: 5.9 against 7.7 us)
    const int enough = K <= 16 ? 1024 : 512;  // (measured: 1024 x 32000 at K = 8 / 64: 22.8 / 51.6 us with 1024, 24.0 / 49.4 with 512)
    int CB = 1;
    while (CB < 8 && (long)row_blocks * ((col_blocks + 4 * CB * 2 - 1) / (4 * CB * 2)) >= enough) CB *= 2;
    const int col_groups = (col_blocks + 4 * CB - 1) / (4 * CB);
    if (col_groups > 65535) return 0;
    SmallKArgs a;
    a.M = M; a.N = N; a.K = K; a.CB = CB;
    a.A = A; a.B = B; a.C = C;
    a.a_row = ta ? 1 : lda; a.a_k = ta ? lda : 1;
    a.a_extent = ta ? (K - 1) * lda + M : (M - 1) * lda + K;
    a.ldb = ldb; a.ldc = ldc;
    a.alpha = alpha; a.beta = beta;
    const dim3 grid((unsigned)row_blocks, (unsigned)col_groups);
    const int S = (K + 3) / 4;
    if (S <= 2) hipLaunchKernelGGL(sgemm_smallk_kernel<2>, grid, dim3(256), 0, stream(), a);
    else if (S <= 4) hipLaunchKernelGGL(sgemm_smallk_kernel<4>, grid, dim3(256), 0, stream(), a);
    else if (S <= 8) hipLaunchKernelGGL(sgemm_smallk_kernel<8>, grid, dim3(256), 0, stream(), a);
    else hipLaunchKernelGGL(sgemm_smallk_kernel<16>, grid, dim3(256), 0, stream(), a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        fail("sgemm (inner extent of at most 64) launch failed: %s", hipGetErrorString(e));
        return -1;
    }
    return 1;
}

}  // namespace dali_hip
