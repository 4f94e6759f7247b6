// fp32 GEMM on the CDNA4 matrix cores (v_mfma_f32_32x32x2_f32), LDS-staged with
// a multi-slab register prefetch, for dali_hip_sgemm / dali_hip_sgemm_pair.
//
// Row-major view used inside this file: C[M,N] = alpha * sum_s A_s[M,K_s] * B_s[K_s,N] + beta * C
// for one or two (A_s, B_s) segments. The column-major entry points map onto it
// by swapping the operands (C^T = B^T A^T), exactly as the reference does when it
// calls a column-major BLAS (dali/array/gemm/cpu_gemm.cpp:43-68).
//
// Work decomposition: a workgroup of KW wave sets (4 waves each, 2x2) owns a BM x BN
// tile of C; each wave owns (BM/2) x (BN/2), built from 32x32 MFMA accumulators, and
// the KW sets split the k-groups of every slab (summed through LDS at the end). K is
// walked in slabs of BK (32 or 64).
//
// LDS layout.  As[m][k]: rows of BK floats in 16-byte granules, granule g of row m
// stored in slot (g & ~7) | ((g ^ m) & 7). A lane's MFMA operands for four consecutive
// MFMAs are one ds_read_b128 (granule 2t + h of its row), and the eight lanes the
// LDS serves per cycle hit eight different slots, so the read is conflict-free.
// Bs[k][n]: natural rows; lane l reads column l % 32 of row k, a conflict-free
// 32-float row read. Within a group of eight k the two half-waves (h = lane / 32)
// take k = 8t + 4h + c for c = 0..3, the same assignment for A and B, so every
// MFMA still sums two distinct k.
//
// Latency.  One workgroup per CU means one wave per SIMD, so nothing hides a
// global-memory round trip except distance: slabs are fetched into registers
// DEPTH slabs ahead of their use, written to the other LDS buffer one slab ahead,
// and consumed from LDS while the MFMA pipe works (one barrier per slab).
#include "runtime.h"
#include "gate_math.h"

#include <cstdlib>
#include <cstring>
#include <type_traits>

namespace dali_hip {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// 16-byte accesses through the native vector type (an aggregate float4 copy is a memcpy to the
// optimiser, which keeps the register stages from being promoted out of private memory)
// (the load claims element alignment only: global memory takes a 16-byte access at any dword address as one
// instruction, so operands whose rows start off a 16-byte boundary - an odd leading dimension, a view that starts inside
// a row - go through the same kernels)
typedef floatx4 floatx4u __attribute__((aligned(4)));
__device__ __forceinline__ float4 ld16(const void* p) {
    const floatx4 v = *(const floatx4u*)p;
    return make_float4(v.x, v.y, v.z, v.w);
}
// 16-byte aligned (LDS)
__device__ __forceinline__ float4 ld16a(const void* p) {
    const floatx4 v = *(const floatx4*)p;
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void st16(void* p, const float4& v) {
    floatx4 w = {v.x, v.y, v.z, v.w};
    *(floatx4*)p = w;
}

struct GemmSeg {
    const float* A;
    const float* B;
    int lda, ldb, K;
};

constexpr int kMaxSeg = 8;

struct GemmArgs {
    GemmSeg seg[kMaxSeg];
    int nseg;
    int M, N;
    float* C;
    int ldc;
    float alpha, beta;
    // split-K: gridDim.z workgroups share one tile of C, each walking a contiguous share of the
    // slabs; partial tiles and the per-tile ticket counters live in the library workspace
    unsigned int* counters;
    float* partials;
    // fused LSTM gate epilogue (GATES kernels): C is not written; the tile's pre-activations go through the
    // gate arithmetic with bias[4H], c_prev[M, H] and leave as c_out[M, H], h_out[M, H]
    const float* bias;
    const float* c_prev;
    float* c_out;
    float* h_out;
    int H;
    // Output row map (convolution over a padded image computed at every padded position): row m stands for position
    // (n, i, j) of an [., map_h, map_w] grid; only i < map_oh, j < map_ow are stored, at row (n * map_oh + i) * map_ow + j.
    // hw = map_h * map_w and map_w come with the multiplier / shift of an exact division (see row_map_div).
    int map_on;
    unsigned map_hw, map_hw_m, map_w, map_w_m;
    int map_hw_s, map_w_s, map_oh, map_ow;
};

// n / d for n < 2^31: m = ceil(2^(31+s) / d) with 2^(s-1) < d <= 2^s, computed by the launcher
__device__ __forceinline__ unsigned row_map_div(unsigned n, unsigned m, int s) { return (unsigned)(((unsigned long long)n * m) >> (31 + s)); }

__device__ __forceinline__ void publish(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float observe(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// MAXSEG: how many terms the instantiation can walk. Two (the LSTM pair) keeps the segment switch of the main loop a
// pair of scalar selects; the eight-term form (convolution by filter rows) carries a short select chain instead.
template <int BM, int BN, int BK, bool TA, bool TB, bool VEC, int DEPTH, bool EDGE, int KW, bool MIDB, bool GATES = false, int MAXSEG = 2>
__global__ __launch_bounds__(256 * KW, (BM == 128 && !EDGE && KW == 1) ? 2 : 1) void sgemm_kernel(GemmArgs g) {
    // KW wave sets share the tile: set kw takes every KW-th k-group of a slab, so each SIMD holds
    // KW waves that cover each other's LDS and barrier waits; the sets are summed through LDS at the end
    constexpr int THREADS = 256 * KW;
    constexpr int WTM = BM / 2, WTN = BN / 2;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int A_F4 = BM * BK / 4 / THREADS;  // float4 fetches per thread for the A slab
    constexpr int B_F4 = BN * BK / 4 / THREADS;
    constexpr int BPAD = 8;  // rows 4 apart (the two half-waves of a B operand read) land 32 banks apart
    // a lone accumulator per wave would serialise dependent MFMAs: split k over two chains
    constexpr int CHAINS = (TM * TN == 1) ? 2 : 1;
    static_assert(A_F4 >= 1 && B_F4 >= 1, "tile too small for the workgroup");
    static_assert((BK / 8) % KW == 0, "k-groups must divide among the wave sets");

    // The small-tile interior kernel runs a software pipeline with the workgroup barrier in the middle of a slab
    // (see its loop below), which needs a third slab buffer.
    constexpr int G = BK / 8 / KW;  // k-groups of a slab per wave set
    constexpr bool PIPE = !EDGE && DEPTH == 2 && G >= 2 && G % 2 == 0;
    constexpr int NBUF = PIPE && MIDB ? 4 : 2;
    // one LDS block: the A slab buffers, the B slab buffers; reused for the wave-set fold at the end
    constexpr int AS_FLOATS = NBUF * BM * BK, BS_FLOATS = NBUF * BK * (BN + BPAD), RED_FLOATS = (KW - 1) * BM * BN;
    constexpr int LDS_FLOATS = AS_FLOATS + BS_FLOATS > RED_FLOATS ? AS_FLOATS + BS_FLOATS : RED_FLOATS;
    __shared__ __attribute__((aligned(16))) float lds[LDS_FLOATS];
    float (*As)[BM][BK] = reinterpret_cast<float (*)[BM][BK]>(lds);
    float (*Bs)[BK][BN + BPAD] = reinterpret_cast<float (*)[BK][BN + BPAD]>(lds + AS_FLOATS);

    // slot of 16-byte granule `gr` in row m: the low three bits are permuted per row
    auto swz = [](int gr, int m) __attribute__((always_inline)) { return (gr & ~7) | ((gr ^ m) & 7); };

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = (tid >> 6) & 3;
    const int kw = tid >> 8;  // wave set
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, h = lane >> 5;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    // Gate epilogue: first of the sixteen hidden units of this workgroup. Workgroups are dealt to the eight XCDs
    // round-robin, so consecutive groups of hidden units go to workgroups of the same XCD: the two 64-byte
    // halves of a 128-byte line of the weights are then asked for by the same L2.
    const int hu_base = GATES ? 16 * (gridDim.x % 8 == 0 ? (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8 : blockIdx.x) : 0;
    (void)hu_base;
    const int M = g.M, N = g.N;

    floatx16 acc[CHAINS][TM][TN];
#pragma unroll
    for (int c = 0; c < CHAINS; ++c)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[c][i][j][v] = 0.f;

    float4 ra[DEPTH][A_F4], rb[DEPTH][B_F4];

    // flat list of slabs over the segments
    int nslab_all = 0;
    for (int sg = 0; sg < g.nseg; ++sg) nslab_all += (g.seg[sg].K + BK - 1) / BK;
    // this workgroup's share of the slabs (all of them without split-K)
    const int s_begin = (int)((long)blockIdx.z * nslab_all / gridDim.z);
    const int nslab = (int)((long)(blockIdx.z + 1) * nslab_all / gridDim.z) - s_begin;

    // Per-thread source coordinates of its fetches within a slab (fixed for the whole kernel).
    // A: row `ar` (or k row for the transposed storage), 4-float granule starting at column `ac`.
    int a_r[A_F4], a_c[A_F4], b_r[B_F4], b_c[B_F4];
#pragma unroll
    for (int t = 0; t < A_F4; ++t) {
        int idx = tid + t * THREADS;
        if (!TA) {
            a_r[t] = m0 + idx / (BK / 4);        // m
            a_c[t] = (idx % (BK / 4)) * 4;       // k offset inside the slab
        } else {
            a_r[t] = idx / (BM / 4);             // k offset inside the slab
            a_c[t] = m0 + (idx % (BM / 4)) * 4;  // m
        }
    }
#pragma unroll
    for (int t = 0; t < B_F4; ++t) {
        int idx = tid + t * THREADS;
        if (!TB) {
            b_r[t] = idx / (BN / 4);             // k offset inside the slab
            b_c[t] = n0 + (idx % (BN / 4)) * 4;  // n
            if (GATES) {
                // tile column n' = 16 * gate + j stands for column gate * H + 16 * blockIdx.x + j of the packed weights:
                // the four gates of sixteen hidden units meet in one workgroup
                const int np = (idx % (BN / 4)) * 4;
                b_c[t] = (np / 16) * g.H + hu_base + np % 16;
            }
        } else {
            b_r[t] = n0 + idx / (BK / 4);        // n
            b_c[t] = (idx % (BK / 4)) * 4;       // k offset inside the slab
        }
    }
    if (!EDGE) {
        // Tiles that hang over the edge of C read the last valid row (or 4-column granule) instead: what
        // they compute for rows and columns outside C is never stored, so no zeros are needed, only
        // addresses inside the operands. Granules along M or N are whole here (the launcher checks).
#pragma unroll
        for (int t = 0; t < A_F4; ++t) {
            if (!TA) a_r[t] = a_r[t] < M ? a_r[t] : M - 1;
            else a_c[t] = a_c[t] < M ? a_c[t] : M - 4;
        }
#pragma unroll
        for (int t = 0; t < B_F4; ++t) {
            if (!TB) b_c[t] = b_c[t] < N ? b_c[t] : N - 4;
            else b_r[t] = b_r[t] < N ? b_r[t] : N - 1;
        }
    }

    // One 4-float granule at row r, columns c..c+3 of a row-major array with `rows` x `cols`
    // valid entries. Interior tiles (EDGE == false) load unconditionally; edge tiles clamp the
    // address and zero what lies outside, without branching.
    auto load4 = [&](const float* base, int ld, int r, int c, int rows, int cols) __attribute__((always_inline)) -> float4 {
        if (!EDGE) return ld16(base + (size_t)r * ld + c);
        const bool rv = r < rows;
        const size_t ro = (size_t)(rv ? r : 0) * ld;
        if (VEC) {
            // cols is a multiple of 4 here or the granule is cut: handle both with per-element masks
            const bool full = rv && c + 3 < cols;
            const float4 v = ld16(base + ro + (full ? c : 0));
            if (full) return v;
        }
        float4 v;
        v.x = base[ro + ((rv && c + 0 < cols) ? c + 0 : 0)];
        v.y = base[ro + ((rv && c + 1 < cols) ? c + 1 : 0)];
        v.z = base[ro + ((rv && c + 2 < cols) ? c + 2 : 0)];
        v.w = base[ro + ((rv && c + 3 < cols) ? c + 3 : 0)];
        v.x = (rv && c + 0 < cols) ? v.x : 0.f;
        v.y = (rv && c + 1 < cols) ? v.y : 0.f;
        v.z = (rv && c + 2 < cols) ? v.z : 0.f;
        v.w = (rv && c + 3 < cols) ? v.w : 0.f;
        return v;
    };

    // fetch slab `i` (index into the flat slab list) into register stage S
    auto fetch = [&](auto S, int i) __attribute__((always_inline)) {
        constexpr int st = decltype(S)::value;
        // the segment that holds flat slab i (a uniform walk over at most MAXSEG entries)
        int sg = 0, first_slab = 0;
#pragma unroll
        for (int q = 0; q + 1 < MAXSEG; ++q) {
            const int here = (g.seg[q].K + BK - 1) / BK;
            if (sg == q && q + 1 < g.nseg && i >= first_slab + here) {
                first_slab += here;
                sg = q + 1;
            }
        }
        const float* sa = g.seg[sg].A;
        const float* sb = g.seg[sg].B;
        const int lda = g.seg[sg].lda;
        const int ldb = g.seg[sg].ldb;
        const int K = g.seg[sg].K;
        const int k0 = (i - first_slab) * BK;
#pragma unroll
        for (int t = 0; t < A_F4; ++t) {
            if (!TA)
                ra[st][t] = load4(sa, lda, a_r[t], k0 + a_c[t], M, K);
            else
                ra[st][t] = load4(sa, lda, k0 + a_r[t], a_c[t], K, M);
        }
#pragma unroll
        for (int t = 0; t < B_F4; ++t) {
            if (!TB)
                rb[st][t] = load4(sb, ldb, k0 + b_r[t], b_c[t], K, N);
            else
                rb[st][t] = load4(sb, ldb, b_r[t], k0 + b_c[t], N, K);
        }
    };

    // register stage S -> LDS buffer `buf`, the A half and the B half
    auto stageA = [&](auto S, int buf) __attribute__((always_inline)) {
        constexpr int st = decltype(S)::value;
#pragma unroll
        for (int t = 0; t < A_F4; ++t) {
            int idx = tid + t * THREADS;
            if (!TA) {
                int m = idx / (BK / 4), gr = idx % (BK / 4);
                st16(&As[buf][m][swz(gr, m) * 4], ra[st][t]);
            } else {
                int k = idx / (BM / 4), m = (idx % (BM / 4)) * 4;
                const float vals[4] = {ra[st][t].x, ra[st][t].y, ra[st][t].z, ra[st][t].w};
#pragma unroll
                for (int c = 0; c < 4; ++c) As[buf][m + c][(swz(k >> 2, m + c) << 2) | (k & 3)] = vals[c];
            }
        }
    };
    auto stageB = [&](auto S, int buf) __attribute__((always_inline)) {
        constexpr int st = decltype(S)::value;
#pragma unroll
        for (int t = 0; t < B_F4; ++t) {
            int idx = tid + t * THREADS;
            if (!TB) {
                int k = idx / (BN / 4), n = (idx % (BN / 4)) * 4;
                st16(&Bs[buf][k][n], rb[st][t]);
            } else {
                int n = idx / (BK / 4), k = (idx % (BK / 4)) * 4;
                Bs[buf][k + 0][n] = rb[st][t].x;
                Bs[buf][k + 1][n] = rb[st][t].y;
                Bs[buf][k + 2][n] = rb[st][t].z;
                Bs[buf][k + 3][n] = rb[st][t].w;
            }
        }
    };
    auto stage = [&](auto S, int buf) __attribute__((always_inline)) {
        stageA(S, buf);
        stageB(S, buf);
    };

    // MFMA operands of k-group t (eight k): one granule of A per 32-row block, four B values per
    // 32-column block.
    auto load_ops = [&](int buf, int t, float4 (&a4)[TM], float (&b)[TN][4]) __attribute__((always_inline)) {
#pragma unroll
        for (int ii = 0; ii < TM; ++ii) {
            int m = wm * WTM + ii * 32 + l32;
            a4[ii] = ld16a(&As[buf][m][swz(2 * t + h, m) << 2]);
        }
#pragma unroll
        for (int jj = 0; jj < TN; ++jj)
#pragma unroll
            for (int c = 0; c < 4; ++c) b[jj][c] = Bs[buf][8 * t + 4 * h + c][wn * WTN + jj * 32 + l32];
    };

    // With a single 32x32 accumulator tile per wave the LDS reads of group t+1 are issued before
    // the MFMAs of group t and kept there (scheduling barriers), so an LDS round trip hides
    // behind a full group of MFMAs instead of being waited for in front of every pair. Larger
    // wave tiles have enough independent MFMAs per group and are left to the compiler's scheduler.
    auto compute = [&](int buf) __attribute__((always_inline)) {
        float4 a4[2][TM];
        float b[2][TN][4];
        load_ops(buf, kw, a4[0], b[0]);
#pragma unroll
        for (int tt = 0; tt < BK / 8 / KW; ++tt) {
            const int cur = tt & 1;
            if (tt + 1 < BK / 8 / KW) load_ops(buf, (tt + 1) * KW + kw, a4[cur ^ 1], b[cur ^ 1]);
            if (TM * TN == 1) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int ii = 0; ii < TM; ++ii) {
                    const float a = c == 0 ? a4[cur][ii].x : (c == 1 ? a4[cur][ii].y : (c == 2 ? a4[cur][ii].z : a4[cur][ii].w));
#pragma unroll
                    for (int jj = 0; jj < TN; ++jj) {
                        const int ch = CHAINS == 2 ? (c & 1) : 0;
                        acc[ch][ii][jj] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b[cur][jj][c], acc[ch][ii][jj], 0, 0, 0);
                    }
                }
            if (TM * TN == 1) __builtin_amdgcn_sched_barrier(0);
        }
    };

    // gate epilogue operands, requested now so that they have arrived long before the epilogue
    constexpr int GATE_PAIRS = GATES ? BM * 16 / THREADS : 1;
    float gate_bias[GATE_PAIRS][4], gate_c[GATE_PAIRS];
    if constexpr (GATES) {
#pragma unroll
        for (int q = 0; q < GATE_PAIRS; ++q) {
            const int e = tid + q * THREADS, r = e / 16, j = e % 16, hu = hu_base + j;
            const int m = m0 + r < M ? m0 + r : M - 1;
#pragma unroll
            for (int k = 0; k < 4; ++k) gate_bias[q][k] = g.bias[k * g.H + hu];
            gate_c[q] = g.c_prev[(size_t)m * g.H + hu];
        }
    }

    if constexpr (PIPE) {
        // Unchecked kernel: every instruction that is not an MFMA has to run in the shadow of the MFMAs (vector
        // ALU instructions in particular take issue time from the matrix pipe, measured ~6 cycles each). The loads of slab i+2, the
        // LDS writes of slab i+1 and the operand reads of the next k-group are placed between the MFMAs of
        // slab i, one piece per MFMA, and pinned there. The workgroup barrier sits in the middle of the slab,
        // after the writes of slab i+1: the operands of the k-groups behind it were read in front of it, and
        // the first operands of slab i+1 are read during the last k-group of slab i, so no wave leaves the
        // barrier with nothing to feed the matrix pipe. A wave that is past the barrier of slab i may write
        // slab i+2 while a slower one still reads slab i, hence more than two LDS buffers (four, so that buffer indices repeat with the unrolled loop). Addresses are a
        // wave-uniform base pointer that advances per slab plus a per-thread 32-bit byte offset that never
        // changes (no vector address arithmetic in the loop). The steady-state loop has no branch around a
        // load, so the wait for the registers of slab i+1 can leave the four younger loads of slab i+2 in
        // flight; the last slabs are peeled into branch-free copies for the same reason.
        unsigned a_off[A_F4], b_off[B_F4];
        const char* ap = nullptr;
        const char* bp = nullptr;
        long a_step = 0, b_step = 0;
        int fj = s_begin;  // next flat slab to fetch
        // both segments share their leading dimensions here (the launcher checks it), so the offsets and the
        // per-slab steps are loop constants and a segment switch only replaces the two base pointers
        const int lda = g.seg[0].lda, ldb = g.seg[0].ldb;
#pragma unroll
        for (int t = 0; t < A_F4; ++t) a_off[t] = (unsigned)(((size_t)a_r[t] * lda + a_c[t]) * sizeof(float));
#pragma unroll
        for (int t = 0; t < B_F4; ++t) b_off[t] = (unsigned)(((size_t)b_r[t] * ldb + b_c[t]) * sizeof(float));
        a_step = (TA ? (long)BK * lda : (long)BK) * (long)sizeof(float);
        b_step = (TB ? (long)BK : (long)BK * ldb) * (long)sizeof(float);
        // Segment bases and slab counts are read into (scalar) registers here, once: a kernel-argument load inside the
        // main loop would share its wait counter with the LDS operand reads and stall the pipeline at every switch.
        const char* seg_a[MAXSEG];
        const char* seg_b[MAXSEG];
        int seg_slabs[MAXSEG];
#pragma unroll
        for (int q = 0; q < MAXSEG; ++q) {
            const bool used = q < g.nseg;
            seg_a[q] = used ? (const char*)g.seg[q].A : nullptr;
            seg_b[q] = used ? (const char*)g.seg[q].B : nullptr;
            seg_slabs[q] = used ? (g.seg[q].K + BK - 1) / BK : 0;
        }
        const int nseg = g.nseg;
        int seg_i = 0, seg_end = seg_slabs[0];  // current segment and the flat slab index behind its last slab
        ap = seg_a[0];
        bp = seg_b[0];
#pragma unroll
        for (int q = 1; q < MAXSEG; ++q)
            if (q < nseg && s_begin >= seg_end) {
                seg_i = q;
                ap = seg_a[q];
                bp = seg_b[q];
                seg_end += seg_slabs[q];
            }
        {
            int cur_slabs = seg_slabs[0];
#pragma unroll
            for (int q = 1; q < MAXSEG; ++q) cur_slabs = seg_i == q ? seg_slabs[q] : cur_slabs;
            const int local_slab = s_begin - (seg_end - cur_slabs);
            ap += (long)local_slab * a_step;
            bp += (long)local_slab * b_step;
        }
        auto fetchA = [&](auto S) __attribute__((always_inline)) {
#pragma unroll
            for (int t = 0; t < A_F4; ++t) ra[decltype(S)::value][t] = ld16(ap + a_off[t]);
        };
        auto fetchB = [&](auto S) __attribute__((always_inline)) {
#pragma unroll
            for (int t = 0; t < B_F4; ++t) rb[decltype(S)::value][t] = ld16(bp + b_off[t]);
        };
        auto advance = [&]() __attribute__((always_inline)) {
            ++fj;
            ap += a_step;
            bp += b_step;
            if constexpr (MAXSEG == 2) {
                // two terms: one compare and two pointer selects
                if (fj == seg_slabs[0] && seg_slabs[1] > 0) {
                    ap = seg_a[1];
                    bp = seg_b[1];
                }
            } else {
                if (fj == seg_end && seg_i + 1 < nseg) {
                    ++seg_i;
#pragma unroll
                    for (int q = 1; q < MAXSEG; ++q)
                        if (seg_i == q) {
                            ap = seg_a[q];
                            bp = seg_b[q];
                            seg_end += seg_slabs[q];
                        }
                }
            }
        };
        float4 a4[2][TM];
        float b[2][TN][4];
        // the TM x TN MFMAs of one k (two k, one per half-wave) of the current k-group
        auto mfma = [&](int o, int c) __attribute__((always_inline)) {
#pragma unroll
            for (int ii = 0; ii < TM; ++ii) {
                const float a = c == 0 ? a4[o][ii].x : (c == 1 ? a4[o][ii].y : (c == 2 ? a4[o][ii].z : a4[o][ii].w));
#pragma unroll
                for (int jj = 0; jj < TN; ++jj) {
                    const int ch = CHAINS == 2 ? (c & 1) : 0;
                    acc[ch][ii][jj] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b[o][jj][c], acc[ch][ii][jj], 0, 0, 0);
                }
            }
        };
        // P: position of the step in the unrolled loop; it fixes the register stage (P % 2) and the LDS
        // buffers (slab i in P % NBUF, slab i+1 in the next one) at compile time.
        auto slab_step = [&](auto P, auto H1, auto H2) __attribute__((always_inline)) {
            constexpr int ST = decltype(P)::value % 2;
            constexpr int cur = decltype(P)::value % NBUF, nxt = (decltype(P)::value + 1) % NBUF;
            constexpr bool has1 = decltype(H1)::value, has2 = decltype(H2)::value;
            using S = std::integral_constant<int, ST>;
            using NX = std::integral_constant<int, ST ^ 1>;
            constexpr int WT = MIDB ? G / 2 - 1 : G - 1;  // k-group that carries the LDS writes and the barrier
#pragma unroll
            for (int tt = 0; tt < G; ++tt) {
                const int o = tt & 1;
                mfma(o, 0);
                if (tt + 1 < G)
                    load_ops(cur, (tt + 1) * KW + kw, a4[o ^ 1], b[o ^ 1]);
                else if (has1 && MIDB)
                    load_ops(nxt, kw, a4[0], b[0]);  // G is even: the last group used a4[1] / b[1]
                __builtin_amdgcn_sched_barrier(0);
                mfma(o, 1);
                if (has2 && tt == 0) fetchA(S{});
                if (has1 && tt == WT) stageA(NX{}, nxt);
                __builtin_amdgcn_sched_barrier(0);
                mfma(o, 2);
                if (has2 && tt == 0) fetchB(S{});
                if (has1 && tt == WT) stageB(NX{}, nxt);
                __builtin_amdgcn_sched_barrier(0);
                mfma(o, 3);
                __builtin_amdgcn_sched_barrier(0);
                if (tt == WT) {
                    if (has2) advance();
                    if (has1) __syncthreads();
                }
            }
            if (has1 && !MIDB) load_ops(nxt, kw, a4[0], b[0]);
        };
        constexpr int U = NBUF;  // steps per trip of the unrolled loop (even)
        // the last `r` slabs, r <= U + 1, starting at position 0
        auto tail_step = [&](auto J, auto R) __attribute__((always_inline)) {
            constexpr int j = decltype(J)::value, r = decltype(R)::value;
            if constexpr (j < r)
                slab_step(std::integral_constant<int, j % U>{}, std::integral_constant<bool, (j + 1 < r)>{},
                          std::integral_constant<bool, (j + 2 < r)>{});
        };
        auto run_tail = [&](auto R) __attribute__((always_inline)) {
            tail_step(std::integral_constant<int, 0>{}, R);
            tail_step(std::integral_constant<int, 1>{}, R);
            tail_step(std::integral_constant<int, 2>{}, R);
            tail_step(std::integral_constant<int, 3>{}, R);
            tail_step(std::integral_constant<int, 4>{}, R);
        };
        static_assert(U + 1 <= 5, "run_tail covers five steps");
        using S0 = std::integral_constant<int, 0>;
        using S1 = std::integral_constant<int, 1>;
        using Yes = std::true_type;
        if (nslab > 0) {
            fetchA(S0{});
            fetchB(S0{});
            advance();
            if (nslab > 1) {
                fetchA(S1{});
                fetchB(S1{});
                advance();
            }
            stage(S0{}, 0);
            __syncthreads();
            load_ops(0, kw, a4[0], b[0]);
            int i = 0;
            for (; i + U + 1 < nslab; i += U) {
                slab_step(std::integral_constant<int, 0>{}, Yes{}, Yes{});
                slab_step(std::integral_constant<int, 1>{}, Yes{}, Yes{});
                if constexpr (U > 2) {
                    slab_step(std::integral_constant<int, 2>{}, Yes{}, Yes{});
                    slab_step(std::integral_constant<int, 3>{}, Yes{}, Yes{});
                }
            }
            const int rest = nslab - i;  // 1 .. U + 1
            if (rest == 1) run_tail(std::integral_constant<int, 1>{});
            else if (rest == 2) run_tail(std::integral_constant<int, 2>{});
            else if (rest == 3) run_tail(std::integral_constant<int, 3>{});
            else if (U > 2 && rest == 4) run_tail(std::integral_constant<int, (U > 2 ? 4 : 1)>{});
            else if (U > 2 && rest == 5) run_tail(std::integral_constant<int, (U > 2 ? 5 : 1)>{});
        }
    } else {
        // prologue: slabs 0 .. DEPTH-1 in flight, slab 0 staged
        auto for_stages = [&](auto f) __attribute__((always_inline)) {
            f(std::integral_constant<int, 0>{});
            if constexpr (DEPTH > 1) f(std::integral_constant<int, 1>{});
            if constexpr (DEPTH > 2) f(std::integral_constant<int, 2>{});
            if constexpr (DEPTH > 3) f(std::integral_constant<int, 3>{});
        };
        for_stages([&](auto S) __attribute__((always_inline)) {
            if (decltype(S)::value < nslab) fetch(S, s_begin + decltype(S)::value);
        });
        if (nslab > 0) stage(std::integral_constant<int, 0>{}, 0);
        __syncthreads();

        // slab i lives in register stage i % DEPTH until it is staged; the loop is
        // unrolled DEPTH times so that the stage index is a compile-time constant
        for (int base = 0; base < nslab; base += DEPTH) {
            for_stages([&](auto S) __attribute__((always_inline)) {
                constexpr int st = decltype(S)::value;
                const int i = base + st;
                if (i < nslab) {
                    const int cur = i & 1;
                    // stage slab i+1 (already in registers) into the other buffer, then reuse
                    // the registers slab i occupied for slab i+DEPTH
                    if (i + 1 < nslab) stage(std::integral_constant<int, (st + 1) % DEPTH>{}, cur ^ 1);
                    if (i + DEPTH < nslab) fetch(S, s_begin + i + DEPTH);
                    compute(cur);
                    __syncthreads();
                }
            });
        }
    }

    if (CHAINS == 2) {
#pragma unroll
        for (int ii = 0; ii < TM; ++ii)
#pragma unroll
            for (int jj = 0; jj < TN; ++jj) acc[0][ii][jj] += acc[CHAINS - 1][ii][jj];
    }
    if (KW > 1) {
        // wave sets 1.. hand their accumulators to set 0 through LDS (the slab buffers are free now)
        float* red = lds;
        __syncthreads();  // the last slab's operand reads are done in every wave
        if (kw > 0) {
#pragma unroll
            for (int ii = 0; ii < TM; ++ii)
#pragma unroll
                for (int jj = 0; jj < TN; ++jj)
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        red[(size_t)(kw - 1) * BM * BN + ((wave * TM + ii) * TN + jj) * 1024 + v * 64 + lane] = acc[0][ii][jj][v];
        }
        __syncthreads();
        if (kw > 0 && !GATES) return;  // with the gate epilogue the other wave sets stay to share its arithmetic
        if (kw == 0)
#pragma unroll
        for (int s2 = 1; s2 < KW; ++s2)
#pragma unroll
            for (int ii = 0; ii < TM; ++ii)
#pragma unroll
                for (int jj = 0; jj < TN; ++jj)
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        acc[0][ii][jj][v] += red[(size_t)(s2 - 1) * BM * BN + ((wave * TM + ii) * TN + jj) * 1024 + v * 64 + lane];
    }
    if constexpr (GATES) {
        // The sums go to LDS as a [BM][BN] tile of pre-activations (behind the fold area), then every thread of
        // the workgroup finishes its (row, hidden unit) pairs: gate = pre + bias, i / f / o = sigmoid, g = tanh,
        // c' = f * c + i * g, h' = o * tanh(c'), each operation rounded on its own like the generated gate kernel
        // (dali/layers/lstm.cpp:238-261). Bias and previous cell values were fetched before the main loop.
        static_assert(BM == 64 && BN == 64 && TM * TN == 1, "gate epilogue is written for the 64x64 tile");
        static_assert(LDS_FLOATS >= RED_FLOATS + BM * BN, "no room for the pre-activation tile");
        float* tile = lds + RED_FLOATS;
        if (kw == 0) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int lm = wm * WTM + 8 * (v / 4) + 4 * h + (v % 4), ln = wn * WTN + l32;
                tile[lm * BN + ln] = acc[0][0][0][v];
            }
        }
        __syncthreads();
        const int H = g.H;
#pragma unroll
        for (int q = 0; q < GATE_PAIRS; ++q) {
#pragma clang fp contract(off)
            const int e = tid + q * THREADS, r = e / 16, j = e % 16, m = m0 + r;
            if (m >= M) continue;
            const float gi = tile[r * BN + j] + gate_bias[q][0];
            const float gf = tile[r * BN + 16 + j] + gate_bias[q][1];
            const float go = tile[r * BN + 32 + j] + gate_bias[q][2];
            const float gg = tile[r * BN + 48 + j] + gate_bias[q][3];
            const float iv = (float)(1.0 / (1.0 + (double)gate_expf(-gi)));
            const float fv = (float)(1.0 / (1.0 + (double)gate_expf(-gf)));
            const float ov = (float)(1.0 / (1.0 + (double)gate_expf(-go)));
            const float gv = tanhf(gg);
            const float fc = fv * gate_c[q];
            const float ig = iv * gv;
            const float cn = fc + ig;
            const size_t o = (size_t)m * H + hu_base + j;
            g.c_out[o] = cn;
            g.h_out[o] = ov * tanhf(cn);
        }
        return;
    }
    // epilogue: lane holds column l32 and rows 8*(v/4) + 4*h + v%4 of each 32x32 tile
    const float alpha = g.alpha, beta = g.beta;
    const bool split = gridDim.z > 1;
    float* part = nullptr;
    const int tile_id = blockIdx.y * gridDim.x + blockIdx.x;
    if (split) {
        // every share publishes its partial tile (agent-scope stores, no cache-wide fence); the
        // workgroup that draws the last ticket folds all shares in z order, so the sum does not
        // depend on which share finished last
        part = g.partials + (size_t)tile_id * gridDim.z * (BM * BN);
        float* mine = part + (size_t)blockIdx.z * (BM * BN);
#pragma unroll
        for (int ii = 0; ii < TM; ++ii)
#pragma unroll
            for (int jj = 0; jj < TN; ++jj)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    int lm = wm * WTM + ii * 32 + 8 * (v / 4) + 4 * h + (v % 4), ln = wn * WTN + jj * 32 + l32;
                    publish(mine + lm * BN + ln, acc[0][ii][jj][v]);
                }
        // the partial tile is acknowledged by memory before the ticket is drawn; the clobber keeps the compiler from moving the stores
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __shared__ int is_last;
        __syncthreads();
        if (tid == 0) {
            unsigned int ticket = __hip_atomic_fetch_add(g.counters + tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            is_last = ticket == gridDim.z - 1;
        }
        __syncthreads();
        if (!is_last) return;
        // The fold: shares in z order per element, but the loads of four shares x sixteen elements are issued before
        // the first of them is awaited (one awaited load per share and element cost ~270 ns each: 128 shares of a lone
        // 64x64 tile took 550 us to fold).
        constexpr int ZB = 4;
#pragma unroll
        for (int ii = 0; ii < TM; ++ii)
#pragma unroll
            for (int jj = 0; jj < TN; ++jj) {
                const int ln = wn * WTN + jj * 32 + l32;
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[0][ii][jj][v] = 0.f;
                for (unsigned z0 = 0; z0 < gridDim.z; z0 += ZB) {
                    float t[ZB][16];
#pragma unroll
                    for (int u = 0; u < ZB; ++u) {
                        const bool on = z0 + u < gridDim.z;
                        const float* src = part + (size_t)(on ? z0 + u : z0) * (BM * BN);
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int lm = wm * WTM + ii * 32 + 8 * (v / 4) + 4 * h + (v % 4);
                            t[u][v] = observe(src + lm * BN + ln);
                        }
                    }
#pragma unroll
                    for (int u = 0; u < ZB; ++u)
                        if (z0 + u < gridDim.z) {
#pragma unroll
                            for (int v = 0; v < 16; ++v) acc[0][ii][jj][v] += t[u][v];
                        }
                }
            }
    }
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
                    size_t out_row = (size_t)m;
                    if (MAXSEG > 2 && g.map_on) {  // only the multi-term kernels carry the map
                        const unsigned img = row_map_div((unsigned)m, g.map_hw_m, g.map_hw_s), rest = (unsigned)m - img * g.map_hw;
                        const unsigned i = row_map_div(rest, g.map_w_m, g.map_w_s), j = rest - i * g.map_w;
                        if ((int)i >= g.map_oh || (int)j >= g.map_ow) continue;
                        out_row = ((size_t)img * g.map_oh + i) * g.map_ow + j;
                    }
                    float* c = g.C + out_row * g.ldc + n;
                    const float sum = acc[0][ii][jj][v];  // (with split-K: the fold above)
                    float r = alpha * sum;
                    if (beta != 0.f) r += beta * *c;
                    *c = r;
                }
            }
        }
    if (split && tid == 0) __hip_atomic_store(g.counters + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int BM, int BN, int BK, int DEPTH, int KW = 1, bool MIDB = false>
static int launch_tile(GemmArgs g, bool ta, bool tb, bool vec, int split_k, bool edge) {
    if (KW > 1) split_k = 1;  // the wave-set fold and the cross-workgroup fold are alternatives
    if (!vec) edge = true;
    dim3 grid((g.N + BN - 1) / BN, (g.M + BM - 1) / BM);
    int nslab = 0;
    for (int s = 0; s < g.nseg; ++s) nslab += (g.seg[s].K + BK - 1) / BK;
    size_t tiles = (size_t)grid.x * grid.y;
    if (split_k > nslab) split_k = nslab > 0 ? nslab : 1;
    if (split_k > 1 && (tiles > (size_t)kWorkspaceCounters || tiles * split_k * BM * BN * sizeof(float) > kWorkspacePartialBytes)) split_k = 1;
    grid.z = split_k;
    g.counters = (unsigned int*)workspace();
    g.partials = (float*)(workspace() + kWorkspaceCounterBytes);
    dim3 block(256 * KW);
    hipStream_t st = stream();
    static const int pad_env = getenv("DALI_HIP_GEMM_PAD_LDS") ? atoi(getenv("DALI_HIP_GEMM_PAD_LDS")) : 0;
    const unsigned pad_lds = (unsigned)pad_env;
#define DALI_GEMM_CASE(TA_, TB_, V_)                                                                        \
    if (ta == TA_ && tb == TB_ && vec == V_) {                                                              \
        if (edge)                                                                                           \
            hipLaunchKernelGGL((sgemm_kernel<BM, BN, BK, TA_, TB_, V_, DEPTH, true, KW, false>), grid, block, pad_lds, st, g);  \
        else if (V_)                                                                                        \
            hipLaunchKernelGGL((sgemm_kernel<BM, BN, BK, TA_, TB_, true, DEPTH, false, KW, MIDB>), grid, block, pad_lds, st, g); \
    }
#define DALI_GEMM_CASE_TERMS(TB_, V_)                                                                       \
    if (tb == TB_ && vec == V_) {                                                                           \
        if (edge)                                                                                           \
            hipLaunchKernelGGL((sgemm_kernel<BM, BN, BK, false, TB_, V_, DEPTH, true, KW, false, false, kMaxSeg>), grid, block, pad_lds, st, g);  \
        else if (V_)                                                                                        \
            hipLaunchKernelGGL((sgemm_kernel<BM, BN, BK, false, TB_, true, DEPTH, false, KW, MIDB, false, kMaxSeg>), grid, block, pad_lds, st, g); \
    }
    if (g.nseg > 2 || g.map_on) {
        if (ta) return fail("sgemm: more than two terms, or an output row map, need a left operand stored by rows");
        DALI_GEMM_CASE_TERMS(false, true)
        DALI_GEMM_CASE_TERMS(false, false)
        DALI_GEMM_CASE_TERMS(true, true)
        DALI_GEMM_CASE_TERMS(true, false)
        hipError_t e2 = hipGetLastError();
        if (e2 != hipSuccess) return fail("sgemm launch failed: %s", hipGetErrorString(e2));
        return DALI_HIP_OK;
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
#undef DALI_GEMM_CASE_TERMS
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("sgemm launch failed: %s", hipGetErrorString(e));
    return DALI_HIP_OK;
}

// One product on one tile configuration. When the operands allow the unchecked kernel (16-byte aligned rows,
// whole 4-column granules along M / N where a granule runs along them, offsets that fit 32 bits, one pair of
// leading dimensions), the whole slabs of every segment go through it, whatever M and N are; what is left of
// K (less than one slab per segment) is added by a second, checked launch with beta = 1.
template <int BM, int BN, int BK, int DEPTH, int KW = 1, bool MIDB = false>
static int run_tile(const GemmArgs& g, bool ta, bool tb, bool vec, int split_k) {
    bool fast = vec && g.nseg > 0 && (!ta || g.M % 4 == 0) && (tb || g.N % 4 == 0);
    bool same_ld = true;  // the register-staged kernel takes one pair of leading dimensions, the other one a pair per term
    for (int s = 0; s < g.nseg && fast; ++s) {
        const size_t a_span = ((size_t)(ta ? BK : g.M) * g.seg[s].lda + (ta ? g.M : BK)) * sizeof(float);
        const size_t b_span = ((size_t)(tb ? g.N : BK) * g.seg[s].ldb + (tb ? BK : g.N)) * sizeof(float);
        fast = fast && a_span < ((size_t)1 << 32) && b_span < ((size_t)1 << 32);
        same_ld = same_ld && g.seg[s].lda == g.seg[0].lda && g.seg[s].ldb == g.seg[0].ldb;
    }
    constexpr bool dma_tile = BM == 64 && BN == 64 && BK == 64 && KW == 2 && !MIDB;
    if (!fast || (!same_ld && !(dma_tile && split_k == 1 && g.nseg <= 2 && !g.map_on))) return launch_tile<BM, BN, BK, DEPTH, KW, MIDB>(g, ta, tb, vec, split_k, true);
    if (dma_tile && split_k == 1 && g.nseg <= 2 && !g.map_on) {
        // inner extents that end in a partly filled slab: the same kernel fills what is missing with zeros as the slab arrives,
        // instead of a second launch for the rest ([256,1000].[1000,4000] twice: 47.7 -> 38 us)
        bool partly = false;
        for (int s = 0; s < g.nseg; ++s) partly = partly || g.seg[s].K % BK != 0;
        if (partly) {
            const float* as[2] = {g.seg[0].A, g.seg[1].A};
            const float* bs[2] = {g.seg[0].B, g.seg[1].B};
            const int ks[2] = {g.seg[0].K, g.seg[1].K};
            const int las[2] = {g.seg[0].lda, g.seg[1].lda}, lbs[2] = {g.seg[0].ldb, g.seg[1].ldb};
            const int r = sgemm_dma(ta, tb, g.M, g.N, g.nseg, ks, as, bs, las, lbs, g.alpha, g.beta, g.C, g.ldc, nullptr, nullptr, nullptr, nullptr, 0);
            if (r < 0) return DALI_HIP_ERROR;
            if (r > 0) return DALI_HIP_OK;
        }
    }
    GemmArgs whole = g, rest = g;
    whole.nseg = rest.nseg = 0;
    for (int s = 0; s < g.nseg; ++s) {
        const GemmSeg& sg = g.seg[s];
        const int kw = sg.K / BK * BK, kr = sg.K - kw;
        if (kw > 0) {
            GemmSeg& d = whole.seg[whole.nseg++];
            d = sg;
            d.K = kw;
        }
        if (kr > 0) {
            GemmSeg& d = rest.seg[rest.nseg++];
            d = sg;
            d.A = sg.A + (ta ? (size_t)kw * sg.lda : (size_t)kw);
            d.B = sg.B + (tb ? (size_t)kw : (size_t)kw * sg.ldb);
            d.K = kr;
        }
    }
    if (whole.nseg > 0) {
        int st = 0;
        bool done = false;
        if (dma_tile && split_k == 1 && whole.nseg <= 2 && !whole.map_on) {
            // small grids of whole slabs: the kernel that has its operand slabs written into LDS by the loads themselves
            const float* as[2] = {whole.seg[0].A, whole.seg[1].A};
            const float* bs[2] = {whole.seg[0].B, whole.seg[1].B};
            const int ks[2] = {whole.seg[0].K, whole.seg[1].K};
            const int las[2] = {whole.seg[0].lda, whole.seg[1].lda}, lbs[2] = {whole.seg[0].ldb, whole.seg[1].ldb};
            const int r = sgemm_dma(ta, tb, whole.M, whole.N, whole.nseg, ks, as, bs, las, lbs, whole.alpha, whole.beta,
                                    whole.C, whole.ldc, nullptr, nullptr, nullptr, nullptr, 0);
            if (r < 0) return DALI_HIP_ERROR;
            done = r > 0;
        }
        // (terms with rows of different lengths that the kernel above did not take: everything through the guarded kernel)
        if (!done && !same_ld) return launch_tile<BM, BN, BK, DEPTH, KW, MIDB>(g, ta, tb, vec, split_k, true);
        if (!done) st = launch_tile<BM, BN, BK, DEPTH, KW, MIDB>(whole, ta, tb, true, split_k, false);
        if (st || rest.nseg == 0) return st;
        rest.beta = 1.0f;
    }
    return launch_tile<BM, BN, BK, DEPTH, KW, MIDB>(rest, ta, tb, true, 1, true);
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// compute units of the bound device (0 when they cannot be read)
static int device_cus() {
    static int cus = -1;
    if (cus < 0) {
        int v = 0;
        cus = hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, bound_device()) == hipSuccess ? v : 0;
    }
    return cus;
}

// shares of the inner extent (64-deep slabs) for a product of `tiles64` 64x64 tiles that leaves compute units idle: one work
// item per compute unit, at least four slabs each; below 2 the product is not cut
static int stream_shares(long tiles64, int nslab64) {
    const int cus = device_cus();
    if (cus <= 0 || tiles64 <= 0 || tiles64 >= cus || nslab64 < 8) return 1;
    // Estimated time in units of one slab (about 1.1 us): rounds x (slabs of a share + what a cut costs: publishing the share,
    // the ticket and the fetch by whoever adds the shares up, 5 slab times and 0.15 more per share; measured on [64,64] over
    // K = 65536 and on the LSTM shapes). The cut has to win a tenth to be made.
    const int most = nslab64 / 4 < 256 ? nslab64 / 4 : 256;
    int best = 1;
    double best_time = (double)nslab64;
    for (int sh = 2; sh <= most; ++sh) {
        const long items = tiles64 * sh;
        if (items > 2048) break;  // 16 KiB of partial sums each in the 32 MiB workspace
        const long rounds = (items + cus - 1) / cus;
        const double t = (double)rounds * ((double)nslab64 / sh + 5.0 + 0.15 * sh);
        if (t < best_time) {
            best = sh;
            best_time = t;
        }
    }
    return best_time <= 0.9 * nslab64 ? best : 1;
}

// The whole slabs of a product of one or two terms through the streaming kernel, what is left of the inner extents by a
// checked launch that adds to the result. -1: not a case for it (nothing was launched).
static int stream_product(const GemmArgs& g, bool ta, bool tb, int shares) {
    GemmArgs whole = g, rest = g;
    whole.nseg = rest.nseg = 0;
    for (int s = 0; s < g.nseg; ++s) {
        const GemmSeg& sg = g.seg[s];
        const int kw = sg.K / 64 * 64, kr = sg.K - kw;
        if (kw > 0) {
            GemmSeg& d = whole.seg[whole.nseg++];
            d = sg;
            d.K = kw;
        }
        if (kr > 0) {
            GemmSeg& d = rest.seg[rest.nseg++];
            d = sg;
            d.A = sg.A + (ta ? (size_t)kw * sg.lda : (size_t)kw);
            d.B = sg.B + (tb ? (size_t)kw : (size_t)kw * sg.ldb);
            d.K = kr;
        }
    }
    if (whole.nseg == 0) return -1;
    const float* as[2] = {whole.seg[0].A, whole.seg[1].A};
    const float* bs[2] = {whole.seg[0].B, whole.seg[1].B};
    const int ks[2] = {whole.seg[0].K, whole.seg[1].K};
    const int cus = device_cus();
    if (cus <= 0) return -1;
    const int las[2] = {whole.seg[0].lda, whole.seg[1].lda}, lbs[2] = {whole.seg[0].ldb, whole.seg[1].ldb};
    const int r = sgemm_dma_stream(ta, tb, whole.M, whole.N, whole.nseg, ks, as, bs, las, lbs, whole.alpha, whole.beta, whole.C,
                                   whole.ldc, shares, cus);
    if (r < 0) return DALI_HIP_ERROR;
    if (r == 0) return -1;
    if (rest.nseg == 0) return DALI_HIP_OK;
    rest.beta = 1.0f;
    return launch_tile<64, 64, 64, 2, 2, false>(rest, ta, tb, true, 1, true);
}

// Many 128x128 tiles of a single product: the whole 32-deep slabs through the kernel that walks a list of tiles per compute
// unit, what is left of the inner extent by a checked launch that adds to the result. -1: not a case for it.
static int tiles128_product(const GemmArgs& g, bool ta, bool tb) {
    const GemmSeg& sg = g.seg[0];
    const int cus = device_cus();
    if (cus <= 0) return -1;
    if (sg.K % 32 != 0 && sg.K % 4 == 0 && sg.K > 32) {
        // the kernel fills a partly filled last slab with zeros as it arrives (no second launch for the rest)
        const int r = sgemm_dma128(ta, tb, g.M, g.N, sg.K, sg.A, sg.lda, sg.B, sg.ldb, g.alpha, g.beta, g.C, g.ldc, cus);
        if (r < 0) return DALI_HIP_ERROR;
        if (r > 0) return DALI_HIP_OK;
    }
    const int kw = sg.K / 32 * 32, kr = sg.K - kw;
    if (kw == 0) return -1;
    const int r = sgemm_dma128(ta, tb, g.M, g.N, kw, sg.A, sg.lda, sg.B, sg.ldb, g.alpha, g.beta, g.C, g.ldc, cus);
    if (r < 0) return DALI_HIP_ERROR;
    if (r == 0) return -1;
    if (kr == 0) return DALI_HIP_OK;
    GemmArgs rest = g;
    rest.seg[0].A = sg.A + (ta ? (size_t)kw * sg.lda : (size_t)kw);
    rest.seg[0].B = sg.B + (tb ? (size_t)kw : (size_t)kw * sg.ldb);
    rest.seg[0].K = kr;
    rest.beta = 1.0f;
    return launch_tile<128, 128, 32, 2>(rest, ta, tb, true, 1, true);
}

// Row-major driver: C[M,N] = alpha * sum_s opA_s * opB_s + beta * C.
// ta: A_s is stored as [K][M]; tb: B_s is stored as [N][K].
static int sgemm_rowmajor(int nseg, bool ta, bool tb, int M, int N, const int* K, const float* const* A,
                          const int* lda, const float* const* B, const int* ldb, float alpha, float beta, float* C,
                          int ldc, bool rows_may_overlap = false, const int* row_map = nullptr) {
    if (ensure_init()) return DALI_HIP_ERROR;
    if (M < 0 || N < 0) return fail("sgemm: negative extent (M=%d, N=%d)", M, N);
    if (M == 0 || N == 0) return DALI_HIP_OK;
    if (!C) return fail("sgemm: C is NULL");
    if (ldc < N) return fail("sgemm: ldc=%d smaller than row length %d", ldc, N);
    if (nseg > kMaxSeg) return fail("sgemm: %d terms exceed the limit of %d", nseg, kMaxSeg);
    GemmArgs g = {};
    g.nseg = 0;
    bool vec = true;
    for (int s = 0; s < nseg; ++s) {
        if (K[s] < 0) return fail("sgemm: negative inner extent %d", K[s]);
        if (K[s] == 0) continue;
        if (!A[s] || !B[s]) return fail("sgemm: operand %d is NULL", s);
        int a_row = ta ? M : K[s], b_row = tb ? K[s] : N;
        if (lda[s] < a_row && !(rows_may_overlap && !ta && lda[s] >= 1)) return fail("sgemm: leading dimension %d of the left operand is smaller than its row length %d", lda[s], a_row);
        if (ldb[s] < b_row) return fail("sgemm: leading dimension %d of the right operand is smaller than its row length %d", ldb[s], b_row);
        GemmSeg& sg = g.seg[g.nseg++];
        sg.A = A[s];
        sg.B = B[s];
        sg.lda = lda[s];
        sg.ldb = ldb[s];
        sg.K = K[s];
        (void)aligned16;  // the vector kernels no longer need 16-byte aligned rows
    }
    g.M = M;
    g.N = N;
    g.C = C;
    g.ldc = ldc;
    g.alpha = alpha;
    g.beta = beta;
    if (row_map) {
        const int map_h = row_map[0], map_w = row_map[1];
        if (map_h < 1 || map_w < 1 || row_map[2] < 1 || row_map[3] < 1 || row_map[2] > map_h || row_map[3] > map_w || M % (map_h * map_w) != 0)
            return fail("sgemm: bad output row map [%d x %d] -> [%d x %d] for %d rows", map_h, map_w, row_map[2], row_map[3], M);
        auto set_div = [](unsigned d, unsigned* m, int* sh) {
            int sft = 0;
            while (((unsigned long long)1 << sft) < d) ++sft;
            *m = (unsigned)((((unsigned long long)1 << (31 + sft)) + d - 1) / d);
            *sh = sft;
        };
        g.map_on = 1;
        g.map_hw = (unsigned)(map_h * map_w);
        g.map_w = (unsigned)map_w;
        set_div(g.map_hw, &g.map_hw_m, &g.map_hw_s);
        set_div(g.map_w, &g.map_w_m, &g.map_w_s);
        g.map_oh = row_map[2];
        g.map_ow = row_map[3];
    }
    if (g.nseg == 0) {
        // empty inner extent: C = beta * C
        g.nseg = 1;
        g.seg[0].K = 0;
        vec = false;
    }
    // More than `low_rows_from` and at most 64 rows against a wide B stored [K][N]: bound by the matrix pipe rather than by
    // streaming B, so 64-row tiles fed through LDS, one workgroup per compute unit ([64,1024].[1024,32000]: 45 -> 41 us, 0.65 of the fp32 matrix peak; the row-streaming
    // kernel takes 26 us at 32 rows and grows with the rows, this one takes 38 to 41 us whatever they are)
    static const int low_rows_from = getenv("DALI_HIP_GEMM_LOW_ROWS") ? atoi(getenv("DALI_HIP_GEMM_LOW_ROWS")) : 52;
    if (g.nseg == 1 && vec && !ta && !tb && !row_map && !rows_may_overlap && M > low_rows_from && M <= 64 && N >= 8192 && g.seg[0].K >= 256) {
        const int st = tiles128_product(g, false, false);
        if (st >= 0) return st;
    }
    static const int gemv_on = getenv("DALI_HIP_GEMV") ? atoi(getenv("DALI_HIP_GEMV")) : 1;
    if (gemv_on && g.nseg >= 1 && g.nseg <= 2 && g.seg[0].K > 0 && !ta && !tb && !row_map && !rows_may_overlap && N % 4 != 0 && N >= 1024 && M > 64) {
        // A wide row-major B whose row length is no multiple of four (a vocabulary of 50257 words): the kernels that take whole
        // 16-byte granules along N serve the columns up to the last multiple of four, and the one to three columns left over
        // are matrix-vector products ([256,1024].[1024,50257]: 334 -> 289 us; the guarded kernel would serve all of it; up to 64 rows the
        // row-streaming kernel below takes any N)
        const int N4 = N & ~3;
        const float* as[kMaxSeg];
        const float* bs[kMaxSeg];
        int ks[kMaxSeg], las[kMaxSeg], lbs[kMaxSeg];
        for (int s = 0; s < g.nseg; ++s) {
            as[s] = g.seg[s].A;
            bs[s] = g.seg[s].B;
            ks[s] = g.seg[s].K;
            las[s] = g.seg[s].lda;
            lbs[s] = g.seg[s].ldb;
        }
        const int st = sgemm_rowmajor(g.nseg, false, false, M, N4, ks, as, las, bs, lbs, alpha, beta, C, ldc);
        if (st != DALI_HIP_OK) return st;
        for (int j = N4; j < N; ++j)
            for (int s = 0; s < g.nseg; ++s) {
                const int r = sgemv_rows(M, ks[s], alpha, as[s], las[s], bs[s] + j, lbs[s], s == 0 ? beta : 1.0f, C + j, ldc);
                if (r < 0) return DALI_HIP_ERROR;
                if (r == 0) return fail("sgemm: the matrix-vector kernel refused column %d of a validated product", j);
            }
        return DALI_HIP_OK;
    }
    if (gemv_on && g.nseg == 1 && N == 1 && g.seg[0].K > 0 && !ta && !row_map && !rows_may_overlap && (M >= 64 || g.seg[0].K <= 65536)) {
        // a matrix times a column: the rows of A streamed once, each against the same vector
        const int st = sgemv_rows(M, g.seg[0].K, alpha, g.seg[0].A, g.seg[0].lda, g.seg[0].B, tb ? 1 : g.seg[0].ldb, beta, C, ldc);
        if (st != 0) return st > 0 ? DALI_HIP_OK : DALI_HIP_ERROR;
    }
    if (g.nseg == 1 && g.seg[0].K > 0 && !ta && !row_map && !rows_may_overlap && M <= 64) {
        // few rows against a wide right operand: stream it once instead of tiling it through LDS
        const int st = sgemm_skinny(tb, M, N, g.seg[0].K, alpha, g.seg[0].A, g.seg[0].lda, g.seg[0].B, g.seg[0].ldb, beta, C, ldc);
        if (st != 0) return st > 0 ? DALI_HIP_OK : DALI_HIP_ERROR;
    }
    if (g.nseg == 2 && !ta && !row_map && !rows_may_overlap && M <= 64) {
        // a sum of two such products (an LSTM's x.W + h.U at a small batch whose sizes the fused kernels do not take): the
        // first streams its right operand, the second adds to the result
        const int st = sgemm_skinny(tb, M, N, g.seg[0].K, alpha, g.seg[0].A, g.seg[0].lda, g.seg[0].B, g.seg[0].ldb, beta, C, ldc);
        if (st < 0) return DALI_HIP_ERROR;
        if (st > 0) {
            const int k1[1] = {g.seg[1].K}, lda1[1] = {g.seg[1].lda}, ldb1[1] = {g.seg[1].ldb};
            const float* a1[1] = {g.seg[1].A};
            const float* b1[1] = {g.seg[1].B};
            return sgemm_rowmajor(1, ta, tb, M, N, k1, a1, lda1, b1, ldb1, alpha, 1.0f, C, ldc);
        }
    }
    if (g.nseg == 1 && g.seg[0].K > 0 && g.seg[0].K <= 64 && !row_map && !rows_may_overlap) {
        // a short inner extent against a large result (the weight gradient of a layer at a small batch)
        const int st = sgemm_smallk(ta, tb, M, N, g.seg[0].K, alpha, g.seg[0].A, g.seg[0].lda, g.seg[0].B, g.seg[0].ldb, beta, C, ldc);
        if (st != 0) return st > 0 ? DALI_HIP_OK : DALI_HIP_ERROR;
    }
    long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128);
    static const int variant = getenv("DALI_HIP_GEMM_VARIANT") ? atoi(getenv("DALI_HIP_GEMM_VARIANT")) : 0;
    // >0: that many shares of the inner extent through the streaming kernel for every product it takes; <0: never
    static const int stream_env = getenv("DALI_HIP_GEMM_STREAM") ? atoi(getenv("DALI_HIP_GEMM_STREAM")) : 0;
    const bool stream_fits = vec && g.nseg <= 2 && !g.map_on && !rows_may_overlap;
    if (stream_env > 0 && stream_fits) {
        const int st = stream_product(g, ta, tb, stream_env);
        if (st >= 0) return st;
    }
    // From 64 tiles of 128x128 on, a long inner extent (2048 and more) also goes there when 64x64 tiles would leave a quarter of
    // the compute units idle in their last round: the 128x128 tiles are then cut into one share of the inner extent per compute
    // unit (1536x1536 over K = 4096: 200 -> 179 us, 768x1536: 130 -> 101 us).
    long tiles64_all = (long)((M + 63) / 64) * ((N + 63) / 64);
    const int cus_all = device_cus() > 0 ? device_cus() : 256;
    const long rounds64 = (tiles64_all + cus_all - 1) / cus_all;
    const bool uneven64 = tiles128 >= 64 && g.nseg == 1 && g.seg[0].K >= 2048 && (double)tiles64_all < 0.8 * (double)(rounds64 * cus_all);
    if (tiles128 >= 192 || uneven64) {
        if (vec && g.nseg == 1 && !g.map_on && !rows_may_overlap) {
            const int st = tiles128_product(g, ta, tb);
            if (st >= 0) return st;
        }
        if (tiles128 >= 192) return run_tile<128, 128, 32, 2>(g, ta, tb, vec, 1);
    }
    // Small grids: 64x64 tiles, and when even those leave CUs with a single workgroup, split K so
    // that two workgroups share a CU and one's barriers and memory waits hide behind the other's MFMAs.
    long tiles64 = (long)((M + 63) / 64) * ((N + 63) / 64);
    static const int split_env = getenv("DALI_HIP_GEMM_SPLITK") ? atoi(getenv("DALI_HIP_GEMM_SPLITK")) : 0;
    int split_k = split_env > 0 ? split_env : 1;
    {
        // a short inner extent that ends in a partly filled slab: one launch of the kernel that fills the slab up, rather than
        // shares of the whole slabs and a second launch for the rest ([256,300].[300,2048]: 17.0 -> 11 us)
        int nslab64 = 0;
        bool partly = false, pieces = true;
        for (int s = 0; s < g.nseg; ++s) {
            nslab64 += (g.seg[s].K + 63) / 64;
            partly = partly || g.seg[s].K % 64 != 0;
            pieces = pieces && g.seg[s].K % 4 == 0 && g.seg[s].K >= 64;
        }
        if (split_env == 0 && variant == 0 && stream_env == 0 && stream_fits && partly && pieces && nslab64 <= 16) return run_tile<64, 64, 64, 2, 2>(g, ta, tb, vec, 1);
    }
    if (split_env == 0 && variant == 0 && stream_env == 0 && stream_fits && tiles64 > 128) {
        // between half a round and a whole one of 64x64 tiles: shares that fill whole rounds (384x1536 over K = 4096, 144 tiles: 66 -> 58 us)
        int nslab64 = 0;
        for (int s = 0; s < g.nseg; ++s) nslab64 += (g.seg[s].K + 63) / 64;
        const int shares = stream_shares(tiles64, nslab64);
        if (shares >= 2) {
            const int st = stream_product(g, ta, tb, shares);
            if (st >= 0) return st;
        }
    }
    // (an inner extent of up to four slabs, or up to eight with a tile for half the compute units: nothing to share; one launch of the
    // kernel that loads into LDS takes [512,256].[256,1024] in 7.1 us against 9.5 us in two shares, [256,512].[512,2048] in 10.9 against 12.6)
    int nslab64_all = 0;
    for (int s = 0; s < g.nseg; ++s) nslab64_all += (g.seg[s].K + 63) / 64;
    const bool nothing_to_share = nslab64_all <= 4 || (tiles64 >= 128 && nslab64_all <= 8);
    if (split_env == 0 && variant == 0 && tiles64 <= 128 && !nothing_to_share) {
        // A few tiles over a long inner extent (the weight gradient of a convolution: [out, window] from tens of
        // thousands of patches) would leave most of the device idle: about two workgroups per CU, folded in a fixed
        // order by the workgroup that finishes last.
        int nslab64 = 0;
        for (int s = 0; s < g.nseg; ++s) nslab64 += (g.seg[s].K + 63) / 64;
        if (stream_env == 0 && stream_fits) {
            // one item per compute unit through the kernel whose loads write LDS themselves, in shares of at least four slabs
            // ([256,1024] over 32000: 145 us against 158 us, against 210 us with B stored as [N][K]; [64,64] over 65536:
            // 34 us against 65 us). A sum of two products is cut the same way as the fused LSTM step of its shape, whose
            // results it then matches bit for bit.
            const int shares = stream_shares(tiles64, nslab64);
            if (shares >= 2) {
                const int st = stream_product(g, ta, tb, shares);
                if (st >= 0) return st;
            }
        }
        const int want = (int)((512 + tiles64 - 1) / tiles64);
        // (shares of at least four slabs, two when there are no more than eight: [256,1024] over K = 1024 16.4 -> 12.9 us,
        // [100,512] over K = 512 12.4 -> 8.9 us against shares of at least eight; shorter shares lose to their fold)
        // A sum of several products keeps shares of eight: the LSTM pair over short inner extents then stays whole and
        // bit-equal to the fused step, which sums its slabs in one workgroup.
        const int min_slabs = g.nseg > 1 ? 8 : nslab64 <= 8 ? 2 : 4;
        const int share = nslab64 / min_slabs < want ? nslab64 / min_slabs : want;
        if (share >= 2) return run_tile<64, 64, 64, 2>(g, ta, tb, vec, share);
    }
    if (variant == 8) return run_tile<64, 64, 64, 2>(g, ta, tb, vec, split_k);
    if (variant == 5) return run_tile<64, 64, 64, 2, 2, true>(g, ta, tb, vec, split_k);
    if (variant == 9) return run_tile<64, 64, 64, 2, 4>(g, ta, tb, vec, split_k);
    // default for small grids: two wave sets per 64x64 tile (two waves per SIMD)
    return run_tile<64, 64, 64, 2, 2>(g, ta, tb, vec, split_k);
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

int dali_hip_sgemm_terms(int nterms, int transA, int transB, int M, int N, const int* K, const float* const* A, int lda,
                         const float* const* B, int ldb, float alpha, float beta, float* C, int ldc, const int* row_map) {
    if (nterms < 1 || nterms > kMaxSeg) return fail("dali_hip_sgemm_terms: between 1 and %d terms (got %d)", kMaxSeg, nterms);
    if (!K || !A || !B) return fail("dali_hip_sgemm_terms: NULL argument");
    if (M >= (1 << 30) / 2 * 2 && row_map) return fail("dali_hip_sgemm_terms: too many rows for a row map");
    int ldas[kMaxSeg], ldbs[kMaxSeg];
    for (int s = 0; s < nterms; ++s) {
        ldas[s] = lda;
        ldbs[s] = ldb;
    }
    return sgemm_rowmajor(nterms, transA != 0, transB != 0, M, N, K, A, ldas, B, ldbs, alpha, beta, C, ldc, true, row_map);
}

int dali_hip_lstm_step(int batch, int input, int hidden, const float* X, int ldx, const float* Hprev, int ldh,
                       const float* Cprev, const float* W, int ldw, const float* U, int ldu, const float* bias,
                       float* Cout, float* Hout) {
    if (ensure_init()) return DALI_HIP_ERROR;
    if (batch <= 0 || input <= 0 || hidden <= 0) return fail("lstm_step: extents must be positive (batch=%d, input=%d, hidden=%d)", batch, input, hidden);
    if (!X || !Hprev || !Cprev || !W || !U || !bias || !Cout || !Hout) return fail("lstm_step: NULL argument");
    const bool ok = hidden % 64 == 0 && input % 64 == 0 && ldx % 4 == 0 && ldh % 4 == 0 && ldw % 4 == 0 && ldu % 4 == 0 && ldx >= input &&
                    ldh >= hidden && ldw >= 4 * hidden && ldu >= 4 * hidden && aligned16(X) && aligned16(Hprev) && aligned16(W) && aligned16(U) &&
                    (size_t)64 * (ldw > ldu ? ldw : ldu) * sizeof(float) + (size_t)4 * hidden * sizeof(float) < ((size_t)1 << 32) &&
                    ((size_t)batch * (ldx > ldh ? ldx : ldh) + 64) * sizeof(float) < ((size_t)1 << 32);
    if (!ok)
        return fail("lstm_step: the fused kernel needs input and hidden sizes that are multiples of 64 and 16-byte aligned operands whose "
                    "leading dimensions are multiples of 4");
    {
        const float* as[2] = {X, Hprev};
        const float* bs[2] = {W, U};
        const int ks[2] = {input, hidden}, las[2] = {ldx, ldh}, lbs[2] = {ldw, ldu};
        // a batch whose tiles leave compute units idle: shares of the inner extent, one work item per compute unit; whoever
        // draws a tile's last ticket adds the shares and computes the gates (up to 64 rows of 1024: 32 -> 17-19 us, 128 rows: 35 -> 27 us)
        static const int share_env = getenv("DALI_HIP_LSTM_STEP_SHARES") ? atoi(getenv("DALI_HIP_LSTM_STEP_SHARES")) : 1;
        const int shares = share_env ? stream_shares((long)((batch + 63) / 64) * (4 * hidden / 64), (input + hidden) / 64) : 1;
        if (shares >= 2) {
            const int r = sgemm_dma_stream(false, false, batch, 4 * hidden, 2, ks, as, bs, las, lbs, 1.0f, 0.0f, nullptr, 0, shares, device_cus(), bias, Cprev, Cout, Hout,
                                           hidden);
            if (r < 0) return DALI_HIP_ERROR;
            if (r > 0) return DALI_HIP_OK;
        }
        const int r = sgemm_dma(false, false, batch, 4 * hidden, 2, ks, as, bs, las, lbs, 1.0f, 0.0f, nullptr, 0, bias, Cprev, Cout, Hout, hidden);
        if (r < 0) return DALI_HIP_ERROR;
        if (r > 0) return DALI_HIP_OK;
    }
    // (the register-staged kernel below takes one pair of leading dimensions)
    if (ldx != ldh || ldw != ldu) return fail("lstm_step: X / Hprev (or W / U) with different leading dimensions need the kernel that DALI_HIP_GEMM_DMA=0 switches off");
    GemmArgs g = {};
    g.nseg = 2;
    g.seg[0].A = X;
    g.seg[0].B = W;
    g.seg[0].lda = ldx;
    g.seg[0].ldb = ldw;
    g.seg[0].K = input;
    g.seg[1].A = Hprev;
    g.seg[1].B = U;
    g.seg[1].lda = ldh;
    g.seg[1].ldb = ldu;
    g.seg[1].K = hidden;
    g.M = batch;
    g.N = 4 * hidden;
    g.alpha = 1.0f;
    g.beta = 0.0f;
    g.bias = bias;
    g.c_prev = Cprev;
    g.c_out = Cout;
    g.h_out = Hout;
    g.H = hidden;
    dim3 grid(4 * hidden / 64, (batch + 63) / 64);
    hipLaunchKernelGGL((sgemm_kernel<64, 64, 64, false, false, true, 2, false, 2, false, true>), grid, dim3(512), 0, stream(), g);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("lstm_step launch failed: %s", hipGetErrorString(e));
    return DALI_HIP_OK;
}

}  // extern "C"
