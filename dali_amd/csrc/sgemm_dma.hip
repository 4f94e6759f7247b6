// fp32 GEMM for small grids (at most a few 64x64 tiles of C per CU; the LSTM step is exactly one): the memory pipeline
// writes the operand slabs into LDS itself (global_load_lds_dwordx4), four slabs are in flight, and the waves do
// nothing but read operands from LDS and issue v_mfma_f32_16x16x4_f32.
//
// Row-major view: C[M,N] = alpha * sum_s A_s[M,K_s] * B_s[K_s,N] + beta * C for one or two terms (dali_hip_sgemm,
// dali_hip_sgemm_pair, dali_hip_lstm_step; the reference's call is dali/array/gemm/cublas_gemm.cu:153-166).
//
// What shaped it (measured on MI355X with timestamps inside the kernel, one 64x64 tile over K = 2048 per CU):
//  * with every CU busy the fp32 matrix pipe is held back by power, not by issue: the shader clock settles near
//    2.05 GHz on random operands (2.25 GHz on zeros), so cycles saved in the loop come back as a lower clock unless
//    energy is saved with them. Staging through registers (global load, ds_write) and 32x32x2 instructions (which
//    read and write a 4 KiB accumulator per 4096 flops) both cost energy; loads straight into LDS and 16x16x4
//    instructions (half the accumulator traffic) gave 44.3 -> 36.4 us for the LSTM pair on the same device.
//  * one workgroup barrier per slab is enough, and it costs nothing when it sits inside the first k-group of a slab:
//    at that point a wave has the operands of its next k-group in registers, the barrier proves that every wave's
//    loads of slab i+1 have landed (they are first read in the second k-group) and that slab i-1 is no longer read,
//    and the loads of slab i+3 are issued into the buffer of slab i-1 one matrix instruction later (issuing them
//    right behind the barrier delayed the first instruction after it: 2133 -> 2071 cycles per slab of 2048).
//  * two wave sets split the k-groups of a slab (two waves per SIMD cover each other's waits: 2316 -> 2071 cycles)
//    and exchange halves of their sums through LDS at the end.
//
// LDS: four slabs of A, then four of B, 16 KiB each, no padding. An operand whose k runs along memory rows
// (A [M,K], B stored [N,K]) is kept as [row][k] with the 16-byte granule g of row r in slot (g ^ r) & 15: the 16 lanes
// of an operand read (same granule, consecutive rows) hit 16 different slots. An operand whose k runs across rows
// (B [K,N], A stored [K,M]) is kept as [k][col] with granule g of row k in slot g ^ (((k >> 2) & 3) << 2): the four lane
// groups of an operand read (k, k+4, k+8, k+12, sixteen consecutive columns each) hit the four quarters of a bank row.
// A lane of a load always writes LDS bytes [16 * lane, 16 * lane + 16) of its 1 KiB chunk, so the permutation is
// applied to the global address the lane fetches.
#include "runtime.h"

#include <cstdlib>
#include <type_traits>

#include "gate_math.h"

namespace dali_hip {

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kStage = 16384;          // bytes of one operand's slab: 64 x 64 floats
constexpr int kBRegion = 4 * kStage;   // the B slabs follow the four A slabs
constexpr int kDmaLds = 8 * kStage;

struct DmaArgs {
    const float* A[2];
    const float* B[2];
    int slabs[2];  // 64-deep slabs per term (the second is 0 for a single product), the last one of a term partly filled when
    int ktail[2];  // ... its inner extent is no multiple of 64: values of k in that slab (a multiple of 4), 0 = the slab is whole
    int lda[2], ldb[2];  // per term (x [batch, input] and h [batch, hidden] of an LSTM step have rows of different length)
    int M, N;
    float* C;
    int ldc;
    float alpha, beta;
    // gate epilogue (GATES): C is not written; see gate_math.h
    const float* bias;
    const float* c_prev;
    float* c_out;
    float* h_out;
    int H;
};

// One 16-byte piece per lane from global memory straight into LDS: lane l writes bytes [16 l, 16 l + 16) behind
// `lds_addr` (wave-uniform, goes through M0); the source is base + voff.
__device__ __forceinline__ void dma16(unsigned lds_addr, unsigned voff, const char* base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(base) : "memory");
}
// A pointer that is the same in every lane, said so where the compiler cannot prove it (a pointer chosen per work item): what is
// computed from it afterwards stays on the scalar unit.
__device__ __forceinline__ const char* wave_uniform(const char* p) {
    const unsigned long long b = (unsigned long long)p;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)b), hi = __builtin_amdgcn_readfirstlane((unsigned)(b >> 32));
    return (const char*)(((unsigned long long)hi << 32) | lo);
}
// The compiler does not see these loads, so the waits for them are written out; they are also compiler barriers.
__device__ __forceinline__ void wait_loads_but_4() { asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); }
__device__ __forceinline__ void wait_loads_but_8() { asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); }
__device__ __forceinline__ void wait_loads_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// TA: A stored as [K][M]; TB: B stored as [N][K]. 512 threads: waves 0-3 (wave set 0) and 4-7 (set 1) each cover the
// 64x64 tile as 2x2 wave tiles of 32x32; set kw takes the k-groups (16 k) kw and kw + 2 of every slab.
// KT: a term may end in a partly filled slab. Its loads fetch, for the values of k past the end, a piece that exists (the first
// of the same row, or row 0 of the slab: nothing outside the operands is read), and every lane overwrites what it fetched that
// way with zeros once its loads have landed, before the barrier that releases the slab.
template <bool TA, bool TB, bool GATES, bool LD2, bool KT>
__global__ __launch_bounds__(512, 1) void sgemm_dma_kernel(DmaArgs g) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave = w & 3, kw = w >> 2;
    const int wm = wave >> 1, wn = wave & 1, l16 = lane & 15, kq = lane >> 4;
    const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
    const int M = g.M, N = g.N;
    // Gate epilogue: the tile's columns are the four gates of sixteen hidden units. Workgroups are dealt to the eight
    // XCDs round-robin, so consecutive groups of hidden units go to workgroups of the same XCD: both 64-byte halves
    // of a 128-byte line of the weights are then asked for by the same L2.
    const int hu_base = GATES ? 16 * (gridDim.x % 8 == 0 ? (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8 : blockIdx.x) : 0;

    // gate epilogue operands first: they are then older than every load below, which keeps the counted waits exact
    float gate_bias[2][4], gate_c[2];
    if constexpr (GATES) {
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const int e = tid + q * 512, r = e / 16, j = e % 16, hu = hu_base + j;
            const int m = m0 + r < M ? m0 + r : M - 1;
#pragma unroll
            for (int k = 0; k < 4; ++k) gate_bias[q][k] = g.bias[k * g.H + hu];
            gate_c[q] = g.c_prev[(size_t)m * g.H + hu];
        }
    }

    // Sources of this wave's four loads per slab (byte offsets, constant over the kernel) and their LDS chunks.
    // Tiles that hang over the edge of C fetch the last valid row (or granule) instead: what they compute for rows and
    // columns outside C is never stored.
    // (the offsets of the second term, whose rows may be of another length, wait in a_next / b_next)
    unsigned a_off[2], b_off[2], a_next[2], b_next[2], a_dst[2], b_dst[2];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        const int c = w + 8 * q;                         // 1 KiB chunk: LDS rows 4c .. 4c+3 of the slab
        const int r = 4 * c + (lane >> 4), s = lane & 15;  // LDS row and slot of this lane's piece
        if (!TA) {
            const int row = m0 + r < M ? m0 + r : M - 1;
            a_off[q] = (unsigned)(((size_t)row * g.lda[0] + 4 * ((s ^ r) & 15)) * sizeof(float));
            if (LD2) a_next[q] = (unsigned)(((size_t)row * g.lda[1] + 4 * ((s ^ r) & 15)) * sizeof(float));
        } else {
            int col = m0 + 4 * (s ^ ((c & 3) << 2));
            col = col < M ? col : M - 4;
            a_off[q] = (unsigned)(((size_t)r * g.lda[0] + col) * sizeof(float));
            if (LD2) a_next[q] = (unsigned)(((size_t)r * g.lda[1] + col) * sizeof(float));
        }
        if (!TB) {
            const int gr = s ^ ((c & 3) << 2);
            int col = GATES ? (gr / 4) * g.H + hu_base + 4 * (gr % 4) : n0 + 4 * gr;
            col = col < N ? col : N - 4;
            b_off[q] = (unsigned)(((size_t)r * g.ldb[0] + col) * sizeof(float));
            if (LD2) b_next[q] = (unsigned)(((size_t)r * g.ldb[1] + col) * sizeof(float));
        } else {
            const int row = n0 + r < N ? n0 + r : N - 1;
            b_off[q] = (unsigned)(((size_t)row * g.ldb[0] + 4 * ((s ^ r) & 15)) * sizeof(float));
            if (LD2) b_next[q] = (unsigned)(((size_t)row * g.ldb[1] + 4 * ((s ^ r) & 15)) * sizeof(float));
        }
        a_dst[q] = (unsigned)(c * 1024);
        b_dst[q] = (unsigned)(kBRegion + c * 1024);
    }
    const char* ap = (const char*)g.A[0];
    const char* bp = (const char*)g.B[0];
    long a_step = (TA ? (long)64 * g.lda[0] : 64L) * (long)sizeof(float);
    long b_step = (TB ? 64L : (long)64 * g.ldb[0]) * (long)sizeof(float);
    const int slabs0 = g.slabs[0];
    const int n = slabs0 + g.slabs[1];
    int fj = 0;  // next slab to request
    // partly filled slabs: index within the whole sequence (-1: none) and, per load of this lane, whether its piece lies past the
    // end of such a slab and how far in front of it (bytes) the piece fetched in its place is
    const int tail0 = KT && g.ktail[0] ? slabs0 - 1 : -1, tail1 = KT && g.ktail[1] ? n - 1 : -1;
    auto past_end = [&](int q, bool of_b, int kr, unsigned* back, int term) __attribute__((always_inline)) -> bool {
        const int c = w + 8 * q, r = 4 * c + (lane >> 4), p = ((lane & 15) ^ r) & 15;
        const bool along_k = of_b ? TB : !TA;  // the 16 pieces of an LDS row run along k
        if (along_k) {
            *back = 16u * (unsigned)p;
            return 4 * p >= kr;
        }
        *back = (unsigned)r * (unsigned)(of_b ? g.ldb[term] : g.lda[term]) * 4u;
        return r >= kr;
    };
    auto issue = [&](int stage) __attribute__((always_inline)) {
        if (KT && (fj == tail0 || fj == tail1)) {
            const int term = fj == tail0 ? 0 : 1, kr = g.ktail[term];
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                unsigned back;
                dma16(a_dst[q] + stage * kStage, past_end(q, false, kr, &back, term) ? a_off[q] - back : a_off[q], ap);
            }
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                unsigned back;
                dma16(b_dst[q] + stage * kStage, past_end(q, true, kr, &back, term) ? b_off[q] - back : b_off[q], bp);
            }
        } else {
            dma16(a_dst[0] + stage * kStage, a_off[0], ap);
            dma16(a_dst[1] + stage * kStage, a_off[1], ap);
            dma16(b_dst[0] + stage * kStage, b_off[0], bp);
            dma16(b_dst[1] + stage * kStage, b_off[1], bp);
        }
        ++fj;
        ap += a_step;
        bp += b_step;
        if (fj == slabs0) {
            ap = (const char*)g.A[1];
            bp = (const char*)g.B[1];
            if (LD2) {
                a_step = (TA ? (long)64 * g.lda[1] : 64L) * (long)sizeof(float);
                b_step = (TB ? 64L : (long)64 * g.ldb[1]) * (long)sizeof(float);
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    a_off[q] = a_next[q];
                    b_off[q] = b_next[q];
                }
            }
        }
    };
    issue(0);
    if (n > 1) issue(1);
    if (n > 2) issue(2);

    // operand addresses of this lane: [k-group of the wave set][16-row block of the wave tile]
    unsigned a_addr[2][2], b_addr[2][2];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const int t = kw + 2 * tt;
            const int ra = wm * 32 + s * 16 + l16, rb = wn * 32 + s * 16 + l16;
            a_addr[tt][s] = !TA ? (unsigned)(ra * 256 + (((4 * t + kq) ^ ra) & 15) * 16) : (unsigned)((16 * t + 4 * kq) * 256 + ((ra ^ (kq << 4)) * 4));
            b_addr[tt][s] = kBRegion + (TB ? (unsigned)(rb * 256 + (((4 * t + kq) ^ rb) & 15) * 16) : (unsigned)((16 * t + 4 * kq) * 256 + ((rb ^ (kq << 4)) * 4)));
        }

    floatx4 acc[2][2];
#pragma unroll
    for (int si = 0; si < 2; ++si)
#pragma unroll
        for (int sj = 0; sj < 2; ++sj)
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[si][sj][v] = 0.f;

    // operands of one k-group: element c of a vector belongs to k = 16 t + 4 kq + c
    floatx4 a4[2][2], b4[2][2];
    auto load_ops = [&](auto ST, int tt, int o) __attribute__((always_inline)) {
        constexpr int st = decltype(ST)::value;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            if (!TA) {
                a4[o][s] = *(const floatx4*)(lds + a_addr[tt][s] + st * kStage);
            } else {
#pragma unroll
                for (int c = 0; c < 4; ++c) a4[o][s][c] = *(const float*)(lds + a_addr[tt][s] + st * kStage + c * 256);
            }
            if (TB) {
                b4[o][s] = *(const floatx4*)(lds + b_addr[tt][s] + st * kStage);
            } else {
#pragma unroll
                for (int c = 0; c < 4; ++c) b4[o][s][c] = *(const float*)(lds + b_addr[tt][s] + st * kStage + c * 256);
            }
        }
    };
    auto mfma = [&](int o, int c) __attribute__((always_inline)) {
#pragma unroll
        for (int si = 0; si < 2; ++si)
#pragma unroll
            for (int sj = 0; sj < 2; ++sj) acc[si][sj] = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[o][si][c], b4[o][sj][c], acc[si][sj], 0, 0, 0);
    };
    int cj = 0;  // (KT) the slab being multiplied
    auto zero_past_end = [&](int stage, int term) __attribute__((always_inline)) {
        const int kr = g.ktail[term];
        const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            unsigned back;
            if (past_end(q, false, kr, &back, term)) *(floatx4*)(lds + a_dst[q] + stage * kStage + 16 * lane) = zero;
            if (past_end(q, true, kr, &back, term)) *(floatx4*)(lds + b_dst[q] + stage * kStage + 16 * lane) = zero;
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
    // Slab i lives in LDS stage i % 4 (ST). The barrier inside slab i is for slab i+1; behind it the buffer of slab
    // i-1 is free and takes slab i+3.
    auto slab_step = [&](auto ST, auto H1, auto H2, auto H3) __attribute__((always_inline)) {
        constexpr int st = decltype(ST)::value;
        constexpr bool has1 = decltype(H1)::value, has2 = decltype(H2)::value, has3 = decltype(H3)::value;  // slabs i+1, i+2, i+3 exist
        using NX = std::integral_constant<int, (st + 1) % 4>;
        mfma(0, 0);
        load_ops(ST, 1, 1);
        __builtin_amdgcn_sched_barrier(0);
        mfma(0, 1);
        if (has1) {
            // own loads of slab i+1 done (those of slab i+2 may still be in flight), then everybody's
            if (has2) wait_loads_but_4(); else wait_loads_all();
            if (KT && (cj + 1 == tail0 || cj + 1 == tail1)) zero_past_end((st + 1) % 4, cj + 1 == tail0 ? 0 : 1);
            __builtin_amdgcn_s_barrier();
        }
        if (KT) ++cj;
        __builtin_amdgcn_sched_barrier(0);
        mfma(0, 2);
        if (has3) issue((st + 3) % 4);
        __builtin_amdgcn_sched_barrier(0);
        mfma(0, 3);
        __builtin_amdgcn_sched_barrier(0);
        mfma(1, 0);
        if (has1) load_ops(NX{}, 0, 0);  // behind the barrier: slab i+1 is complete in LDS
        __builtin_amdgcn_sched_barrier(0);
        mfma(1, 1);
        __builtin_amdgcn_sched_barrier(0);
        mfma(1, 2);
        __builtin_amdgcn_sched_barrier(0);
        mfma(1, 3);
        __builtin_amdgcn_sched_barrier(0);
    };
    // the last R slabs, starting in stage 0: step J of them
    auto tail_step = [&](auto J, auto R) __attribute__((always_inline)) {
        constexpr int j = decltype(J)::value, r = decltype(R)::value;
        if constexpr (j < r)
            slab_step(std::integral_constant<int, j % 4>{}, std::integral_constant<bool, (j + 1 < r)>{}, std::integral_constant<bool, (j + 2 < r)>{},
                      std::integral_constant<bool, (j + 3 < r)>{});
    };
    auto run_tail = [&](auto R) __attribute__((always_inline)) {
        tail_step(std::integral_constant<int, 0>{}, R);
        tail_step(std::integral_constant<int, 1>{}, R);
        tail_step(std::integral_constant<int, 2>{}, R);
        tail_step(std::integral_constant<int, 3>{}, R);
        tail_step(std::integral_constant<int, 4>{}, R);
        tail_step(std::integral_constant<int, 5>{}, R);
    };
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    using S2 = std::integral_constant<int, 2>;
    using S3 = std::integral_constant<int, 3>;
    using Yes = std::true_type;

    // slab 0 has landed once at most the loads of slabs 1 and 2 are outstanding
    if (n > 2) wait_loads_but_8();
    else if (n > 1) wait_loads_but_4();
    else wait_loads_all();
    __builtin_amdgcn_s_barrier();
    load_ops(S0{}, 0, 0);
    int i = 0;
    // steady state: slabs that still have three successors, four per trip so that the stage is a constant
    for (; i + 7 <= n; i += 4) {
        slab_step(S0{}, Yes{}, Yes{}, Yes{});
        slab_step(S1{}, Yes{}, Yes{}, Yes{});
        slab_step(S2{}, Yes{}, Yes{}, Yes{});
        slab_step(S3{}, Yes{}, Yes{}, Yes{});
    }
    const int rest = n - i;  // 1 .. 6
    if (rest == 1) run_tail(std::integral_constant<int, 1>{});
    else if (rest == 2) run_tail(std::integral_constant<int, 2>{});
    else if (rest == 3) run_tail(std::integral_constant<int, 3>{});
    else if (rest == 4) run_tail(std::integral_constant<int, 4>{});
    else if (rest == 5) run_tail(std::integral_constant<int, 5>{});
    else run_tail(std::integral_constant<int, 6>{});

    // The 16 sums of a lane: element e = (si * 2 + sj) * 4 + v is row wm*32 + si*16 + 4*kq + v, column wn*32 + sj*16 + l16
    // of the tile. The stages n % 4 and (n + 1) % 4 are read by no wave any more (the last two slabs sit in the two
    // others and every wave has passed the barrier inside slab n - 2, which it reaches after its last read of slab n - 3),
    // so the exchange needs no barrier in front.
    float out[16];
#pragma unroll
    for (int si = 0; si < 2; ++si)
#pragma unroll
        for (int sj = 0; sj < 2; ++sj)
#pragma unroll
            for (int v = 0; v < 4; ++v) out[(si * 2 + sj) * 4 + v] = acc[si][sj][v];

    if constexpr (GATES) {
        // both wave sets write their sums as a [64][64] tile of pre-activations; every thread then finishes two
        // (row, hidden unit) pairs. Bias and previous cell values were fetched at the start.
        float* mine = (float*)(lds + ((n + kw) & 3) * kStage);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int r = wm * 32 + (e / 8) * 16 + 4 * kq + (e % 4), c = wn * 32 + ((e / 4) % 2) * 16 + l16;
            mine[r * 64 + c] = out[e];
        }
        __syncthreads();
        const float* t0 = (const float*)(lds + (n & 3) * kStage);
        const float* t1 = (const float*)(lds + ((n + 1) & 3) * kStage);
        const int H = g.H;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const int e = tid + q * 512, r = e / 16, j = e % 16, m = m0 + r;
            if (m >= M) continue;
            float pre[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) pre[k] = t0[r * 64 + 16 * k + j] + t1[r * 64 + 16 * k + j];
            const size_t o = (size_t)m * H + hu_base + j;
            lstm_gates(pre[0], pre[1], pre[2], pre[3], gate_bias[q], gate_c[q], g.c_out + o, g.h_out + o);
        }
        return;
    } else {
        // wave set 0 keeps the upper 16 rows of every wave tile (e < 8), set 1 the lower; each hands the other half over
        float* red = (float*)(lds + (n & 3) * kStage);
#pragma unroll
        for (int v = 0; v < 8; ++v) red[(kw * 4 + wave) * 512 + v * 64 + lane] = kw == 0 ? out[8 + v] : out[v];
        __syncthreads();
        const float alpha = g.alpha, beta = g.beta;
#pragma unroll
        for (int v = 0; v < 8; ++v) {
            const float other = red[((1 - kw) * 4 + wave) * 512 + v * 64 + lane];
            // the term of set 0 first, whichever set adds: the sum does not depend on who keeps the element
            const float sum = kw == 0 ? out[v] + other : other + out[8 + v];
            const int e = kw * 8 + v;
            const int m = m0 + wm * 32 + (e / 8) * 16 + 4 * kq + (e % 4), nn = n0 + wn * 32 + ((e / 4) % 2) * 16 + l16;
            if (m < M && nn < N) {
                float* c = g.C + (size_t)m * g.ldc + nn;
                float r = alpha * sum;
                if (beta != 0.f) r += beta * *c;
                *c = r;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------- many tiles
// The same pipeline over a stream of work items. An item is a 64x64 tile of C, or, with Z > 1, one of Z contiguous shares of
// a tile's slabs (few tiles over a long inner extent). A workgroup walks its items one after the other and the loads run
// ahead across the item boundary: while the sums of one item are exchanged and stored, the first slabs of the next are
// already on their way. What it is for is the second case: [256,1024] over an inner extent of 32000 (a weight gradient of the
// vocabulary projection) runs as 64 tiles x 4 shares, one item per compute unit, in 145 us (0.73 of the fp32 matrix peak)
// with either operand order, where the register-staged kernel with shares took 158 us, 210 us with B stored as [N][K].
// With whole tiles as items it is no faster than one workgroup per tile (4096^3: 1150 us against 1033 us; 8000 tiles of four
// slabs: 195 us against 198 us): at 64x64x64 per slab every compute unit asks its die's cache for 32 KiB per microsecond,
// 8 TB/s over the device, which is what those caches deliver, so the product of many tiles stays with the 128x128 kernel.
// Items are numbered by tile (see tile_at) with the share fastest; the workgroups of one die (every eighth workgroup) take
// a contiguous band of them, so that tiles worked on together share their operands in that die's second-level cache. Shares of a tile meet in the workspace: each publishes its 64x64 partial sums and draws a
// ticket, the last one adds them in share order (the order does not depend on who finishes last).
struct StreamArgs {
    const float* A[2];
    const float* B[2];
    int slabs[2];
    int lda[2], ldb[2];  // per term (x [batch, input] and h [batch, hidden] of an LSTM step have rows of different length)
    int M, N;
    float* C;
    int ldc;
    float alpha, beta;
    int tiles_m, tiles_n, Z;
    unsigned int* counters;  // one ticket counter per tile (zero at rest)
    float* partials;         // [tile][share][4096]
    // gate epilogue (GATES): C is not written; a tile's columns are the four gates of sixteen hidden units
    const float* bias;
    const float* c_prev;
    float* c_out;
    float* h_out;
    int H;
};

constexpr int kFoldBytes = 16384;
constexpr int kStreamLds = kDmaLds + kFoldBytes + 16;  // stages, exchange area, one flag

template <bool TA, bool TB, bool GATES, bool LD2>
__global__ __launch_bounds__(512, 1) void sgemm_dma_stream_kernel(StreamArgs g) {
    // (no static LDS beside this: the loads address LDS from offset 0)
    extern __shared__ __attribute__((aligned(16))) char lds[];
    volatile int& is_last = *(volatile int*)(lds + kDmaLds + kFoldBytes);
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave = w & 3, kw = w >> 2;
    const int wm = wave >> 1, wn = wave & 1, l16 = lane & 15, kq = lane >> 4;
    const int M = g.M, N = g.N, Z = g.Z;
    const int slabs0 = g.slabs[0], n_all = slabs0 + g.slabs[1];
    const int items_total = g.tiles_m * g.tiles_n * Z;
    // this workgroup's items: first, first + stride, ... (count of them)
    int first, stride, count;
    {
        const int G = gridDim.x, b = blockIdx.x;
        if ((G & 7) == 0) {
            const int chunk = (items_total + 7) / 8, wgx = G / 8;
            const int lo = (b & 7) * chunk, hi = lo + chunk < items_total ? lo + chunk : items_total;
            first = lo + b / 8;
            stride = wgx;
            count = first < hi ? (hi - first + wgx - 1) / wgx : 0;
        } else {
            first = b;
            stride = G;
            count = first < items_total ? (items_total - first + G - 1) / G : 0;
        }
    }
    if (count == 0) return;
    auto share_begin = [&](int z) __attribute__((always_inline)) { return (int)((long)n_all * z / Z); };
    // Tiles are numbered in column blocks four tiles wide, by rows inside a block: 32 consecutive tiles (what the 32
    // workgroups of a die work on together) are 8 x 4 and ask their die's cache for 12 operand slabs per step, not 33.
    auto tile_at = [&](int tile, int& mt, int& nt) __attribute__((always_inline)) {
        const int per_block = g.tiles_m * 4, nb = tile / per_block, rem = tile - nb * per_block;
        const int width = g.tiles_n - 4 * nb < 4 ? g.tiles_n - 4 * nb : 4;
        mt = rem / width;
        nt = 4 * nb + (rem - mt * width);
    };
    int total = 0;  // slabs of all items of this workgroup
    for (int r = 0; r < count; ++r) {
        const int z = (first + r * stride) % Z;
        total += share_begin(z + 1) - share_begin(z);
    }

    long a_step = (TA ? (long)64 * g.lda[0] : 64L) * (long)sizeof(float), b_step = (TB ? 64L : (long)64 * g.ldb[0]) * (long)sizeof(float);
    auto set_steps = [&](int term) __attribute__((always_inline)) {
        a_step = (TA ? (long)64 * g.lda[term] : 64L) * (long)sizeof(float);
        b_step = (TB ? 64L : (long)64 * g.ldb[term]) * (long)sizeof(float);
    };
    // (the offsets of the second term, whose rows may be of another length, wait in a_next / b_next)
    unsigned a_off[2], b_off[2], a_next[2], b_next[2], a_dst[2], b_dst[2];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        a_dst[q] = (unsigned)((w + 8 * q) * 1024);
        b_dst[q] = (unsigned)(kBRegion + (w + 8 * q) * 1024);
    }
    // ---- the side that requests slabs
    int i_r = 0, i_fj = 0, i_n = 0, i_g = 0;  // item, slab within it, its slabs, slab within the tile's inner extent
    const char* ap = nullptr;
    const char* bp = nullptr;
    auto request_item = [&](int r) __attribute__((always_inline)) {
        const int id = first + r * stride, tile = id / Z, z = id - tile * Z;
        int mt, nt;
        tile_at(tile, mt, nt);
        const int m0 = 64 * mt, n0 = 64 * nt;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const int c = w + 8 * q;
            const int rr = 4 * c + (lane >> 4), s = lane & 15;
            if (!TA) {
                const int row = m0 + rr < M ? m0 + rr : M - 1;
                a_off[q] = (unsigned)(((size_t)row * g.lda[0] + 4 * ((s ^ rr) & 15)) * sizeof(float));
                if (LD2) a_next[q] = (unsigned)(((size_t)row * g.lda[1] + 4 * ((s ^ rr) & 15)) * sizeof(float));
            } else {
                int col = m0 + 4 * (s ^ ((c & 3) << 2));
                col = col < M ? col : M - 4;
                a_off[q] = (unsigned)(((size_t)rr * g.lda[0] + col) * sizeof(float));
                if (LD2) a_next[q] = (unsigned)(((size_t)rr * g.lda[1] + col) * sizeof(float));
            }
            if (!TB) {
                const int gr = s ^ ((c & 3) << 2);
                int col = GATES ? (gr / 4) * g.H + 16 * nt + 4 * (gr % 4) : n0 + 4 * gr;
                col = col < N ? col : N - 4;
                b_off[q] = (unsigned)(((size_t)rr * g.ldb[0] + col) * sizeof(float));
                if (LD2) b_next[q] = (unsigned)(((size_t)rr * g.ldb[1] + col) * sizeof(float));
            } else {
                const int row = n0 + rr < N ? n0 + rr : N - 1;
                b_off[q] = (unsigned)(((size_t)row * g.ldb[0] + 4 * ((s ^ rr) & 15)) * sizeof(float));
                if (LD2) b_next[q] = (unsigned)(((size_t)row * g.ldb[1] + 4 * ((s ^ rr) & 15)) * sizeof(float));
            }
        }
        i_g = share_begin(z);
        i_n = share_begin(z + 1) - i_g;
        i_fj = 0;
        const bool second = i_g >= slabs0;  // (only with two terms; shares are cut from single products)
        if (LD2) set_steps(second ? 1 : 0);
        if (LD2 && second) {
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                a_off[q] = a_next[q];
                b_off[q] = b_next[q];
            }
        }
        ap = wave_uniform((const char*)(second ? g.A[1] : g.A[0]) + (long)(i_g - (second ? slabs0 : 0)) * a_step);
        bp = wave_uniform((const char*)(second ? g.B[1] : g.B[0]) + (long)(i_g - (second ? slabs0 : 0)) * b_step);
    };
    auto issue = [&](int stage) __attribute__((always_inline)) {
        dma16(a_dst[0] + stage * kStage, a_off[0], ap);
        dma16(a_dst[1] + stage * kStage, a_off[1], ap);
        dma16(b_dst[0] + stage * kStage, b_off[0], bp);
        dma16(b_dst[1] + stage * kStage, b_off[1], bp);
        ++i_fj;
        ++i_g;
        ap += a_step;
        bp += b_step;
        if (i_g == slabs0 && g.slabs[1] > 0) {
            ap = (const char*)g.A[1];
            bp = (const char*)g.B[1];
            if (LD2) {
                set_steps(1);
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    a_off[q] = a_next[q];
                    b_off[q] = b_next[q];
                }
            }
        }
        if (i_fj == i_n) {
            ++i_r;
            if (i_r < count) request_item(i_r);
        }
    };
    request_item(0);
    issue(0);
    if (total > 1) issue(1);
    if (total > 2) issue(2);

    unsigned a_addr[2][2], b_addr[2][2];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const int t = kw + 2 * tt;
            const int ra = wm * 32 + s * 16 + l16, rb = wn * 32 + s * 16 + l16;
            a_addr[tt][s] = !TA ? (unsigned)(ra * 256 + (((4 * t + kq) ^ ra) & 15) * 16) : (unsigned)((16 * t + 4 * kq) * 256 + ((ra ^ (kq << 4)) * 4));
            b_addr[tt][s] = kBRegion + (TB ? (unsigned)(rb * 256 + (((4 * t + kq) ^ rb) & 15) * 16) : (unsigned)((16 * t + 4 * kq) * 256 + ((rb ^ (kq << 4)) * 4)));
        }
    floatx4 acc[2][2];
    auto clear = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int si = 0; si < 2; ++si)
#pragma unroll
            for (int sj = 0; sj < 2; ++sj)
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[si][sj][v] = 0.f;
    };
    clear();
    floatx4 a4[2][2], b4[2][2];
    auto load_ops = [&](auto ST, int tt, int o) __attribute__((always_inline)) {
        constexpr int st = decltype(ST)::value;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            if (!TA) {
                a4[o][s] = *(const floatx4*)(lds + a_addr[tt][s] + st * kStage);
            } else {
#pragma unroll
                for (int c = 0; c < 4; ++c) a4[o][s][c] = *(const float*)(lds + a_addr[tt][s] + st * kStage + c * 256);
            }
            if (TB) {
                b4[o][s] = *(const floatx4*)(lds + b_addr[tt][s] + st * kStage);
            } else {
#pragma unroll
                for (int c = 0; c < 4; ++c) b4[o][s][c] = *(const float*)(lds + b_addr[tt][s] + st * kStage + c * 256);
            }
        }
    };
    auto mfma = [&](int o, int c) __attribute__((always_inline)) {
#pragma unroll
        for (int si = 0; si < 2; ++si)
#pragma unroll
            for (int sj = 0; sj < 2; ++sj) acc[si][sj] = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[o][si][c], b4[o][sj][c], acc[si][sj], 0, 0, 0);
    };
    // ---- the side that multiplies: its item, the slab within it
    int c_r = 0, c_fj = 0, c_n;
    {
        const int z = first % Z;
        c_n = share_begin(z + 1) - share_begin(z);
    }
    // the sums of the finished item leave: exchange between the wave sets, then C (or the tile's partial sums and a ticket)
    auto finish_item = [&]() __attribute__((always_inline)) {
        const int id = first + c_r * stride, tile = id / Z, z = id - tile * Z;
        int mt, nt;
        tile_at(tile, mt, nt);
        const int m0 = 64 * mt, n0 = 64 * nt;
        float out[16];
#pragma unroll
        for (int si = 0; si < 2; ++si)
#pragma unroll
            for (int sj = 0; sj < 2; ++sj)
#pragma unroll
                for (int v = 0; v < 4; ++v) out[(si * 2 + sj) * 4 + v] = acc[si][sj][v];
        // (the area was last read in the previous item's exchange, which every wave left before the barrier of a later slab)
        float* red = (float*)(lds + kDmaLds);
#pragma unroll
        for (int v = 0; v < 8; ++v) red[(kw * 4 + wave) * 512 + v * 64 + lane] = kw == 0 ? out[8 + v] : out[v];
        __syncthreads();
        float sum[8];
#pragma unroll
        for (int v = 0; v < 8; ++v) {
            const float other = red[((1 - kw) * 4 + wave) * 512 + v * 64 + lane];
            sum[v] = kw == 0 ? out[v] + other : other + out[8 + v];
        }
        const float alpha = g.alpha, beta = g.beta;
        int last = 1;
        if (Z > 1) {
            float* part = g.partials + (size_t)tile * Z * 4096;
#pragma unroll
            for (int v = 0; v < 8; ++v) __hip_atomic_store(part + (size_t)z * 4096 + v * 512 + tid, sum[v], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            // the partial sums are acknowledged by memory before the ticket is drawn
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            __syncthreads();
            if (tid == 0) {
                const unsigned int ticket = __hip_atomic_fetch_add(g.counters + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                is_last = ticket == (unsigned int)Z - 1;
            }
            __syncthreads();
            last = __builtin_amdgcn_readfirstlane(is_last);
            if (last) {
#pragma unroll
                for (int v = 0; v < 8; ++v) sum[v] = 0.f;
                for (int z0 = 0; z0 < Z; z0 += 4) {
                    float t[4][8];
#pragma unroll
                    for (int u = 0; u < 4; ++u)
#pragma unroll
                        for (int v = 0; v < 8; ++v)
                            t[u][v] = __hip_atomic_load(part + (size_t)(z0 + u < Z ? z0 + u : z0) * 4096 + v * 512 + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                    for (int u = 0; u < 4; ++u)
                        if (z0 + u < Z) {
#pragma unroll
                            for (int v = 0; v < 8; ++v) sum[v] += t[u][v];
                        }
                }
                if (tid == 0) __hip_atomic_store(g.counters + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        if (GATES) {
            if (last) {
                // the sums as a [64][64] tile of pre-activations in the exchange area; every thread then finishes two (row, hidden
                // unit) pairs with the arithmetic of the fused step
                __syncthreads();  // the exchange has been read
#pragma unroll
                for (int v = 0; v < 8; ++v) {
                    const int e = kw * 8 + v;
                    red[(wm * 32 + (e / 8) * 16 + 4 * kq + (e % 4)) * 64 + wn * 32 + ((e / 4) % 2) * 16 + l16] = sum[v];
                }
                __syncthreads();
                const int H = g.H;
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const int e = tid + q * 512, r = e / 16, j = e % 16, m = m0 + r, hu = 16 * nt + j;
                    if (m >= M) continue;
                    float gate_bias[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) gate_bias[k] = g.bias[k * H + hu];
                    const size_t o = (size_t)m * H + hu;
                    lstm_gates(red[r * 64 + j], red[r * 64 + 16 + j], red[r * 64 + 32 + j], red[r * 64 + 48 + j], gate_bias, g.c_prev[o], g.c_out + o, g.h_out + o);
                }
            }
        } else if (last) {
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                const int e = kw * 8 + v;
                const int m = m0 + wm * 32 + (e / 8) * 16 + 4 * kq + (e % 4), nn = n0 + wn * 32 + ((e / 4) % 2) * 16 + l16;
                if (m < M && nn < N) {
                    float* c = g.C + (size_t)m * g.ldc + nn;
                    float r = alpha * sum[v];
                    if (beta != 0.f) r += beta * *c;
                    *c = r;
                }
            }
        }
        clear();
        ++c_r;
        c_fj = 0;
        if (c_r < count) {
            const int zn = (first + c_r * stride) % Z;
            c_n = share_begin(zn + 1) - share_begin(zn);
        }
    };
    auto slab_step = [&](auto ST, auto H1, auto H2, auto H3) __attribute__((always_inline)) {
        constexpr int st = decltype(ST)::value;
        constexpr bool has1 = decltype(H1)::value, has2 = decltype(H2)::value, has3 = decltype(H3)::value;
        using NX = std::integral_constant<int, (st + 1) % 4>;
        mfma(0, 0);
        load_ops(ST, 1, 1);
        __builtin_amdgcn_sched_barrier(0);
        mfma(0, 1);
        if (has1) {
            if (has2) wait_loads_but_4(); else wait_loads_all();
            __builtin_amdgcn_s_barrier();
        }
        __builtin_amdgcn_sched_barrier(0);
        mfma(0, 2);
        if (has3) issue((st + 3) % 4);
        __builtin_amdgcn_sched_barrier(0);
        mfma(0, 3);
        __builtin_amdgcn_sched_barrier(0);
        mfma(1, 0);
        if (has1) load_ops(NX{}, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        mfma(1, 1);
        __builtin_amdgcn_sched_barrier(0);
        mfma(1, 2);
        __builtin_amdgcn_sched_barrier(0);
        mfma(1, 3);
        __builtin_amdgcn_sched_barrier(0);
        if (++c_fj == c_n) finish_item();
    };
    auto tail_step = [&](auto J, auto R) __attribute__((always_inline)) {
        constexpr int j = decltype(J)::value, r = decltype(R)::value;
        if constexpr (j < r)
            slab_step(std::integral_constant<int, j % 4>{}, std::integral_constant<bool, (j + 1 < r)>{}, std::integral_constant<bool, (j + 2 < r)>{},
                      std::integral_constant<bool, (j + 3 < r)>{});
    };
    auto run_tail = [&](auto R) __attribute__((always_inline)) {
        tail_step(std::integral_constant<int, 0>{}, R);
        tail_step(std::integral_constant<int, 1>{}, R);
        tail_step(std::integral_constant<int, 2>{}, R);
        tail_step(std::integral_constant<int, 3>{}, R);
        tail_step(std::integral_constant<int, 4>{}, R);
        tail_step(std::integral_constant<int, 5>{}, R);
    };
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    using S2 = std::integral_constant<int, 2>;
    using S3 = std::integral_constant<int, 3>;
    using Yes = std::true_type;
    if (total > 2) wait_loads_but_8();
    else if (total > 1) wait_loads_but_4();
    else wait_loads_all();
    __builtin_amdgcn_s_barrier();
    load_ops(S0{}, 0, 0);
    int i = 0;
    for (; i + 7 <= total; i += 4) {
        slab_step(S0{}, Yes{}, Yes{}, Yes{});
        slab_step(S1{}, Yes{}, Yes{}, Yes{});
        slab_step(S2{}, Yes{}, Yes{}, Yes{});
        slab_step(S3{}, Yes{}, Yes{}, Yes{});
    }
    const int rest = total - i;  // 1 .. 6
    if (rest == 1) run_tail(std::integral_constant<int, 1>{});
    else if (rest == 2) run_tail(std::integral_constant<int, 2>{});
    else if (rest == 3) run_tail(std::integral_constant<int, 3>{});
    else if (rest == 4) run_tail(std::integral_constant<int, 4>{});
    else if (rest == 5) run_tail(std::integral_constant<int, 5>{});
    else run_tail(std::integral_constant<int, 6>{});
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

template <bool TA, bool TB, bool GATES, bool LD2, bool KT = false>
int launch(const DmaArgs& g, dim3 grid) {
    static bool attribute_set = false;  // one flag per instantiation of this function template
    auto kernel = sgemm_dma_kernel<TA, TB, GATES, LD2, KT>;
    if (!attribute_set) {
        hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kDmaLds);
        if (e != hipSuccess) return fail("sgemm: cannot reserve %d bytes of LDS: %s", kDmaLds, hipGetErrorString(e));
        attribute_set = true;
    }
    hipLaunchKernelGGL(kernel, grid, dim3(512), kDmaLds, stream(), g);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("sgemm launch failed: %s", hipGetErrorString(e));
    return 1;
}


// whole 64-deep slabs, 16-byte pieces that start on 16-byte boundaries and never straddle the end of a row, per-lane offsets
// (relative to a pointer that walks along k) that fit 32 bits
// (`tails`: an inner extent may end in a partly filled slab of whole 16-byte pieces)
bool operands_fit(bool ta, bool tb, int M, int N, int nseg, const int* K, const float* const* A, const float* const* B, const int* lda, const int* ldb,
                  bool tails = false) {
    if (nseg < 1 || nseg > 2 || M < 1 || N < 1) return false;
    if ((ta && M % 4 != 0) || (!tb && N % 4 != 0)) return false;
    for (int s = 0; s < nseg; ++s) {
        if (lda[s] % 4 != 0 || ldb[s] % 4 != 0) return false;
        if (K[s] < 64 || K[s] % (tails ? 4 : 64) != 0 || !aligned16(A[s]) || !aligned16(B[s])) return false;
        const size_t a_span = ((size_t)(ta ? 64 : M) * lda[s] + (ta ? M : 64)) * sizeof(float);
        const size_t b_span = ((size_t)(tb ? N : 64) * ldb[s] + (tb ? 64 : N)) * sizeof(float);
        if (a_span >= ((size_t)1 << 32) || b_span >= ((size_t)1 << 32)) return false;
    }
    return true;
}

template <bool TA, bool TB, bool GATES, bool LD2>
int launch_stream(const StreamArgs& g, int workgroups) {
    auto kernel = sgemm_dma_stream_kernel<TA, TB, GATES, LD2>;
    hipError_t e = reserve_dynamic_lds((const void*)kernel, kStreamLds);
    if (e != hipSuccess) return fail("sgemm: cannot reserve %d bytes of LDS: %s", kStreamLds, hipGetErrorString(e));
    hipLaunchKernelGGL(kernel, dim3(workgroups), dim3(512), kStreamLds, stream(), g);
    e = hipGetLastError();
    if (e != hipSuccess) return fail("sgemm launch failed: %s", hipGetErrorString(e));
    return 1;
}

}  // namespace

int sgemm_dma_stream(bool ta, bool tb, int M, int N, int nseg, const int* K, const float* const* A, const float* const* B, const int* lda, const int* ldb,
                     float alpha, float beta, float* C, int ldc, int shares, int cus, const float* bias, const float* c_prev, float* c_out, float* h_out, int H) {
    static const int enabled = getenv("DALI_HIP_GEMM_DMA") ? atoi(getenv("DALI_HIP_GEMM_DMA")) : 1;
    if (!enabled || cus < 8 || !operands_fit(ta, tb, M, N, nseg, K, A, B, lda, ldb)) return 0;
    StreamArgs g = {};
    int slabs = 0;
    for (int s = 0; s < 2; ++s) {
        g.A[s] = s < nseg ? A[s] : nullptr;
        g.B[s] = s < nseg ? B[s] : nullptr;
        g.slabs[s] = s < nseg ? K[s] / 64 : 0;
        slabs += g.slabs[s];
    }
    for (int s = 0; s < 2; ++s) {
        g.lda[s] = lda[s < nseg ? s : 0];
        g.ldb[s] = ldb[s < nseg ? s : 0];
    }
    const bool ld2 = g.lda[0] != g.lda[1] || g.ldb[0] != g.ldb[1];  // (a kernel of its own: the common case keeps its registers)
    g.M = M;
    g.N = N;
    g.C = C;
    g.ldc = ldc;
    g.alpha = alpha;
    g.beta = beta;
    g.tiles_m = (M + 63) / 64;
    g.tiles_n = (N + 63) / 64;
    const long tiles = (long)g.tiles_m * g.tiles_n;
    if (tiles > (1L << 24)) return 0;
    int Z = shares < 1 ? 1 : shares;
    if (Z > slabs) Z = slabs;
    if (Z > 1 && (tiles > (long)kWorkspaceCounters || (size_t)tiles * Z * 4096 * sizeof(float) > kWorkspacePartialBytes)) Z = 1;
    g.Z = Z;
    g.bias = bias;
    g.c_prev = c_prev;
    g.c_out = c_out;
    g.h_out = h_out;
    g.H = H;
    g.counters = (unsigned int*)workspace();
    g.partials = (float*)(workspace() + kWorkspaceCounterBytes);
    const long items = tiles * Z;
    // every workgroup has a compute unit to itself (its LDS); a whole number of workgroups per die keeps the bands of tiles
    int workgroups = cus - cus % 8;
    if (items < workgroups) workgroups = (int)items;
    if (bias) {
        if (ta || tb || N != 4 * H || H % 16 != 0) return 0;
        return ld2 ? launch_stream<false, false, true, true>(g, workgroups) : launch_stream<false, false, true, false>(g, workgroups);
    }
    if (!ta && !tb) return ld2 ? launch_stream<false, false, false, true>(g, workgroups) : launch_stream<false, false, false, false>(g, workgroups);
    if (!ta && tb) return ld2 ? launch_stream<false, true, false, true>(g, workgroups) : launch_stream<false, true, false, false>(g, workgroups);
    if (ta && !tb) return ld2 ? launch_stream<true, false, false, true>(g, workgroups) : launch_stream<true, false, false, false>(g, workgroups);
    return ld2 ? launch_stream<true, true, false, true>(g, workgroups) : launch_stream<true, true, false, false>(g, workgroups);
}

int sgemm_dma(bool ta, bool tb, int M, int N, int nseg, const int* K, const float* const* A, const float* const* B, const int* lda, const int* ldb,
              float alpha, float beta, float* C, int ldc, const float* bias, const float* c_prev, float* c_out, float* h_out, int H) {
    static const int enabled = getenv("DALI_HIP_GEMM_DMA") ? atoi(getenv("DALI_HIP_GEMM_DMA")) : 1;
    static const int tails_on = getenv("DALI_HIP_GEMM_DMA_TAILS") ? atoi(getenv("DALI_HIP_GEMM_DMA_TAILS")) : 1;
    const bool gates = bias != nullptr;
    if (!enabled || !operands_fit(ta, tb, M, N, nseg, K, A, B, lda, ldb, tails_on && !gates)) return 0;
    DmaArgs g = {};
    bool kt = false;
    for (int s = 0; s < 2; ++s) {
        g.A[s] = s < nseg ? A[s] : nullptr;
        g.B[s] = s < nseg ? B[s] : nullptr;
        g.slabs[s] = s < nseg ? (K[s] + 63) / 64 : 0;
        g.ktail[s] = s < nseg ? K[s] % 64 : 0;
        kt = kt || g.ktail[s] != 0;
    }
    for (int s = 0; s < 2; ++s) {
        g.lda[s] = lda[s < nseg ? s : 0];
        g.ldb[s] = ldb[s < nseg ? s : 0];
    }
    const bool ld2 = g.lda[0] != g.lda[1] || g.ldb[0] != g.ldb[1];  // (a kernel of its own: the common case keeps its registers)
    g.M = M;
    g.N = N;
    g.C = C;
    g.ldc = ldc;
    g.alpha = alpha;
    g.beta = beta;
    g.bias = bias;
    g.c_prev = c_prev;
    g.c_out = c_out;
    g.h_out = h_out;
    g.H = H;
    dim3 grid((N + 63) / 64, (M + 63) / 64);
    if (gates) {
        if (ta || tb) return 0;
        return ld2 ? launch<false, false, true, true>(g, grid) : launch<false, false, true, false>(g, grid);
    }
    if (kt) {
        // (one kernel per layout for every product with a partly filled slab, whatever its leading dimensions)
        if (!ta && !tb) return launch<false, false, false, true, true>(g, grid);
        if (!ta && tb) return launch<false, true, false, true, true>(g, grid);
        if (ta && !tb) return launch<true, false, false, true, true>(g, grid);
        return launch<true, true, false, true, true>(g, grid);
    }
    if (!ta && !tb) return ld2 ? launch<false, false, false, true>(g, grid) : launch<false, false, false, false>(g, grid);
    if (!ta && tb) return ld2 ? launch<false, true, false, true>(g, grid) : launch<false, true, false, false>(g, grid);
    if (ta && !tb) return ld2 ? launch<true, false, false, true>(g, grid) : launch<true, false, false, false>(g, grid);
    return ld2 ? launch<true, true, false, true>(g, grid) : launch<true, true, false, false>(g, grid);
}

}  // namespace dali_hip
