// The recurrent half of an LSTM (dali/layers/lstm.cpp:294-303) along a whole sequence in ONE launch, for any hidden size that is
// a multiple of 64 up to 2048 and up to 128 rows: the sizes that the kernel of lstm_persistent.hip (weights in LDS, at most 64
// rows, four hidden sizes) does not take.
//
// As there, workgroup g (one per compute unit, all resident together) owns HU hidden units and multiplies, every step, the
// previous state [B, H] with its columns of the recurrent weights. What differs:
//
//  * The weights live in registers, not in LDS. A wave owns a quarter of the K range and keeps, for every 16 values of k in
//    it, the B operands of its four v_mfma_f32_16x16x4_f32 (one register per instruction and 16-column tile): 64 registers
//    at H = 1024, 256 at H = 2048 (eight hidden units per workgroup, 32 columns), which is what no longer fits the LDS.
//    The loop over K is unrolled over the registers; trips past H / 64 are skipped by a wave-uniform test.
//  * The batch is cut into phases (row blocks of 16 or 32 rows) that take turns, each with an arrival counter of its own, so
//    that the grid barrier of one block is under way while the others are multiplied.
//  * The rows of h go through LDS, brought in by loads that write LDS themselves (a wave fetches its own quarter of every
//    row and reads its matrix operands from there; no workgroup barrier is involved).
//
// The state rows are exchanged through global memory: written with device-scope stores (written through to memory,
// acknowledged before the arrival is counted), read with ordinary loads after the barrier. An ordinary load may be served
// by the reader's second-level cache; that copy cannot be stale, because a row of hs is written once per launch, nobody
// reads it before the barrier that follows its writes, and caches start a launch clean. Counters of the second-level
// cache confirm it: 93% of the requests hit, 119 MB cross the memory interface in a launch of 32 steps at 64 rows of 1024
// where device-scope loads would move 2 GB.
//
// Where the time goes (timestamps inside the kernel, 64 rows of 1024 hidden units, turns of 32 rows): 3.6 us of a turn's
// 8 us are the issue of the next turn's loads, which is the second-level caches' bandwidth: every compute unit reads
// every row of h, 128 KiB a turn each, 10 TB/s over the chip; 2.7 us are the matrix instructions (1.95 at the peak rate),
// 0.6 us fold and gates, 0.5 us the acknowledgement of the stores, and the barrier itself is hidden. A step therefore costs
// about 2 x 8 us here against 13.6 us for the LDS kernel at the same size (its weights leave the registers free for all of a
// step's loads at once) and 33 us for a launch per step; the dispatcher takes this kernel for the sizes the other one
// does not serve, up to 96 rows (beyond, a launch per step is faster).
//
// Every wait is bounded as in lstm_persistent.hip: a workgroup that does not see the others arrive within spin_limit
// polls raises the host-visible flag, all workgroups leave at their next wait, the kernel ends normally and the next
// synchronising call reports the failure.
#include "runtime.h"

#include <cstdint>
#include <cstdlib>

#include "gate_math.h"

namespace dali_hip {

namespace {

typedef float f4 __attribute__((ext_vector_type(4)));

struct PhasedArgs {
    int T, B, H, HU, ldu, KQ;  // KQ = H / 64: trips of 16 values of k in a wave's quarter of the K range
    int PH;                    // phases: row blocks of 16 * MT rows that take turns
    const float* pre;          // [T, B, 4H] = x(t).W + b
    const float* U;            // [H, 4H], row stride ldu
    const float* h0;           // [B, H]
    const float* c0;           // [B, H]
    float* hs;                 // [T, B, H]
    float* c_out;              // [B, H]
    float* rh;                 // GRU: [T, B, H] scratch for r * h(t-1), written once per row like hs
    int* status;               // host-visible: set to 1 when a wait gave up
    unsigned int spin_limit;
};

constexpr int kMaxBar = 16;     // counters: phases (at most 8: 128 rows in blocks of 16) x rounds of a step (two for the GRU)
constexpr int kBarStride = 64;  // in words: every counter has 256 bytes to itself

// Arrival counters, one per phase, zero at rest (the last workgroup to leave restores that). One arrival per workgroup and one
// polling thread per workgroup: arrivals on one address are served one after the other by the memory side (about 12 ns each:
// an arrival per wave, 1024 on one counter, cost a phase 15 us), and 64 counters per phase polled by whole waves were slower
// than one counter polled by one thread (the polls crowd out the arrivals).
__device__ unsigned int g_bar[kMaxBar][kBarStride];
__device__ unsigned int g_done;

// bounded wait of one thread until `target` workgroups x steps have arrived at the counter of `phase`; false when it (or another
// workgroup) gave up
__device__ __forceinline__ unsigned int read_counter(int phase) { return __hip_atomic_load(&g_bar[phase][0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ bool wait_for(const PhasedArgs& a, int phase, unsigned int target) {
    unsigned int polls = 0;
    while (read_counter(phase) < target) {
        __builtin_amdgcn_s_sleep(1);
        if ((++polls & 63u) == 0u && __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0) return false;
        if (polls >= a.spin_limit) {
            __hip_atomic_store(a.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            return false;
        }
    }
    return true;
}
__device__ __forceinline__ void arrive(int phase) { __hip_atomic_fetch_add(&g_bar[phase][0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// The rows of h for one phase go through LDS. Every wave brings in its own quarter of the K range, row by row, with loads that
// write LDS themselves (one instruction moves up to 1 KiB of one row: whole cache lines, where a lane-per-operand load would
// touch 64 bytes of each of 16 rows), and reads its matrix operands from there; nothing is shared between waves, so no
// workgroup barrier is involved. A row's quarter is kept with a pitch of KW + 4 floats: the 16 rows of an operand read
// then start 4 banks apart and a 16-byte read per lane is conflict-free.
__device__ __forceinline__ void dma16(unsigned lds_addr, unsigned voff, const char* base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(base) : "memory");
}
// rows r0 .. r0 + rows - 1 of the [valid_rows, H] matrix at hp; rows past valid_rows are not fetched (what the matrix
// instructions make of the stale LDS contents lands in rows that nobody stores)
__device__ __forceinline__ void fetch_rows(const float* hp, int valid_rows, int H, int r0, int rows, int kbase, int lane, unsigned stage_base, int pitch_bytes) {
    const int KW = H / 4;  // floats of a row that this wave owns
    for (int r = 0; r < rows; ++r) {
        if (r0 + r >= valid_rows) break;
        const char* row = (const char*)(hp + (size_t)(r0 + r) * H + kbase);
        for (int piece = 0; piece * 256 < KW; ++piece) {
            if (piece * 256 + lane * 4 < KW) dma16(stage_base + (unsigned)(r * pitch_bytes + piece * 1024), (unsigned)(piece * 1024 + lane * 16), row);
        }
    }
}

// acc[m][n] += rows (from this wave's LDS stage) . (this wave's registers of the weight slice), over the wave's quarter of K
template <int KQB, int NT, int MT>
__device__ __forceinline__ void multiply(const char* stage, int pitch_bytes, int KQ, int arow, int kgrp, const float (&wreg)[KQB][4][NT], f4 (&acc)[MT][NT]) {
    const char* mine = stage + arow * pitch_bytes + kgrp * 16;
#pragma unroll
    for (int q = 0; q < KQB; ++q)
        if (q < KQ) {
            f4 av[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m) av[m] = *(const f4*)(mine + 16 * m * pitch_bytes + q * 64);
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int m = 0; m < MT; ++m)
#pragma unroll
                    for (int n = 0; n < NT; ++n) acc[m][n] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[m][c], wreg[q][c][n], acc[m][n], 0, 0, 0);
        }
}

// this wave's registers of the weight slice: NG gate blocks of HU columns, gate g of hidden unit u0 + uu at local column g * HU + uu
template <int KQB, int NT>
__device__ __forceinline__ void load_weights(const float* U, int ldu, int H, int HU, int NG, int u0, int KQ, int kbase, int arow, int kgrp, int gate0,
                                             float (&wreg)[KQB][4][NT]) {
    const int NC = NG * HU;
#pragma unroll
    for (int n = 0; n < NT; ++n) {
        const int j = 16 * n + arow, gate = j / HU, uu = j - gate * HU;
        const bool col_ok = j < NC;
        const size_t col = col_ok ? (size_t)(gate0 + gate) * H + u0 + uu : 0;
#pragma unroll
        for (int q = 0; q < KQB; ++q)
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const bool ok = col_ok && q < KQ;
                const float v = U[ok ? (size_t)(kbase + 16 * q + 4 * kgrp + c) * ldu + col : 0];
                wreg[q][c][n] = ok ? v : 0.0f;
            }
    }
}

// KQB: trips of 16 k that the registers of a wave hold (H <= 64 * KQB); NT: 16-column tiles (NT * 16 >= 4 * HU);
// MT: 16-row tiles of a phase. The phases (row blocks of 16 * MT rows) take turns; phase p of step t is "turn" t * PH + p.
template <int KQB, int NT, int MT>
__global__ __launch_bounds__(256) void lstm_phased_kernel(PhasedArgs a) {
    __shared__ float red[4][MT][NT][256];
    __shared__ float cells[128 * 8];  // the cell state of this workgroup's (row, hidden unit) pairs: row * HU + unit
    __shared__ int give_up;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // (wave-uniform for the compiler too)
    const int arow = lane & 15, kgrp = lane >> 4;
    const int H = a.H, HU = a.HU, B = a.B, KQ = a.KQ, PH = a.PH, kbase = wave * (H / 4);
    // Consecutive workgroups land on different dies (eight, each with a second-level cache of its own): the slices are dealt so
    // that one die holds neighbouring hidden units and whole lines of U and of the state rows belong to one die.
    const int parts = (gridDim.x & 7) == 0 ? 8 : 1;
    const int slice = (blockIdx.x % parts) * (gridDim.x / parts) + blockIdx.x / parts;
    const int u0 = slice * HU;
    float wreg[KQB][4][NT];
    load_weights<KQB, NT>(a.U, a.ldu, H, HU, 4, u0, KQ, kbase, arow, kgrp, 0, wreg);
    for (int e = tid; e < B * HU; e += 256) cells[e] = a.c0[(size_t)(e / HU) * H + u0 + e % HU];
    if (tid == 0) give_up = 0;
    // the (row, hidden unit) pairs this thread finishes in a phase: pair e = tid + 256 i is row e / HU of the phase, unit e % HU
    constexpr int PP = (16 * MT * (NT * 4) + 255) / 256;
    constexpr int ROWS = 16 * MT;
    // this wave's stage: ROWS rows of its quarter of K
    extern __shared__ __attribute__((aligned(16))) char stage_all[];
    const int pitch_bytes = H + 16;
    const unsigned stage_off = (unsigned)wave * (unsigned)(ROWS * pitch_bytes);
    const char* stage = stage_all + stage_off;
    const unsigned stage_base = (unsigned)(uintptr_t)stage_all + stage_off;  // (an LDS address is its low 32 bits)
    fetch_rows(a.h0, B, H, 0, ROWS, kbase, lane, stage_base, pitch_bytes);
    __syncthreads();
    const int turns = a.T * PH;
    for (int turn = 0; turn < turns; ++turn) {
        const int t = turn / PH, p = turn - t * PH, r0 = p * ROWS;
        const int tn = (turn + 1) / PH, pn = (turn + 1) - tn * PH;  // the next turn
        unsigned int early = 0;
        // the input half of the pre-activations
        float pre4[PP][4];
#pragma unroll
        for (int i = 0; i < PP; ++i) {
            const int e = tid + 256 * i, rr = e / HU, row = r0 + rr, uu = e - rr * HU;
            const bool mine = rr < ROWS && row < B;
#pragma unroll
            for (int g = 0; g < 4; ++g) pre4[i][g] = mine ? a.pre[((size_t)t * B + row) * 4 * H + (size_t)g * H + u0 + uu] : 0.0f;
        }
        f4 acc[MT][NT];
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n) acc[m][n] = (f4){0.f, 0.f, 0.f, 0.f};
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's rows have landed in its stage
        multiply<KQB, NT, MT>(stage, pitch_bytes, KQ, arow, kgrp, wreg, acc);
        // whether the next turn's rows of h(tn - 1) are complete is asked now and looked at after the gates
        if (tid == 0 && turn + 1 < turns && tn > 0) early = read_counter(pn);
        // fold the four waves' partial tiles: a lane holds column lane % 16 and rows 4 * (lane / 16) + v
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n)
#pragma unroll
                for (int v = 0; v < 4; ++v) red[wave][m][n][(4 * kgrp + v) * 16 + arow] = acc[m][n][v];
        __syncthreads();
#pragma unroll
        for (int i = 0; i < PP; ++i) {
            const int e = tid + 256 * i, rr = e / HU, row = r0 + rr, uu = e - rr * HU;
            if (rr < ROWS && row < B) {
                float g4[4];
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int j = g * HU + uu;
                    float s = 0.0f;
#pragma unroll
                    for (int w = 0; w < 4; ++w) s += red[w][rr / 16][j / 16][(rr & 15) * 16 + (j & 15)];
                    g4[g] = pre4[i][g] + s;
                }
                const float zero[4] = {0.f, 0.f, 0.f, 0.f};  // the bias is part of `pre`
                float cn, hn;
                lstm_gates(g4[0], g4[1], g4[2], g4[3], zero, cells[row * HU + uu], &cn, &hn);
                cells[row * HU + uu] = cn;
                __hip_atomic_store(a.hs + ((size_t)t * B + row) * H + u0 + uu, hn, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        // every wave's stores are acknowledged by memory before the workgroup counts its arrival
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();  // (also: the fold area is free again)
        if (tid == 0 && t + 1 < a.T) arrive(p);
        if (turn + 1 == turns) break;
        if (tid == 0 && tn > 0) {
            const unsigned int target = gridDim.x * (unsigned int)tn;
            // (a poll limit of zero gives up at the first wait without looking: the give-up path tested independently of timing)
            if (a.spin_limit == 0u || (early < target && !wait_for(a, pn, target))) {
                if (a.spin_limit == 0u) __hip_atomic_store(a.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                give_up = 1;
            }
        }
        __syncthreads();
        if (give_up) break;
        fetch_rows(tn == 0 ? a.h0 : a.hs + (size_t)(tn - 1) * B * H, B, H, pn * ROWS, ROWS, kbase, lane, stage_base, pitch_bytes);
    }
    __syncthreads();
    for (int e = tid; e < B * HU; e += 256) a.c_out[(size_t)(e / HU) * H + u0 + e % HU] = cells[e];
    // the counters go back to zero once every workgroup is past its last wait
    __shared__ int last_out;
    if (tid == 0) last_out = __hip_atomic_fetch_add(&g_done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == gridDim.x - 1;
    __syncthreads();
    if (last_out) {
        if (tid < kMaxBar) __hip_atomic_store(&g_bar[tid][0], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (tid == 0) __hip_atomic_store(&g_done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// The GRU (dali/layers/gru.cpp:27-44) in the same frame. `pre` is [T, B, 3H] = x(t).W + b and U [H, 3H], gates packed reset, update,
// candidate. A step has two rounds, each a product over all of H and therefore each behind a grid barrier:
//   A: (r, z) = sigmoid(pre_r,z + h(t-1).U_r,z); r * h(t-1) goes to the scratch rows rh[t] (the candidate needs it for ALL hidden units)
//   B: c = tanh(pre_c + rh[t].U_c); h(t) = h(t-1) * (1 - z) + c * z goes to hs[t]
// The turns of a step are A(phase 0), A(1), ..., B(0), B(1), ...: the barrier behind A(p) has the other phases' turns to complete in.
// Local columns: gate g of hidden unit u0 + uu at g * HU + uu, so that up to four hidden units put all three gates into one
// 16-column tile and eight put (r, z) into the first tile and the candidate into the second.
template <int KQB, int NT, int MT>
__global__ __launch_bounds__(256) void gru_phased_kernel(PhasedArgs a) {
    __shared__ float red[4][MT][256];
    __shared__ float hown[128 * 8];  // h(t-1) of this workgroup's (row, hidden unit) pairs: row * HU + unit
    __shared__ float zown[128 * 8];  // their update gates between the two rounds
    __shared__ int give_up;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int arow = lane & 15, kgrp = lane >> 4;
    const int H = a.H, HU = a.HU, B = a.B, KQ = a.KQ, PH = a.PH, kbase = wave * (H / 4);
    const int parts = (gridDim.x & 7) == 0 ? 8 : 1;
    const int slice = (blockIdx.x % parts) * (gridDim.x / parts) + blockIdx.x / parts;
    const int u0 = slice * HU;
    float wreg[KQB][4][NT];
    load_weights<KQB, NT>(a.U, a.ldu, H, HU, 3, u0, KQ, kbase, arow, kgrp, 0, wreg);
    for (int e = tid; e < B * HU; e += 256) hown[e] = a.h0[(size_t)(e / HU) * H + u0 + e % HU];
    if (tid == 0) give_up = 0;
    constexpr int ROWS = 16 * MT;
    static_assert(ROWS * (NT * 4) <= 256, "one (row, hidden unit) pair per thread");
    extern __shared__ __attribute__((aligned(16))) char stage_all[];
    const int pitch_bytes = H + 16;
    const unsigned stage_off = (unsigned)wave * (unsigned)(ROWS * pitch_bytes);
    const char* stage = stage_all + stage_off;
    const unsigned stage_base = (unsigned)(uintptr_t)stage_all + stage_off;
    fetch_rows(a.h0, B, H, 0, ROWS, kbase, lane, stage_base, pitch_bytes);
    __syncthreads();
    const int per_step = 2 * PH, turns = a.T * per_step;
    for (int turn = 0; turn < turns; ++turn) {
        const int t = turn / per_step, rest = turn - t * per_step, round = rest / PH, p = rest - round * PH, r0 = p * ROWS;
        const int tn = (turn + 1) / per_step, restn = (turn + 1) - tn * per_step, roundn = restn / PH, pn = restn - roundn * PH;
        // what the next turn reads: round A the rows of h(tn - 1), complete when counter PH + pn has seen tn rounds of arrivals;
        // round B the rows of rh[tn], complete when counter pn has seen tn + 1
        const int next_counter = roundn == 0 ? PH + pn : pn;
        const unsigned int next_target = gridDim.x * (unsigned int)(roundn == 0 ? tn : tn + 1);
        unsigned int early = 0;
        const int e = tid, rr = e / HU, row = r0 + rr, uu = e - rr * HU;
        const bool mine = rr < ROWS && row < B;
        float pre_a = 0.0f, pre_b = 0.0f;  // round A: reset and update; round B: candidate
        if (mine) {
            const float* pr = a.pre + ((size_t)t * B + row) * 3 * H + u0 + uu;
            if (round == 0) { pre_a = pr[0]; pre_b = pr[H]; } else { pre_a = pr[2 * H]; }
        }
        // round A needs the first tile only when (r, z) fill it (eight hidden units); otherwise every gate sits in tile 0
        f4 acc[MT][NT];
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n) acc[m][n] = (f4){0.f, 0.f, 0.f, 0.f};
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's rows have landed in its stage
        multiply<KQB, NT, MT>(stage, pitch_bytes, KQ, arow, kgrp, wreg, acc);
        if (tid == 0 && turn + 1 < turns && next_target > 0) early = read_counter(next_counter);
        // the tile that holds this round's columns: with two tiles, (r, z) are tile 0 and the candidate tile 1
        const int tile = NT == 2 && round == 1 ? 1 : 0;
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[wave][m][(4 * kgrp + v) * 16 + arow] = NT == 2 && tile == 1 ? acc[m][NT - 1][v] : acc[m][0][v];
        __syncthreads();
        if (mine) {
            auto column_sum = [&](int j) {
                float s = 0.0f;
#pragma unroll
                for (int w = 0; w < 4; ++w) s += red[w][rr / 16][(rr & 15) * 16 + (j & 15)];
                return s;
            };
            const float hprev = hown[row * HU + uu];
            if (round == 0) {
#pragma clang fp contract(off)
                const float r = gate_sigmoid(pre_a + column_sum(uu));
                const float z = gate_sigmoid(pre_b + column_sum(HU + uu));
                zown[row * HU + uu] = z;
                __hip_atomic_store(a.rh + ((size_t)t * B + row) * H + u0 + uu, r * hprev, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            } else {
#pragma clang fp contract(off)
                const float c = tanhf(pre_a + column_sum(2 * HU + uu));
                const float z = zown[row * HU + uu];
                const float keep = hprev * (1.0f - z);
                const float take = c * z;
                const float hn = keep + take;
                hown[row * HU + uu] = hn;
                __hip_atomic_store(a.hs + ((size_t)t * B + row) * H + u0 + uu, hn, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        // every wave's stores are acknowledged by memory before the workgroup counts its arrival
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();  // (also: the fold area is free again)
        if (tid == 0 && (round == 0 || t + 1 < a.T)) arrive(round == 0 ? p : PH + p);
        if (turn + 1 == turns) break;
        if (tid == 0 && next_target > 0) {
            if (a.spin_limit == 0u || (early < next_target && !wait_for(a, next_counter, next_target))) {
                if (a.spin_limit == 0u) __hip_atomic_store(a.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                give_up = 1;
            }
        }
        __syncthreads();
        if (give_up) break;
        const float* src = roundn == 1 ? a.rh + (size_t)tn * B * H : (tn == 0 ? a.h0 : a.hs + (size_t)(tn - 1) * B * H);
        fetch_rows(src, B, H, pn * ROWS, ROWS, kbase, lane, stage_base, pitch_bytes);
    }
    __shared__ int last_out;
    if (tid == 0) last_out = __hip_atomic_fetch_add(&g_done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == gridDim.x - 1;
    __syncthreads();
    if (last_out) {
        if (tid < kMaxBar) __hip_atomic_store(&g_bar[tid][0], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (tid == 0) __hip_atomic_store(&g_done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

template <typename K>
int launch(K kernel, const PhasedArgs& a, int grid, int rows_per_phase) {
    const size_t lds_bytes = (size_t)rows_per_phase * (a.H + 16) * 4;  // four waves x rows x (H / 4 + 4) floats
    hipError_t r = reserve_dynamic_lds((const void*)kernel, lds_bytes);
    if (r != hipSuccess) return fail("persistent recurrence: cannot reserve %zu bytes of LDS: %s", lds_bytes, hipGetErrorString(r));
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), lds_bytes, stream(), a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("persistent recurrence launch failed: %s", hipGetErrorString(e));
    return DALI_HIP_OK;
}

}  // namespace

// smallest power of two of hidden units per workgroup that gives every workgroup a compute unit of its own; 0 when there is none
static int units_per_workgroup(int hidden, int cus) {
    for (int hu = 1; hu <= 8; hu *= 2)
        if (hidden % hu == 0 && hidden / hu <= cus) return hu;
    return 0;
}

int recurrent_phased_supported(int batch, int hidden, int cus) {
    return batch >= 1 && batch <= 128 && hidden >= 64 && hidden <= 2048 && hidden % 64 == 0 && units_per_workgroup(hidden, cus) != 0;
}

int lstm_recurrent_phased(int steps, int batch, int hidden, const float* pre, const float* U, int ldu, const float* h0, const float* c0, float* hs,
                          float* c_out, int* status, int cus) {
    const int HU = units_per_workgroup(hidden, cus);
    if (!recurrent_phased_supported(batch, hidden, cus) || HU == 0)
        return fail("persistent recurrence: %d rows of %d hidden units on %d compute units are outside what it serves (at most 128 rows, hidden a multiple "
                    "of 64 up to 2048)", batch, hidden, cus);
    PhasedArgs a = {};
    a.T = steps; a.B = batch; a.H = hidden; a.HU = HU; a.ldu = ldu; a.KQ = hidden / 64;
    a.pre = pre; a.U = U; a.h0 = h0; a.c0 = c0; a.hs = hs; a.c_out = c_out;
    a.status = status;
    static const unsigned int spin_env = getenv("DALI_HIP_PERSISTENT_SPIN_LIMIT") ? (unsigned int)atol(getenv("DALI_HIP_PERSISTENT_SPIN_LIMIT")) : (1u << 20);
    a.spin_limit = spin_env;
    const int tiles = (batch + 15) / 16;
    // register classes: trips held per wave (hidden <= 64 * KQB) and 16-column tiles (4 * HU columns)
    const int KQB = hidden <= 256 ? 4 : hidden <= 512 ? 8 : hidden <= 1024 ? 16 : 32;
    const int NT = 4 * HU > 16 ? 2 : 1;
    // two row tiles per phase where the registers hold their tiles of h (32 x 16-byte pieces) and there are at least two phases then
    const int MT = (KQB <= 16 && tiles >= 4) ? 2 : 1;
    a.PH = (tiles + MT - 1) / MT;
    const int grid = hidden / HU;
#define DALI_PHASED_CASE(kqb, nt)                                                       \
    if (KQB == kqb && NT == nt) {                                                       \
        if (MT == 1) return launch(lstm_phased_kernel<kqb, nt, 1>, a, grid, 16);        \
        return launch(lstm_phased_kernel<kqb, nt, (kqb <= 16 ? 2 : 1)>, a, grid, 32);   \
    }
    DALI_PHASED_CASE(4, 1)
    DALI_PHASED_CASE(8, 1)
    DALI_PHASED_CASE(16, 1)
    DALI_PHASED_CASE(32, 2)
#undef DALI_PHASED_CASE
    return fail("persistent recurrence: no kernel for hidden %d", hidden);
}


// hidden units per workgroup for the GRU: three gates of each; the same rule as above
int gru_recurrent_phased(int steps, int batch, int hidden, const float* pre, const float* U, int ldu, const float* h0, float* hs, float* scratch,
                         int* status, int cus) {
    const int HU = units_per_workgroup(hidden, cus);
    if (!recurrent_phased_supported(batch, hidden, cus) || HU == 0)
        return fail("persistent recurrence: %d rows of %d hidden units on %d compute units are outside what it serves (at most 128 rows, hidden a multiple "
                    "of 64 up to 2048)", batch, hidden, cus);
    PhasedArgs a = {};
    a.T = steps; a.B = batch; a.H = hidden; a.HU = HU; a.ldu = ldu; a.KQ = hidden / 64;
    a.pre = pre; a.U = U; a.h0 = h0; a.hs = hs; a.rh = scratch;
    a.status = status;
    static const unsigned int spin_env = getenv("DALI_HIP_PERSISTENT_SPIN_LIMIT") ? (unsigned int)atol(getenv("DALI_HIP_PERSISTENT_SPIN_LIMIT")) : (1u << 20);
    a.spin_limit = spin_env;
    const int tiles = (batch + 15) / 16;
    const int KQB = hidden <= 256 ? 4 : hidden <= 512 ? 8 : hidden <= 1024 ? 16 : 32;
    const int NT = 3 * HU > 16 ? 2 : 1;
    const int MT = (KQB <= 16 && tiles >= 4) ? 2 : 1;
    a.PH = (tiles + MT - 1) / MT;
    const int grid = hidden / HU;
#define DALI_PHASED_CASE(kqb, nt)                                                      \
    if (KQB == kqb && NT == nt) {                                                      \
        if (MT == 1) return launch(gru_phased_kernel<kqb, nt, 1>, a, grid, 16);        \
        return launch(gru_phased_kernel<kqb, nt, (kqb <= 16 ? 2 : 1)>, a, grid, 32);   \
    }
    DALI_PHASED_CASE(4, 1)
    DALI_PHASED_CASE(8, 1)
    DALI_PHASED_CASE(16, 1)
    DALI_PHASED_CASE(32, 2)
#undef DALI_PHASED_CASE
    return fail("persistent recurrence: no kernel for hidden %d", hidden);
}

}  // namespace dali_hip
