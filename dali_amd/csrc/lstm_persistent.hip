// The recurrent half of an LSTM along a whole sequence in ONE launch, for small batches
// (dali/layers/lstm.cpp:294-303 runs the cell step by step; the reference's third_party/nervana_kernels
// persistent_rnn_fprop.sass was meant to play this role on its hardware).
//
// At batch sizes of a few dozen rows one step is neither bound by the matrix pipe nor by memory: a launch per step
// spends its time waiting (37 us per step whatever the batch, measured up to 128 rows). What a step needs from memory
// is the recurrent weight matrix U [H, 4H], the same every step. The 256 compute units of an MI355X have 40 MiB of
// LDS between them, so U (16 MiB at H = 1024) stays on the chip for the whole sequence: workgroup g (one per compute
// unit) keeps the 4 * HU columns of U that produce the four gates of its HU hidden units, and per step
//   1. multiplies the previous hidden state h(t-1) [B, H] (read from global memory: it is the only thing the
//      workgroups exchange) with its slice of U on the matrix cores (v_mfma_f32_16x16x4_f32, the K range split over
//      the four waves and folded through LDS),
//   2. adds the input half of the pre-activations, pre[t] = x(t).W + bias, which does not depend on h and is computed
//      for all steps at once by one large product before this kernel runs,
//   3. applies the gates for its hidden units (same arithmetic, operation by operation, as the fused single step:
//      double-precision sigmoid, tanhf, no contraction) and writes its HU columns of h(t),
//   4. meets the other workgroups at a barrier (a counter in global memory) so that h(t) is complete before anyone
//      reads it. h is written and read with device-coherent accesses, so the barrier needs no cache-wide fences.
//      Up to 32 rows the barrier is replaced by waiting on the values of h(t-1) themselves (DATA_FLAGS below): a barrier
//      costs three dependent round trips through memory (4 us), a value that is polled one.
// The cell state of a workgroup's hidden units never leaves its registers.
//
// The barrier only works when every workgroup is resident, which holds because the grid has at most one workgroup per
// compute unit. Its wait is bounded: a workgroup that does not see the others arrive within `spin_limit` polls raises a
// flag in host-visible memory, every workgroup leaves at its next poll, and the next synchronising call of the
// library reports the failure instead of hanging the device.
#include "runtime.h"

#include <cstdint>
#include <cstdlib>
#include <type_traits>

namespace dali_hip {

// same sequence as the exp of the generated kernels and of the fused single step (sgemm.hip)
__device__ __forceinline__ float seq_expf(float x) {
    const float c = 0x1.715476p+0f, cc = 0x1.4ae0bep-26f;
    const float t = x * c;
    float r = __builtin_fmaf(x, c, -t);
    r = __builtin_fmaf(x, cc, r);
    const float e = __builtin_amdgcn_exp2f(t);
    const float fixed = __builtin_fmaf(e, r * 0x1.62e430p-1f, e);
    return __builtin_fabsf(t) < 128.0f ? fixed : e;
}

struct PersistentArgs {
    int T, B, H, HU, ldu;
    const float* pre;   // [T, B, 4H]
    const float* U;     // [H, 4H], row stride ldu
    const float* h0;    // [B, H]
    const float* c0;    // [B, H]
    float* hs;          // [T, B, H]
    float* c_out;       // [B, H]
    unsigned int* bar;  // barrier counter (zero at rest)
    unsigned int* done; // exit counter (zero at rest)
    int* status;        // host-visible: set to 1 when a barrier wait gave up
    unsigned int spin_limit;
};

constexpr int kPitchPad = 4;  // LDS row pitch of the U slice = 4 * HU + 4 floats: the four k-groups of a wave land 16 banks apart

typedef float f4 __attribute__((ext_vector_type(4)));
constexpr int kCoherentLoad = 16;  // cache policy of a buffer load: device scope (the sc1 bit)
// the same, marked volatile for the compiler: a load that is repeated until its value changes is not to be merged with
// its earlier instances
constexpr int kPollLoad = (int)(0x80000000u | 16u);

constexpr unsigned int kNotYet = 0xFFFFFFFFu;    // bit pattern that stands for "h not written yet" (a NaN no arithmetic here produces)
constexpr unsigned int kQuietNaN = 0x7FC00000u;

typedef unsigned int u4 __attribute__((ext_vector_type(4)));
// The pattern is the largest unsigned value: one of four words holds it exactly when their maximum does. (The words are
// taken from the whole vector cast to integers: __builtin_bit_cast applied to one element of a float vector, v[i], reads
// element 0 whatever i is with this compiler.)
__device__ __forceinline__ bool any_not_yet(f4 v) {
    const u4 w = __builtin_bit_cast(u4, v);
    const unsigned int hi = max(max(w[0], w[1]), max(w[2], w[3]));
    return hi == kNotYet;
}

// MT: 16-row tiles of the batch (B <= 16 * MT); KQ = H / 64: trips of 16 values of k in a wave's quarter of the K range.
// DATA_FLAGS: instead of a grid barrier per step, the rows of hs that the kernel will read are first filled with a bit
// pattern that means "not written yet" (one barrier, once), and a wave polls the values of h(t-1) it needs until none of
// them shows that pattern: a step then costs one memory round trip after the producers' stores instead of three.
template <int MT, int KQ, bool DATA_FLAGS>
__global__ __launch_bounds__(256) void lstm_persistent_kernel(PersistentArgs a) {
    extern __shared__ float lds[];
    const int H = a.H, HU = a.HU, NC = 4 * HU, P = NC + kPitchPad, B = a.B;
    float* Us = lds;                       // [H][P]
    float* red = lds + (size_t)H * P;      // [4 waves][MT][16][16]
    __shared__ int give_up;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // Consecutive workgroups land on different parts of the chip (eight, each with a second-level cache of its own): the
    // slices are dealt so that one part holds neighbouring columns and the 64-byte lines of U are fetched by one cache only.
    const int parts = (gridDim.x & 7) == 0 ? 8 : 1;
    const int slice = (blockIdx.x % parts) * (gridDim.x / parts) + blockIdx.x / parts;
    const int u0 = slice * HU;
    // the (row, hidden unit) pair this thread finishes every step
    const int pb = tid / HU, puu = tid - pb * HU;
    const bool owner = tid < B * HU;
    if (DATA_FLAGS) {
        // this workgroup's part of the rows of hs that will be read gets the "not written yet" pattern; the arrival is
        // counted now and awaited after the slice of U is in LDS, so the round trips of the one barrier hide behind that load
        if (owner)
            for (int t = 0; t + 1 < a.T; ++t)
                __hip_atomic_store(reinterpret_cast<unsigned int*>(a.hs) + ((size_t)t * B + pb) * H + u0 + puu, kNotYet, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) __hip_atomic_fetch_add(a.bar, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // this workgroup's slice of U: local column j = gate * HU + uu  <->  U column gate * H + u0 + uu
    if (HU == 4 && (a.ldu & 3) == 0 && ((uintptr_t)a.U & 15) == 0) {
        // one 16-byte load per (k, gate), eight in flight per thread
        for (int e0 = tid; e0 < H * 4; e0 += 256 * 8) {
            f4 v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int e = e0 + 256 * i, k = e >> 2, gate = e & 3;
                v[i] = e < H * 4 ? *reinterpret_cast<const f4*>(a.U + (size_t)k * a.ldu + (size_t)gate * H + u0) : (f4){0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int e = e0 + 256 * i, k = e >> 2, gate = e & 3;
                if (e < H * 4) *reinterpret_cast<f4*>(Us + (size_t)k * P + 4 * gate) = v[i];
            }
        }
    } else {
        for (int e0 = tid; e0 < H * NC; e0 += 256 * 8) {
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int e = e0 + 256 * i, k = e / NC, j = e - k * NC, gate = j / HU, uu = j - gate * HU;
                v[i] = e < H * NC ? a.U[(size_t)k * a.ldu + (size_t)gate * H + u0 + uu] : 0.0f;
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int e = e0 + 256 * i, k = e / NC, j = e - k * NC;
                if (e < H * NC) Us[(size_t)k * P + j] = v[i];
            }
        }
    }
    if (tid == 0) give_up = 0;
    float cell = owner ? a.c0[(size_t)pb * H + u0 + puu] : 0.0f;
    __syncthreads();

    const int KW = H / 4;             // K range of a wave
    const int arow = lane & 15, kgrp = lane >> 4;
    // The values of h cross compute units (and their second-level caches) once a step. They are written and read with
    // device-coherent accesses (stores and loads at agent scope go past the caches that are private to a part of the chip),
    // so the step needs no cache-wide release or acquire: those fences write back and invalidate the whole second-level
    // cache and took 15 to 24 us of a step.
    float pre4[4] = {0.f, 0.f, 0.f, 0.f};
    auto fetch_pre = [&](int t) {
        if (owner) {
#pragma unroll
            for (int gate = 0; gate < 4; ++gate) pre4[gate] = a.pre[((size_t)t * B + pb) * 4 * H + (size_t)gate * H + u0 + puu];
        }
    };
    fetch_pre(0);
    // bounded wait of thread 0 on the barrier counter; false when it (or another workgroup) gave up
    auto wait_for = [&](unsigned int target) {
        unsigned int polls = 0;
        while (__hip_atomic_load(a.bar, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
            __builtin_amdgcn_s_sleep(1);
            if ((++polls & 63u) == 0u && __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0) return false;
            if (polls >= a.spin_limit) {
                __hip_atomic_store(a.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                return false;
            }
        }
        return true;
    };
    if (DATA_FLAGS) {
        // every workgroup's pattern has reached memory before anybody's first h does
        if (tid == 0 && !wait_for(gridDim.x)) give_up = 1;
        __syncthreads();
    }
    for (int t = 0; t < a.T && !give_up; ++t) {
        const float* hp = t == 0 ? a.h0 : a.hs + (size_t)(t - 1) * B * H;
        // rows past the batch are out of the buffer's range and read as zero
        const __amdgpu_buffer_rsrc_t hrow = __builtin_amdgcn_make_buffer_rsrc((void*)hp, 0, B * H * 4, 0x00027000);
        f4 acc[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[m] = (f4){0.f, 0.f, 0.f, 0.f};
        // 16 values of k per trip: a lane fetches four consecutive k of its batch row with one 16-byte load and feeds them
        // to four matrix instructions; the slice of U is read at the matching rows, so which k sits in which slot of the
        // instruction does not matter to the sum. Every load of the step is issued before the first product: the step pays
        // the latency of h(t-1) once.
        f4 av[KQ][MT];
        auto load_tile = [&](int m) {
#pragma unroll
            for (int q = 0; q < KQ; ++q) {
                const int kb = wave * KW + 16 * q + 4 * kgrp;
                av[q][m] = __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(hrow, ((16 * m + arow) * H + kb) * 4, 0, DATA_FLAGS ? kPollLoad : kCoherentLoad));
            }
        };
        if (!DATA_FLAGS || t == 0) {
#pragma unroll
            for (int m = 0; m < MT; ++m) load_tile(m);
        } else {
            // every tile is fetched, and a tile in which a lane of this wave still sees the "not written yet" pattern (rows
            // past the batch read as zero) is fetched again until none does
            unsigned int polls = 0;
            bool need[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m) need[m] = true;
            // The waiting is done on one load per lane: a wave that fetched all its tiles again and again would multiply the
            // traffic of the step (at 64 rows every workgroup reads 256 KiB of h) and slow the producers it waits for.
            while (polls < a.spin_limit) {
                const int kb = wave * KW + 4 * kgrp;
                const f4 probe = __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(hrow, (arow * H + kb) * 4, 0, kPollLoad));
                if (!__any(any_not_yet(probe))) break;
                asm volatile("" ::: "memory");
                __builtin_amdgcn_s_sleep(1);
                ++polls;
                if ((polls & 15u) == 0u && __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0) break;
            }
            while (true) {
#pragma unroll
                for (int m = 0; m < MT; ++m)
                    if (need[m]) load_tile(m);
                bool again = false;
#pragma unroll
                for (int m = 0; m < MT; ++m)
                    if (need[m]) {
                        bool missing = false;
#pragma unroll
                        for (int q = 0; q < KQ; ++q) missing = missing || any_not_yet(av[q][m]);
                        need[m] = __any(missing);  // the same for every lane
                        again = again || need[m];
                    }
                if (!again) break;
                asm volatile("" ::: "memory");
                __builtin_amdgcn_s_sleep(1);
                ++polls;
                const bool others = (polls & 15u) == 0u && __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0;
                if (others || polls >= a.spin_limit) {
                    if (!others) __hip_atomic_store(a.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                    give_up = 1;  // (every wave that gives up writes the same value; read behind the next barrier)
                    break;
                }
            }
        }
#pragma unroll
        for (int q = 0; q < KQ; ++q) {
            const int kb = wave * KW + 16 * q + 4 * kgrp;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const float bv = Us[(size_t)(kb + c) * P + arow];  // B operand: row k of the slice, column lane % 16
#pragma unroll
                for (int m = 0; m < MT; ++m) acc[m] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[q][m][c], bv, acc[m], 0, 0, 0);
            }
        }
        // fold the four waves' partial tiles: lane holds column lane % 16 and rows 4 * (lane / 16) + v
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[((size_t)(wave * MT + m) * 16 + 4 * kgrp + v) * 16 + arow] = acc[m][v];
        __syncthreads();
        if (give_up) break;  // a wave stopped waiting for h(t-1): the sums are meaningless
        if (owner) {
#pragma clang fp contract(off)
            float g4[4];
#pragma unroll
            for (int gate = 0; gate < 4; ++gate) {
                const int j = gate * HU + puu;
                float s = 0.0f;
#pragma unroll
                for (int w = 0; w < 4; ++w) s += red[((size_t)(w * MT + pb / 16) * 16 + (pb & 15)) * 16 + j];
                g4[gate] = pre4[gate] + s;
            }
            const float iv = (float)(1.0 / (1.0 + (double)seq_expf(-g4[0])));
            const float fv = (float)(1.0 / (1.0 + (double)seq_expf(-g4[1])));
            const float ov = (float)(1.0 / (1.0 + (double)seq_expf(-g4[2])));
            const float gv = tanhf(g4[3]);
            const float fc = fv * cell;
            const float ig = iv * gv;
            cell = fc + ig;
            float hv = ov * tanhf(cell);
            if (DATA_FLAGS && __builtin_bit_cast(unsigned int, hv) == kNotYet) hv = __builtin_bit_cast(float, kQuietNaN);
            __hip_atomic_store(a.hs + ((size_t)t * B + pb) * H + u0 + puu, hv, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (t + 1 == a.T) break;
        if (DATA_FLAGS) {
            fetch_pre(t + 1);
            __syncthreads();  // the fold area is free again
            continue;
        }
        // grid barrier: everybody's columns of h(t) have reached device memory before anybody reads row t
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();  // (also: the fold area is free again)
        if (tid == 0) __hip_atomic_fetch_add(a.bar, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        fetch_pre(t + 1);  // does not depend on h: in flight during the wait
        if (tid == 0 && !wait_for(gridDim.x * (unsigned int)(t + 1))) give_up = 1;
        __syncthreads();
    }
    if (owner) a.c_out[(size_t)pb * H + u0 + puu] = cell;
    // the counters go back to zero once every workgroup is past its last wait
    __syncthreads();
    if (tid == 0) {
        const unsigned int ticket = __hip_atomic_fetch_add(a.done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (ticket == gridDim.x - 1) {
            __hip_atomic_store(a.bar, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(a.done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// ------------------------------------------------------------------------------------------------ one step, small batch
// A single step for a small batch (a decoder that feeds every output back through the host): the tiles of the general
// product kernel are 64 rows high, so a step of 8 rows costs as much matrix-pipe time as one of 64 and only 64 workgroups
// share the weights (37 us whatever the batch). What such a step has to do is stream W and U (32 MiB at I = H = 1024) once.
// Workgroup (unit block, gate, k share) owns 64 consecutive columns of one gate, 256 bytes of every weight row, over a
// 1 / KS share of the K range of x.W + h.U, the share split over its four waves. The weights go straight from memory into
// the B operand of the matrix instruction: a lane loads four consecutive columns of row k with one 16-byte load and feeds
// them to four instructions, whose 16-column tiles are therefore the columns congruent to 0, 1, 2 and 3 modulo 4 (a tile need
// not be contiguous). Whole cache lines and few load instructions: a first version that gave every workgroup the four gates
// of four hidden units read 16 bytes of each line, one value per lane and instruction, and took 14 to 32 us. The workgroups
// of a unit block publish their partial pre-activations in the library workspace and take a ticket; the last of them adds
// the k shares in order, then bias, gates and cell update as in the fused step.
struct SmallStepArgs {
    int B, I, H, KS;
    const float* X;   // [B, I]
    const float* Hp;  // [B, H]
    const float* Cp;  // [B, H]
    const float* W;   // [I, 4H]
    const float* U;   // [H, 4H]
    const float* bias;  // [4H]
    float* Cout;      // [B, H]
    float* Hout;      // [B, H]
    int ldx, ldh, ldw, ldu;
    unsigned int* tickets;  // one per unit block, zero at rest
    float* partials;        // [unit blocks][4 gates][KS][B][64]
};

constexpr int kSmallUnits = 64;  // hidden units (columns of one gate) per workgroup
constexpr int kSmallMaxShares = 8;  // k shares per unit block at most

template <int MT, int G>
__global__ __launch_bounds__(256) void lstm_step_small_kernel(SmallStepArgs a) {
    extern __shared__ float red_flat[];  // [4 waves][4 column tiles][MT][16][16]
    float (*red)[4][MT][16][16] = reinterpret_cast<float (*)[4][MT][16][16]>(red_flat);
    __shared__ int is_last;
    const int H = a.H, B = a.B, I = a.I, KS = a.KS;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ks = blockIdx.x % KS, gate = (blockIdx.x / KS) & 3, ub = blockIdx.x / (4 * KS);
    const int col0 = gate * H + ub * kSmallUnits;
    const int arow = lane & 15, kgrp = lane >> 4;
    const int KP = (I + H) / KS, KW = KP / 4;  // K range of the workgroup and of a wave (a multiple of 16)
    const __amdgpu_buffer_rsrc_t xrows = __builtin_amdgcn_make_buffer_rsrc((void*)a.X, 0, ((B - 1) * a.ldx + I) * 4, 0x00027000);
    const __amdgpu_buffer_rsrc_t hrows = __builtin_amdgcn_make_buffer_rsrc((void*)a.Hp, 0, ((B - 1) * a.ldh + H) * 4, 0x00027000);
    f4 acc[4][MT];
#pragma unroll
    for (int ct = 0; ct < 4; ++ct)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[ct][m] = (f4){0.f, 0.f, 0.f, 0.f};
    for (int q0 = 0; q0 < KW / 16; q0 += G) {
        f4 av[G][MT];
        f4 bv[G][4];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const int k0 = ks * KP + wave * KW + 16 * (q0 + g);  // wave-uniform; a trip of 16 lies wholly in x.W or in h.U
            const bool valid = q0 + g < KW / 16;
            const bool in_x = k0 < I;
            const int kk = (in_x ? k0 : k0 - I) + 4 * kgrp;
            const float* wp = (in_x ? a.W + (size_t)kk * a.ldw : a.U + (size_t)kk * a.ldu) + col0 + 4 * arow;
            const size_t ldk = in_x ? a.ldw : a.ldu;
#pragma unroll
            for (int c = 0; c < 4; ++c) bv[g][c] = valid ? *reinterpret_cast<const f4*>(wp + (size_t)c * ldk) : (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const int row = 16 * m + arow;
                // rows past the batch lie beyond the buffer's range and read as zero
                const int off = row < B && valid ? (row * (in_x ? a.ldx : a.ldh) + kk) * 4 : 0x7ffffff0;
                av[g][m] = __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(in_x ? xrows : hrows, off, 0, 0));
            }
        }
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int ct = 0; ct < 4; ++ct)
#pragma unroll
                    for (int m = 0; m < MT; ++m) acc[ct][m] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[g][m][c], bv[g][c][ct], acc[ct][m], 0, 0, 0);
    }
    // a lane holds column lane % 16 (of tile ct: column 4 * (lane % 16) + ct of the block) and rows 4 * (lane / 16) + v
#pragma unroll
    for (int ct = 0; ct < 4; ++ct)
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[wave][ct][m][4 * kgrp + v][arow] = acc[ct][m][v];
    __syncthreads();
    // this workgroup's share of the pre-activations of (row b, unit u): the four waves in order
    float* mine = a.partials + (((size_t)ub * 4 + gate) * KS + ks) * (size_t)B * kSmallUnits;
    for (int e = tid; e < B * kSmallUnits; e += 256) {
        const int bb = e / kSmallUnits, u = e % kSmallUnits;
        float s = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) s += red[w][u & 3][bb / 16][bb & 15][u >> 2];
        __hip_atomic_store(mine + e, s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // the shares are acknowledged by memory before the ticket is drawn; the clobber keeps the compiler from moving them
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        const unsigned int ticket = __hip_atomic_fetch_add(a.tickets + ub, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        is_last = ticket == (unsigned int)(4 * KS - 1);
    }
    __syncthreads();
    if (!is_last) return;
    // The fold: a thread takes four neighbouring units of one row at a time; the 16-byte shares of all four gates are asked
    // for (device-coherent loads) before the first is awaited, then added in k order. (Awaiting every 4-byte share in turn
    // cost a memory round trip each: 90 us for 64 rows.)
    const float* blockp = a.partials + (size_t)ub * 4 * KS * (size_t)B * kSmallUnits;
    const __amdgpu_buffer_rsrc_t shares = __builtin_amdgcn_make_buffer_rsrc((void*)blockp, 0, 4 * KS * B * kSmallUnits * 4, 0x00027000);
    // With at most four k shares a thread asks for the shares of two quads at once (the registers that eight shares of one
    // quad would take): half as many round trips for 17 rows and more.
    const int quads = B * (kSmallUnits / 4);
    auto fold = [&](auto per_trip_tag, auto shares_tag) {
        constexpr int QI = decltype(per_trip_tag)::value, KSM = decltype(shares_tag)::value;
        for (int quad0 = tid; quad0 < quads; quad0 += 256 * QI) {
#pragma clang fp contract(off)
            f4 pv[QI][4][KSM];
#pragma unroll
            for (int i = 0; i < QI; ++i) {
                const int quad = quad0 + 256 * i;
                const int bb = quad / (kSmallUnits / 4), u = (quad % (kSmallUnits / 4)) * 4;
#pragma unroll
                for (int gt = 0; gt < 4; ++gt)
#pragma unroll
                    for (int k = 0; k < KSM; ++k)
                        pv[i][gt][k] = k < KS && quad < quads
                                           ? __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(shares, (((gt * KS + k) * B + bb) * kSmallUnits + u) * 4, 0, kCoherentLoad))
                                           : (f4){0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int i = 0; i < QI; ++i) {
                const int quad = quad0 + 256 * i;
                if (quad >= quads) break;
                const int bb = quad / (kSmallUnits / 4), u = (quad % (kSmallUnits / 4)) * 4, unit = ub * kSmallUnits + u;
                const f4 cells = *reinterpret_cast<const f4*>(a.Cp + (size_t)bb * H + unit);
                f4 cn4, hn4;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float g4[4];
#pragma unroll
                    for (int gt = 0; gt < 4; ++gt) {
                        float sum = 0.0f;
#pragma unroll
                        for (int k = 0; k < KSM; ++k)
                            if (k < KS) sum += pv[i][gt][k][j];
                        g4[gt] = sum + a.bias[gt * H + unit + j];
                    }
                    const float iv = (float)(1.0 / (1.0 + (double)seq_expf(-g4[0])));
                    const float fv = (float)(1.0 / (1.0 + (double)seq_expf(-g4[1])));
                    const float ov = (float)(1.0 / (1.0 + (double)seq_expf(-g4[2])));
                    const float gv = tanhf(g4[3]);
                    const float fc = fv * cells[j];
                    const float ig = iv * gv;
                    const float cn = fc + ig;
                    cn4[j] = cn;
                    hn4[j] = ov * tanhf(cn);
                }
                *reinterpret_cast<f4*>(a.Cout + (size_t)bb * H + unit) = cn4;
                *reinterpret_cast<f4*>(a.Hout + (size_t)bb * H + unit) = hn4;
            }
        }
    };
    if (KS <= 4 && quads > 256) fold(std::integral_constant<int, 2>(), std::integral_constant<int, 4>());
    else fold(std::integral_constant<int, 1>(), std::integral_constant<int, kSmallMaxShares>());
    if (tid == 0) __hip_atomic_store(a.tickets + ub, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

static int* g_status = nullptr;  // pinned host word the kernel raises on a barrier time-out

int persistent_status_take() {
    if (!g_status) return 0;
    const int v = __atomic_exchange_n(g_status, 0, __ATOMIC_RELAXED);
    return v;
}

}  // namespace dali_hip

using namespace dali_hip;

// host-visible status word shared by the persistent kernels (pinned, allocated on first use outside a capture)
static int ensure_status_word(const char* who) {
    if (g_status) return DALI_HIP_OK;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    (void)hipStreamIsCapturing(stream(), &cs);
    if (cs != hipStreamCaptureStatusNone) return fail("%s: first use cannot be inside a capture", who);
    if (hipHostMalloc((void**)&g_status, sizeof(int), hipHostMallocMapped) != hipSuccess) return fail("%s: no pinned status word", who);
    *g_status = 0;
    return DALI_HIP_OK;
}

static int compute_units() {
    static int cus = 0;  // (the library is bound to one device)
    if (cus == 0) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, bound_device()) != hipSuccess) return 0;
        cus = prop.multiProcessorCount;
    }
    return cus;
}

// the kernel that keeps U in LDS: up to 64 rows of 256, 512, 768 or 1024 hidden units (faster than the phased kernel wherever it
// runs: 19 against 21 us per step at 64 rows of 1024, 12 against 13.4 at 32)
static bool lds_kernel_serves(int batch, int hidden, int cus) {
    // DALI_HIP_PERSISTENT_PHASED=1: never this kernel (for comparisons and tests of the other)
    static const bool phased_only = getenv("DALI_HIP_PERSISTENT_PHASED") && atoi(getenv("DALI_HIP_PERSISTENT_PHASED")) == 1;
    if (phased_only || batch > 64 || hidden % 256 != 0 || hidden > 1024) return false;
    int HU = 1;
    while (HU <= 4 && !(hidden % HU == 0 && hidden / HU <= cus)) ++HU;
    return HU <= 4;
}

extern "C" int dali_hip_lstm_recurrent_persistent_supported(int batch, int hidden) {
    if (ensure_init()) return 0;
    const int cus = compute_units();
    if (cus <= 0 || batch < 1) return 0;
    if (!lds_kernel_serves(batch, hidden, cus) && !recurrent_phased_supported(batch, hidden, cus)) return 0;
    // Measured against one fused launch per step, whose inner extent is cut into one share per compute unit at these batches
    // (us per step over 32 steps, persistent / per step). 1024 hidden units: 6.2 / 16.7 at 8 rows, 11.7 / 17.2 at 32, 16.3 / 17.9 at
    // 48, 18.8 / 18.3 at 64, 30.8 / 25.0 at 96; 512: 7.3 / 11.4 at 32, 11.7 / 11.7 at 48, 14.0 / 12.0 at 64; 2048: 27.3 / 40.2 at 32,
    // 40.2 / 40.7 at 48, 52.8 / 40.7 at 64, 104 / 67 at 128.
    return batch <= 32 || (batch <= 48 && hidden >= 1024) ? 2 : 1;
}

extern "C" int dali_hip_lstm_recurrent_persistent(int steps, int batch, int hidden, const float* pre, const float* U, int ldu, const float* h0,
                                                  const float* c0, float* hs, float* c_out) {
    if (ensure_init()) return DALI_HIP_ERROR;
    if (steps < 1 || batch < 1 || hidden < 1) return fail("dali_hip_lstm_recurrent_persistent: steps, batch and hidden must be positive");
    if (!pre || !U || !h0 || !c0 || !hs || !c_out) return fail("dali_hip_lstm_recurrent_persistent: NULL argument");
    if (ldu < 4 * hidden) return fail("dali_hip_lstm_recurrent_persistent: ldu %d is smaller than a row of U (%d)", ldu, 4 * hidden);
    if (((uintptr_t)h0 | (uintptr_t)hs) % 16 != 0) return fail("dali_hip_lstm_recurrent_persistent: h0 and hs must be 16-byte aligned");
    {
        // rows 0 .. steps-2 of hs are overwritten while h0, c0 and pre are still being read
        const char *lo = (const char*)hs, *hi = lo + (size_t)steps * batch * hidden * sizeof(float);
        auto inside = [&](const void* p, size_t bytes) { return (const char*)p < hi && (const char*)p + bytes > lo; };
        if (inside(h0, (size_t)batch * hidden * 4) || inside(c0, (size_t)batch * hidden * 4) || inside(pre, (size_t)steps * batch * hidden * 16))
            return fail("dali_hip_lstm_recurrent_persistent: hs overlaps an input");
    }
    const int cus = compute_units();
    if (cus == 0) return fail("dali_hip_lstm_recurrent_persistent: no device properties");
    if (ensure_status_word("dali_hip_lstm_recurrent_persistent")) return DALI_HIP_ERROR;
    // a launch that finds the flag of an earlier one would leave at its first wait and hand back rows that were never written
    if (__atomic_load_n(g_status, __ATOMIC_RELAXED) != 0)
        return fail("dali_hip_lstm_recurrent_persistent: an earlier persistent launch gave up waiting; call dali_hip_sync to collect that error first");
    if (!lds_kernel_serves(batch, hidden, cus)) {
        if ((size_t)batch * hidden * 4 >= 0x7ffffff0u) return fail("dali_hip_lstm_recurrent_persistent: state rows beyond the 2 GiB a buffer load addresses");
        return lstm_recurrent_phased(steps, batch, hidden, pre, U, ldu, h0, c0, hs, c_out, g_status, cus);
    }
    // fewest hidden units per workgroup that still give every workgroup a compute unit of its own
    int HU = 1;
    while (HU <= 4 && !(hidden % HU == 0 && hidden / HU <= cus)) ++HU;
    const int grid = hidden / HU, MT = (batch + 15) / 16;
    const size_t lds_bytes = ((size_t)hidden * (4 * HU + kPitchPad) + (size_t)4 * MT * 256) * sizeof(float);
    if (lds_bytes > (size_t)160 * 1024 - 1024)
        return fail("dali_hip_lstm_recurrent_persistent: the slice of U per compute unit (%zu bytes) does not fit the LDS", lds_bytes);
    PersistentArgs a;
    a.T = steps; a.B = batch; a.H = hidden; a.HU = HU; a.ldu = ldu;
    a.pre = pre; a.U = U; a.h0 = h0; a.c0 = c0; a.hs = hs; a.c_out = c_out;
    // the last two counters of the workspace (zero at rest, like the reduction tickets)
    a.bar = (unsigned int*)workspace() + kWorkspaceCounters - 2;
    a.done = (unsigned int*)workspace() + kWorkspaceCounters - 1;
    a.status = g_status;
    static const unsigned int spin_env = getenv("DALI_HIP_PERSISTENT_SPIN_LIMIT") ? (unsigned int)atol(getenv("DALI_HIP_PERSISTENT_SPIN_LIMIT")) : (1u << 20);
    a.spin_limit = spin_env;
    hipError_t e = hipSuccess;
    auto launch = [&](auto kernel) {
        e = reserve_dynamic_lds((const void*)kernel, lds_bytes);
        if (e == hipSuccess) hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), lds_bytes, stream(), a);
    };
    const int KQ = hidden / 64;
    // Waiting on the values themselves beats the barrier up to 32 rows (3.7 / 4.9 / 8.8 us a step at 1 / 8 / 32 rows of
    // 1024 units against 6.6 / 7.5 / 10.3); from 33 rows on the tiles that have to be fetched a second time cost more than
    // the barrier (12.8 against 11.3 us at 33 rows, 17.4 against 13.6 at 64). DALI_HIP_PERSISTENT_DATA_FLAGS=0: always barriers.
    static const bool flags_allowed = !(getenv("DALI_HIP_PERSISTENT_DATA_FLAGS") && atoi(getenv("DALI_HIP_PERSISTENT_DATA_FLAGS")) == 0);
    const bool data_flags = flags_allowed && MT <= 2;
#define DALI_PERSISTENT_CASE(mt, kq)                                              \
    if (MT == mt && KQ == kq) {                                                   \
        if (data_flags) launch(lstm_persistent_kernel<mt, kq, (mt <= 2)>);        \
        else launch(lstm_persistent_kernel<mt, kq, false>);                       \
    }
    DALI_PERSISTENT_CASE(1, 4) DALI_PERSISTENT_CASE(2, 4) DALI_PERSISTENT_CASE(3, 4) DALI_PERSISTENT_CASE(4, 4)
    DALI_PERSISTENT_CASE(1, 8) DALI_PERSISTENT_CASE(2, 8) DALI_PERSISTENT_CASE(3, 8) DALI_PERSISTENT_CASE(4, 8)
    DALI_PERSISTENT_CASE(1, 12) DALI_PERSISTENT_CASE(2, 12) DALI_PERSISTENT_CASE(3, 12) DALI_PERSISTENT_CASE(4, 12)
    DALI_PERSISTENT_CASE(1, 16) DALI_PERSISTENT_CASE(2, 16) DALI_PERSISTENT_CASE(3, 16) DALI_PERSISTENT_CASE(4, 16)
#undef DALI_PERSISTENT_CASE
    if (e == hipSuccess) e = hipGetLastError();
    if (e != hipSuccess) return fail("dali_hip_lstm_recurrent_persistent launch failed: %s", hipGetErrorString(e));
    return DALI_HIP_OK;
}

extern "C" int dali_hip_gru_recurrent_persistent_supported(int batch, int hidden) {
    if (ensure_init()) return 0;
    const int cus = compute_units();
    if (cus <= 0 || batch < 1 || !recurrent_phased_supported(batch, hidden, cus)) return 0;
    // measured against the launch-per-step form (us per step): 17 / 25 at 8 rows of 1024, 23 / 32 at 32, 37 / 37 at 64, 57 / 42 at 96; 15 / 18
    // at 8 rows of 512, 29 / 24 at 64; 46 / 44 at 32 rows of 2048: two barriers per step leave less to win than the LSTM's one
    return batch <= 48 && hidden <= 1536 ? 2 : 1;
}

extern "C" int dali_hip_gru_recurrent_persistent(int steps, int batch, int hidden, const float* pre, const float* U, int ldu, const float* h0, float* hs,
                                                 float* scratch) {
    if (ensure_init()) return DALI_HIP_ERROR;
    if (steps < 1 || batch < 1 || hidden < 1) return fail("dali_hip_gru_recurrent_persistent: steps, batch and hidden must be positive");
    if (!pre || !U || !h0 || !hs || !scratch) return fail("dali_hip_gru_recurrent_persistent: NULL argument");
    if (ldu < 3 * hidden) return fail("dali_hip_gru_recurrent_persistent: ldu %d is smaller than a row of U (%d)", ldu, 3 * hidden);
    if (((uintptr_t)h0 | (uintptr_t)hs | (uintptr_t)scratch) % 16 != 0) return fail("dali_hip_gru_recurrent_persistent: h0, hs and scratch must be 16-byte aligned");
    {
        const size_t seq = (size_t)steps * batch * hidden * sizeof(float);
        auto meet = [](const void* p, size_t pb, const void* q, size_t qb) { return (const char*)p < (const char*)q + qb && (const char*)q < (const char*)p + pb; };
        if (meet(hs, seq, h0, (size_t)batch * hidden * 4) || meet(hs, seq, pre, 3 * seq) || meet(scratch, seq, h0, (size_t)batch * hidden * 4) ||
            meet(scratch, seq, pre, 3 * seq) || meet(hs, seq, scratch, seq))
            return fail("dali_hip_gru_recurrent_persistent: hs and scratch must not overlap each other or an input");
    }
    if ((size_t)batch * hidden * 4 >= 0x7ffffff0u) return fail("dali_hip_gru_recurrent_persistent: state rows beyond the 2 GiB a buffer load addresses");
    const int cus = compute_units();
    if (cus == 0) return fail("dali_hip_gru_recurrent_persistent: no device properties");
    if (ensure_status_word("dali_hip_gru_recurrent_persistent")) return DALI_HIP_ERROR;
    if (__atomic_load_n(g_status, __ATOMIC_RELAXED) != 0)
        return fail("dali_hip_gru_recurrent_persistent: an earlier persistent launch gave up waiting; call dali_hip_sync to collect that error first");
    return gru_recurrent_phased(steps, batch, hidden, pre, U, ldu, h0, hs, scratch, g_status, cus);
}

extern "C" int dali_hip_lstm_step_small(int batch, int input, int hidden, const float* X, int ldx, const float* Hprev, int ldh, const float* Cprev,
                                        const float* W, int ldw, const float* U, int ldu, const float* bias, float* Cout, float* Hout) {
    if (ensure_init()) return DALI_HIP_ERROR;
    if (batch < 1 || input < 1 || hidden < 1) return fail("dali_hip_lstm_step_small: batch, input and hidden must be positive");
    if (!X || !Hprev || !Cprev || !W || !U || !bias || !Cout || !Hout) return fail("dali_hip_lstm_step_small: NULL argument");
    if (batch > 64) return fail("dali_hip_lstm_step_small: batch %d exceeds 64 rows (use dali_hip_lstm_step)", batch);
    if (hidden % 256 != 0 || hidden > 1024) return fail("dali_hip_lstm_step_small: hidden %d must be 256, 512, 768 or 1024", hidden);
    // k shares per unit block: as many as bring the grid to about one workgroup per compute unit (256)
    int KS = 4096 / hidden;
    if (KS > kSmallMaxShares) KS = kSmallMaxShares;
    if (KS < 1) KS = 1;
    while (KS > 1 && (input + hidden) % (64 * KS) != 0) KS /= 2;
    if (input % 16 != 0 || (input + hidden) % (64 * KS) != 0)
        return fail("dali_hip_lstm_step_small: input %d must be a multiple of 16 and input + hidden of 64", input);
    if (ldx < input || ldh < hidden || ldw < 4 * hidden || ldu < 4 * hidden) return fail("dali_hip_lstm_step_small: a leading dimension is smaller than its row");
    if ((((uintptr_t)X | (uintptr_t)Hprev | (uintptr_t)W | (uintptr_t)U | (uintptr_t)Cprev | (uintptr_t)Cout | (uintptr_t)Hout) & 15) != 0 || ldx % 4 != 0 ||
        ldh % 4 != 0 || ldw % 4 != 0 || ldu % 4 != 0)
        return fail("dali_hip_lstm_step_small: the matrices must be 16-byte aligned with leading dimensions that are multiples of 4");
    if ((size_t)batch * (size_t)(ldx > ldh ? ldx : ldh) * 4 >= 0x7ffffff0u) return fail("dali_hip_lstm_step_small: operand rows beyond the 2 GiB a buffer load addresses");
    const int unit_blocks = hidden / kSmallUnits;
    if ((size_t)unit_blocks * 4 * KS * batch * kSmallUnits * sizeof(float) > kWorkspacePartialBytes || unit_blocks > kWorkspaceCounters - 2)
        return fail("dali_hip_lstm_step_small: partial sums exceed the workspace");
    SmallStepArgs a;
    a.B = batch; a.I = input; a.H = hidden; a.KS = KS;
    a.X = X; a.Hp = Hprev; a.Cp = Cprev; a.W = W; a.U = U; a.bias = bias; a.Cout = Cout; a.Hout = Hout;
    a.ldx = ldx; a.ldh = ldh; a.ldw = ldw; a.ldu = ldu;
    a.tickets = (unsigned int*)workspace();
    a.partials = (float*)(workspace() + kWorkspaceCounterBytes);
    const int MT = (batch + 15) / 16, grid = unit_blocks * 4 * KS;
    const size_t lds_bytes = (size_t)4 * 4 * MT * 256 * sizeof(float);
    hipError_t e = hipSuccess;
    auto launch = [&](auto kernel) {
        e = reserve_dynamic_lds((const void*)kernel, lds_bytes);
        if (e == hipSuccess) hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), lds_bytes, stream(), a);
    };
    switch (MT) {
        case 1: launch(lstm_step_small_kernel<1, 8>); break;
        case 2: launch(lstm_step_small_kernel<2, 8>); break;
        case 3: launch(lstm_step_small_kernel<3, 8>); break;
        default: launch(lstm_step_small_kernel<4, 8>); break;
    }
    if (e == hipSuccess) e = hipGetLastError();
    if (e != hipSuccess) return fail("dali_hip_lstm_step_small launch failed: %s", hipGetErrorString(e));
    return DALI_HIP_OK;
}
