// fp32 GEMM for grids of many tiles: 128x128 tiles of C, one workgroup per compute unit walking a list of them, operand slabs
// written into LDS by the loads themselves (global_load_lds_dwordx4), four slabs of 32 in flight.
//
// Row-major view: C[M,N] = alpha * A[M,K] * B[K,N] + beta * C with A stored [M][K] or [K][M] and B stored [K][N] or [N][K]
// (dali_hip_sgemm; the reference's call is dali/array/gemm/cublas_gemm.cu:153-166; with a transposed operand the products
// matmul(a.w.transpose(), out_dw) and matmul(out_dw, b.w.transpose()) of dali/tensor/op/dot.cpp:17-18).
//
// Against the 64x64 kernel of the same kind (sgemm_dma.hip) a tile of 128x128 asks the caches for half as many operand bytes
// per flop, which is what limits that kernel once every compute unit runs it (32 KiB per microsecond each). Eight waves
// form 2 x 4 wave tiles of 64 rows x 32 columns; a wave keeps its sums for the whole inner extent, so nothing is exchanged
// at the end of a tile, and the loads of the next tile's first slabs are under way while the sums of this one are stored.
//
// Operands whose k runs across memory rows ([K][N], [K][M]) are read "outer product" fashion: a lane takes a 16-byte piece
// (8 bytes for B) of row k = 4 kk + lane / 16 and feeds its elements to different matrix instructions, so that the 16x16 tile
// of instruction u holds the rows (columns) congruent to u modulo 4 (modulo 2). One 16-byte and one 8-byte LDS read feed
// eight v_mfma_f32_16x16x4_f32; the operand stored [M][K] is read as 16-byte pieces along k, as in the 64x64 kernel, and
// then sixteen reads feed sixty-four instructions.
//
// LDS, per stage of 32 KiB: A (16 KiB) then B. [K][x] operands are kept as rows of 128 x values, 512 bytes, with the
// sixteen-byte piece p of row k in slot p ^ 8 when bit `swizzle_bit` of k is set: the two rows that one pass of an 8-byte
// read touches then lie in different halves of the banks. A stored [M][K] is kept as rows of 32 k values, 128 bytes, piece
// g of row r in slot g ^ ((r >> 1) & 7): the sixteen rows of one pass hit sixteen different slots of a 256-byte bank row.
// A lane of a load always writes bytes [16 lane, 16 lane + 16) of its 1 KiB chunk, so the permutations are applied to the
// global address the lane fetches.
#include <cstdlib>
#include <type_traits>

#include "runtime.h"

namespace dali_hip {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

constexpr int kStageBytes = 32768;
constexpr int kBOffset = 16384;
constexpr int kLdsBytes = 4 * kStageBytes + 16;  // four stages and one flag
constexpr int kDeviceScope = 16;                 // cache policy of a buffer access: device scope (the sc1 bit)

struct Args128 {
    const float* A;
    const float* B;
    int slabs;  // 32-deep slabs of the inner extent, the last one partly filled when ...
    int ktail;  // ... the inner extent is no multiple of 32: values of k in that slab (a multiple of 4), 0 = the slab is whole
    int lda, ldb;
    int M, N;
    float* C;
    int ldc;
    float alpha, beta;
    int tiles_m, tiles_n;
    // The tiles are dealt in `rounds` whole rounds of one tile per workgroup; the `rem` tiles left over (fewer than there are
    // workgroups) are either worked whole by the first `rem` workgroups (shares = 0) or cut along the inner extent into equal
    // shares, one per workgroup (boundaries within `min_frag` slabs of a tile's edge move to the edge).
    int rounds, rem, shares, min_frag;  // shares: workgroups that take a share of the left-over tiles (0: those tiles go whole)
    unsigned int* counters;  // one ticket counter per left-over tile (zero at rest)
    float* partials;         // [2 * workgroups][128 * 128]: a workgroup's share that starts inside a tile, then the one that ends inside one
};

// One 16-byte piece per lane from global memory straight into LDS: lane l writes bytes [16 l, 16 l + 16) behind `lds_addr`
// (wave-uniform, goes through M0); the source is base + voff, base in scalar registers.
__device__ __forceinline__ void load_to_lds(unsigned lds_addr, unsigned voff, const char* base) {
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
template <int N>
__device__ __forceinline__ void wait_but() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
__device__ __forceinline__ void wait_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// TA: A stored as [K][M]. TM: rows of a tile, 128, or 64 for products of at most 64 rows against a wide B (the output
// projection of a decoder step at a batch the row-streaming kernel no longer serves well: such a product is bound by the matrix
// pipe, 4.2 GFLOP at [64,1024].[1024,32000], and 128-row tiles would double that); the wave tiles are then 32 rows high.
// TB: B stored as [N][K]; it is then kept and read like A stored [M][K], and a lane's two 16-column tiles are two runs of
// sixteen consecutive columns. With A stored [K][M] as well, A's rows are read one k at a time (k = 16 t + 4 kq + c, the order
// in which the pieces of B deliver theirs), still four row classes to a 16-byte read.
// SHARE: the launch cuts left-over tiles into shares (the code that publishes and adds them up is left out of the other form,
// where it would sit, unused, behind every slab of the loop).
// KT: the last slab of the inner extent is partly filled. Its loads fetch, for the values of k past the end, a piece that exists
// (the first of the same row, or row 0 of the slab: nothing outside the operands is read), and every lane overwrites what it
// fetched that way with zeros once its loads have landed, before the barrier that releases the slab.
template <bool TA, bool TB, int TM, bool SHARE, bool KT>
__global__ __launch_bounds__(512, 1) void sgemm_dma128_kernel(Args128 g) {
    static_assert(TM == 128 || (TM == 64 && !TA), "64-row tiles are built for A stored [M][K]");
    constexpr bool OUTER = TA && !TB;  // both operands run across memory rows: one k-quad per step
    constexpr int RB = TM / 32;   // 16-row blocks of a wave tile
    constexpr int AQ = TM / 64;   // loads of A per wave and slab
    constexpr int LPS = AQ + 2;   // loads per wave and slab
    // (no static LDS beside this: the loads address LDS from offset 0)
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = w >> 2, wn = w & 3, l16 = lane & 15, kq = lane >> 4;
    const int M = g.M, N = g.N, n = g.slabs;
    // This workgroup's work items: one whole tile per round, then its part of the left-over tiles. Workgroups are numbered die by
    // die (every eighth workgroup runs on the same die): a die takes a contiguous band of the tiles of the whole rounds, and
    // neighbouring shares of a left-over tile belong to workgroups of one die.
    const int G = gridDim.x, wg = blockIdx.x;
    const bool banded = (G & 7) == 0;
    const int p = banded ? (wg & 7) * (G / 8) + wg / 8 : wg;
    const int R = g.rounds;
    const long T2 = (long)g.rem * n;  // slabs of the left-over tiles
    auto bound = [&](int q) __attribute__((always_inline)) -> long {
        if (q >= g.shares) return T2;
        long x = (long)q * T2 / g.shares;
        const int j = (int)(x % n);
        if (j < g.min_frag) x -= j;
        else if (n - j < g.min_frag) x += n - j;
        return x;
    };
    long s2 = 0, e2 = 0;
    if (g.rem > 0) {
        if (SHARE) {
            s2 = bound(p);
            e2 = bound(p + 1);
        } else if (p < g.rem) {
            s2 = (long)p * n;
            e2 = s2 + n;
        }
    }
    const int t2_first = (int)(s2 / n), t2_last = e2 > s2 ? (int)((e2 - 1) / n) : -1;
    const int count2 = e2 > s2 ? t2_last - t2_first + 1 : 0;
    const int count = count2 + R;
    if (count == 0) return;
    const int total = R * n + (int)(e2 - s2);  // slabs of all items of this workgroup
    // item -> tile and slabs [j0, j1) of it. The left-over tiles come first: their shares are then published and added up while
    // everybody still has whole tiles to do, not at the end of the launch with every workgroup waiting on memory.
    auto item_at = [&](int idx, int& tile, int& j0, int& j1) __attribute__((always_inline)) {
        if (idx >= count2) {
            const int r = idx - count2;
            tile = banded ? (wg & 7) * (R * (G / 8)) + r * (G / 8) + wg / 8 : r * G + wg;
            j0 = 0;
            j1 = n;
        } else {
            const int t = t2_first + idx;
            tile = R * G + t;
            j0 = idx == 0 ? (int)(s2 - (long)t2_first * n) : 0;
            j1 = t == t2_last ? (int)(e2 - (long)t * n) : n;
        }
    };
    // Tiles are numbered in column blocks four tiles wide, by rows inside a block: the 32 tiles that the workgroups of a die
    // work on together are 8 x 4 and share their operand slabs in that die's cache.
    auto tile_at = [&](int tile, int& mt, int& nt) __attribute__((always_inline)) {
        const int per_block = g.tiles_m * 4, nb = tile / per_block, rem = tile - nb * per_block;
        const int width = g.tiles_n - 4 * nb < 4 ? g.tiles_n - 4 * nb : 4;
        mt = rem / width;
        nt = 4 * nb + (rem - mt * width);
    };

    const long a_step = (TA ? (long)32 * g.lda : 32L) * (long)sizeof(float);
    const long b_step = (TB ? 32L : (long)32 * g.ldb) * (long)sizeof(float);
    unsigned a_off[2], b_off[2], a_dst[2], b_dst[2];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        a_dst[q] = (unsigned)((w + 8 * q) * 1024);
        b_dst[q] = (unsigned)(kBOffset + (w + 8 * q) * 1024);
    }
    // ---- the side that requests slabs
    int i_r = 0, i_j = 0, i_j1 = 0;
    const char* ap = nullptr;
    const char* bp = nullptr;
    auto request_tile = [&](int r) __attribute__((always_inline)) {
        int tile, j0, mt, nt;
        item_at(r, tile, j0, i_j1);
        tile_at(tile, mt, nt);
        const int m0 = TM * mt, n0 = 128 * nt;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const int c = w + 8 * q;  // 1 KiB chunk of the slab
            if (q >= AQ) {
                a_off[q] = 0;
            } else if (!TA) {
                const int r_in = 8 * c + (lane >> 3), s = lane & 7;
                const int row = m0 + r_in < M ? m0 + r_in : M - 1;
                a_off[q] = (unsigned)(((size_t)row * g.lda + 4 * (s ^ ((r_in >> 1) & 7))) * sizeof(float));
            } else {
                const int k = 2 * c + (lane >> 5), s = lane & 31;
                int col = m0 + 4 * s;
                col = col < M ? col : M - 4;
                a_off[q] = (unsigned)(((size_t)k * g.lda + col) * sizeof(float));
            }
            if (TB) {
                const int r_in = 8 * c + (lane >> 3), s = lane & 7;
                const int row = n0 + r_in < N ? n0 + r_in : N - 1;
                b_off[q] = (unsigned)(((size_t)row * g.ldb + 4 * (s ^ ((r_in >> 1) & 7))) * sizeof(float));
            } else {
                const int k = 2 * c + (lane >> 5), s = lane & 31;
                const int bit = OUTER ? (k & 1) : ((k >> 2) & 1);
                int col = n0 + 4 * (s ^ (bit << 3));
                col = col < N ? col : N - 4;
                b_off[q] = (unsigned)(((size_t)k * g.ldb + col) * sizeof(float));
            }
        }
        i_j = j0;
        ap = wave_uniform((const char*)g.A + (long)j0 * a_step);
        bp = wave_uniform((const char*)g.B + (long)j0 * b_step);
    };
    // (KT) whether this lane's piece of load q lies past the end of the partly filled slab, and how far in front of it (bytes) the
    // piece fetched in its place is
    auto past_end = [&](int q, bool of_b, unsigned* back) __attribute__((always_inline)) -> bool {
        const int c = w + 8 * q;
        if (of_b ? TB : !TA) {  // the eight pieces of an LDS row run along k
            const int r_in = 8 * c + (lane >> 3), pk = (lane & 7) ^ ((r_in >> 1) & 7);
            *back = 16u * (unsigned)pk;
            return 4 * pk >= g.ktail;
        }
        const int k = 2 * c + (lane >> 5);
        *back = (unsigned)k * (unsigned)(of_b ? g.ldb : g.lda) * 4u;
        return k >= g.ktail;
    };
    unsigned tail_stages = 0;  // (KT) bit s: the slab in stage s is the partly filled one
    auto issue = [&](int stage) __attribute__((always_inline)) {
        if (KT && i_j == n - 1) {
            unsigned back;
            tail_stages |= 1u << stage;
            load_to_lds(a_dst[0] + stage * kStageBytes, past_end(0, false, &back) ? a_off[0] - back : a_off[0], ap);
            if (AQ > 1) load_to_lds(a_dst[1] + stage * kStageBytes, past_end(1, false, &back) ? a_off[1] - back : a_off[1], ap);
            load_to_lds(b_dst[0] + stage * kStageBytes, past_end(0, true, &back) ? b_off[0] - back : b_off[0], bp);
            load_to_lds(b_dst[1] + stage * kStageBytes, past_end(1, true, &back) ? b_off[1] - back : b_off[1], bp);
        } else {
            if (KT) tail_stages &= ~(1u << stage);
            load_to_lds(a_dst[0] + stage * kStageBytes, a_off[0], ap);
            if (AQ > 1) load_to_lds(a_dst[1] + stage * kStageBytes, a_off[1], ap);
            load_to_lds(b_dst[0] + stage * kStageBytes, b_off[0], bp);
            load_to_lds(b_dst[1] + stage * kStageBytes, b_off[1], bp);
        }
        ++i_j;
        ap += a_step;
        bp += b_step;
        if (i_j == i_j1) {
            ++i_r;
            if (i_r < count) request_tile(i_r);
        }
    };
    request_tile(0);
    issue(0);
    if (total > 1) issue(1);
    if (total > 2) issue(2);

    // ---- operand addresses of this lane within a stage
    // [K][x] operands: row 4 kk + kq of the slab; A [M][K]: row block rb of the wave tile, piece 4 t + kq
    unsigned a_addr[4], b_addr, b_addr_t[2];
    if (TA) {
        a_addr[0] = (unsigned)(kq * (OUTER ? 512 : 2048) + (wm * 64 + 4 * l16) * 4);  // row kq, or row 4 kq of a k-group
        a_addr[1] = a_addr[2] = a_addr[3] = 0;
    } else {
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) {
            const int r_in = wm * (TM / 2) + 16 * rb + l16;
            a_addr[rb] = rb < RB ? (unsigned)(r_in * 128 + ((kq ^ ((r_in >> 1) & 7)) * 16)) : 0u;  // piece kq of k-group 0; k-group 1 flips bit 2 of the slot
        }
    }
    // (the swizzle bit of B's row is bit 0 of kq in both forms: k = 4 kk + kq, or (k >> 2) = 4 t + kq)
    b_addr = (unsigned)(kBOffset + ((wn * 8 + (l16 >> 1)) ^ ((kq & 1) << 3)) * 16 + (l16 & 1) * 8);
#pragma unroll
    for (int cb = 0; cb < 2; ++cb) {
        const int r_in = wn * 32 + 16 * cb + l16;
        b_addr_t[cb] = (unsigned)(kBOffset + r_in * 128 + ((kq ^ ((r_in >> 1) & 7)) * 16));
    }

    floatx4 acc[RB][2];
    auto clear = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < RB; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.f;
    };
    clear();
    // Operand registers, two sets. TA: set o holds one k-quad (a: 4 rows congruent classes, b: 2 column classes).
    // !TA: set o holds one k-group of 16 (a[rb]: four k of row block rb, b[c]: row 16 t + 4 kq + c).
    floatx4 a_tn[2];
    floatx2 b_tn[2];
    floatx4 a_nn[2][4];  // A [M][K]: [row block] with four k; A [K][M] beside B [N][K]: [c] with four row classes
    floatx2 b_nn[2][4];
    floatx4 b_nt[2][2];  // B [N][K]: [column block] with four k
    auto load_ops = [&](auto ST, int step, int o) __attribute__((always_inline)) {
        constexpr int st = decltype(ST)::value;
        const char* base = lds + st * kStageBytes;
        if (OUTER) {
            // step = kk (0..7)
            a_tn[o] = *(const floatx4*)(base + a_addr[0] + step * 2048);
            b_tn[o] = *(const floatx2*)(base + b_addr + kq * 512 + step * 2048);
        } else {
            // step = t (0..1)
            if (TA) {
#pragma unroll
                for (int c = 0; c < 4; ++c) a_nn[o][c] = *(const floatx4*)(base + a_addr[0] + (16 * step + c) * 512);
            } else {
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) a_nn[o][rb] = *(const floatx4*)(base + (a_addr[rb] ^ (unsigned)(step * 64)));
            }
            if (TB) {
#pragma unroll
                for (int cb = 0; cb < 2; ++cb) b_nt[o][cb] = *(const floatx4*)(base + (b_addr_t[cb] ^ (unsigned)(step * 64)));
            } else {
#pragma unroll
                for (int c = 0; c < 4; ++c) b_nn[o][c] = *(const floatx2*)(base + b_addr + (16 * step + 4 * kq + c) * 512);
            }
        }
    };
    // eight matrix instructions on independent sums
    auto mfma_tn = [&](int o) __attribute__((always_inline)) {
#pragma unroll
        for (int ua = 0; ua < RB; ++ua)
#pragma unroll
            for (int ub = 0; ub < 2; ++ub) acc[ua][ub] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_tn[o][ua], b_tn[o][ub], acc[ua][ub], 0, 0, 0);
    };
    auto mfma_nn = [&](int o, int c) __attribute__((always_inline)) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int ub = 0; ub < 2; ++ub)
                acc[rb][ub] = __builtin_amdgcn_mfma_f32_16x16x4f32(TA ? a_nn[o][c][rb] : a_nn[o][rb][c], TB ? b_nt[o][ub][c] : b_nn[o][c][ub], acc[rb][ub], 0, 0, 0);
    };

    // ---- the side that multiplies
    int c_r = 0, c_tile, c_j0, c_j, c_j1;
    item_at(0, c_tile, c_j0, c_j1);
    c_j = c_j0;
    volatile int& is_last = *(volatile int*)(lds + 4 * kStageBytes);
    // slabs [c_j0, c_j1) of tile c_tile are summed: a whole tile goes to C; a share of a left-over tile is published in the
    // workspace and a ticket drawn, and whoever draws the tile's last ticket adds the shares in the order of their slabs (its
    // own from registers), so the sum does not depend on who that is
    auto finish_tile = [&]() __attribute__((always_inline)) {
        bool store = true;
        if (SHARE && (c_j0 != 0 || c_j1 != n)) {
            const int t = c_tile - R * G;  // left-over tile
            // the workgroups whose shares meet in this tile: q0 .. q1 (those of them with a share at all)
            auto owner_of = [&](long it) __attribute__((always_inline)) -> int {
                int q = (int)(it * g.shares / T2);
                q = q < 0 ? 0 : (q > g.shares - 1 ? g.shares - 1 : q);
                while (q + 1 < g.shares && bound(q + 1) <= it) ++q;
                while (bound(q) > it) --q;
                return q;
            };
            const int q0 = owner_of((long)t * n), q1 = owner_of((long)(t + 1) * n - 1);
            int sharers = 0;
            for (int q = q0; q <= q1; ++q) sharers += bound(q + 1) > bound(q) ? 1 : 0;
            // (16-byte device-scope accesses: written through to, and read from, the memory that all dies share)
            float* mine = g.partials + (size_t)(c_j0 > 0 ? 2 * p : 2 * p + 1) * 16384;
            const __amdgpu_buffer_rsrc_t mine_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)mine, 0, 65536, 0x00027000);
#pragma unroll
            for (int i = 0; i < RB; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(__attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned, acc[i][j]), mine_rsrc,
                                                           ((i * 2 + j) * 512 + tid) * 16, 0, kDeviceScope);
            // the share is acknowledged by memory before the ticket is drawn
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            __syncthreads();
            if (tid == 0) {
                const unsigned int ticket = __hip_atomic_fetch_add(g.counters + t, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                is_last = ticket == (unsigned int)sharers - 1;
            }
            __syncthreads();
            store = __builtin_amdgcn_readfirstlane(is_last) != 0;
            if (store) {
                floatx4 sum[RB][2];
#pragma unroll
                for (int i = 0; i < RB; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j) sum[i][j] = (floatx4){0.f, 0.f, 0.f, 0.f};
                for (int q = q0; q <= q1; ++q) {
                    const long qb = bound(q);
                    if (bound(q + 1) <= qb) continue;
                    if (q == p) {
#pragma unroll
                        for (int i = 0; i < RB; ++i)
#pragma unroll
                            for (int j = 0; j < 2; ++j) sum[i][j] += acc[i][j];
                    } else {
                        const float* theirs = g.partials + (size_t)(qb > (long)t * n ? 2 * q : 2 * q + 1) * 16384;
                        const __amdgpu_buffer_rsrc_t their_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)theirs, 0, 65536, 0x00027000);
                        floatx4 got[RB][2];
#pragma unroll
                        for (int i = 0; i < RB; ++i)
#pragma unroll
                            for (int j = 0; j < 2; ++j)
                                got[i][j] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(their_rsrc, ((i * 2 + j) * 512 + tid) * 16, 0, kDeviceScope));
#pragma unroll
                        for (int i = 0; i < RB; ++i)
#pragma unroll
                            for (int j = 0; j < 2; ++j) sum[i][j] += got[i][j];
                    }
                }
#pragma unroll
                for (int i = 0; i < RB; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j) acc[i][j] = sum[i][j];
                if (tid == 0) __hip_atomic_store(g.counters + t, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        int mt, nt;
        tile_at(c_tile, mt, nt);
        const int m_base = TM * mt + wm * (TM / 2), nn = 128 * nt + wn * 32 + 2 * l16;
        const float alpha = g.alpha, beta = g.beta;
        if (!store) {
        } else if (TB) {
            // a lane's two sums of a row are sixteen columns apart
#pragma unroll
            for (int i = 0; i < RB; ++i)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int m = m_base + (TA ? 16 * kq + 4 * v + i : 16 * i + 4 * kq + v);
#pragma unroll
                    for (int cb = 0; cb < 2; ++cb) {
                        const int col = 128 * nt + wn * 32 + 16 * cb + l16;
                        if (m < M && col < N) {
                            float* c = g.C + (size_t)m * g.ldc + col;
                            float r = alpha * acc[i][cb][v];
                            if (beta != 0.f) r += beta * *c;
                            *c = r;
                        }
                    }
                }
        } else if (nn < N) {  // (N is a multiple of 4 and nn even: nn + 1 < N as well)
#pragma unroll
            for (int i = 0; i < RB; ++i)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    // TA: the tile of instruction i holds the rows congruent to i modulo 4; else row block i
                    const int m = m_base + (TA ? 16 * kq + 4 * v + i : 16 * i + 4 * kq + v);
                    if (m < M) {
                        floatx2* c = (floatx2*)(g.C + (size_t)m * g.ldc + nn);
                        floatx2 r;
                        r[0] = alpha * acc[i][0][v];
                        r[1] = alpha * acc[i][1][v];
                        if (beta != 0.f) {
                            const floatx2 old = *c;
                            r[0] += beta * old[0];
                            r[1] += beta * old[1];
                        }
                        *c = r;
                    }
                }
        }
        clear();
        ++c_r;
        if (c_r < count) {
            item_at(c_r, c_tile, c_j0, c_j1);
            c_j = c_j0;
        }
    };
    auto zero_past_end = [&](int stage) __attribute__((always_inline)) {
        const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
        unsigned back;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            if (q < AQ && past_end(q, false, &back)) *(floatx4*)(lds + a_dst[q] + stage * kStageBytes + 16 * lane) = zero;
            if (past_end(q, true, &back)) *(floatx4*)(lds + b_dst[q] + stage * kStageBytes + 16 * lane) = zero;
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
    // Slab i lives in stage i % 4. The barrier inside slab i is for slab i+1 (its loads were issued two slabs earlier); behind
    // it the buffer of slab i-1 is free and takes slab i+3.
    auto slab_step = [&](auto ST, auto H1, auto H2, auto H3) __attribute__((always_inline)) {
        constexpr int st = decltype(ST)::value;
        constexpr bool has1 = decltype(H1)::value, has2 = decltype(H2)::value, has3 = decltype(H3)::value;
        using NX = std::integral_constant<int, (st + 1) % 4>;
        if (OUTER) {
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) {
                if (kk < 7) load_ops(ST, kk + 1, (kk + 1) & 1);
                else if (has1) load_ops(NX{}, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                mfma_tn(kk & 1);
                if (kk == 1 && has1) {
                    if (has2) wait_but<LPS>(); else wait_all();
                    if (KT && ((tail_stages >> ((st + 1) % 4)) & 1u)) zero_past_end((st + 1) % 4);
                    __builtin_amdgcn_s_barrier();
                }
                if (kk == 2 && has3) issue((st + 3) % 4);
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
            load_ops(ST, 1, 1);
            __builtin_amdgcn_sched_barrier(0);
            mfma_nn(0, 0);
            if (has1) {
                if (has2) wait_but<LPS>(); else wait_all();
                if (KT && ((tail_stages >> ((st + 1) % 4)) & 1u)) zero_past_end((st + 1) % 4);
                __builtin_amdgcn_s_barrier();
            }
            __builtin_amdgcn_sched_barrier(0);
            mfma_nn(0, 1);
            if (has3) issue((st + 3) % 4);
            __builtin_amdgcn_sched_barrier(0);
            mfma_nn(0, 2);
            __builtin_amdgcn_sched_barrier(0);
            mfma_nn(0, 3);
            __builtin_amdgcn_sched_barrier(0);
            if (has1) load_ops(NX{}, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            mfma_nn(1, 0);
            __builtin_amdgcn_sched_barrier(0);
            mfma_nn(1, 1);
            __builtin_amdgcn_sched_barrier(0);
            mfma_nn(1, 2);
            __builtin_amdgcn_sched_barrier(0);
            mfma_nn(1, 3);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (++c_j == c_j1) finish_tile();
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
    // slab 0 has landed once at most the loads of slabs 1 and 2 are outstanding
    if (total > 2) wait_but<2 * LPS>();
    else if (total > 1) wait_but<LPS>();
    else wait_all();
    if (KT && (tail_stages & 1u)) zero_past_end(0);  // (a share that is the last slab of its tile alone)
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

bool aligned_to(const void* p, size_t a) { return ((uintptr_t)p & (a - 1)) == 0; }

template <bool TA, bool TB, int TM, bool SHARE, bool KT = false>
int launch128(const Args128& g, int workgroups) {
    auto kernel = sgemm_dma128_kernel<TA, TB, TM, SHARE, KT>;
    hipError_t e = reserve_dynamic_lds((const void*)kernel, kLdsBytes);
    if (e != hipSuccess) return fail("sgemm: cannot reserve %d bytes of LDS: %s", kLdsBytes, hipGetErrorString(e));
    hipLaunchKernelGGL(kernel, dim3(workgroups), dim3(512), kLdsBytes, stream(), g);
    e = hipGetLastError();
    if (e != hipSuccess) return fail("sgemm launch failed: %s", hipGetErrorString(e));
    return 1;
}

}  // namespace

int sgemm_dma128(bool ta, bool tb, int M, int N, int K, const float* A, int lda, const float* B, int ldb, float alpha, float beta, float* C, int ldc, int cus) {
    static const int enabled = getenv("DALI_HIP_GEMM_DMA128") ? atoi(getenv("DALI_HIP_GEMM_DMA128")) : 1;
    static const int tails_on = getenv("DALI_HIP_GEMM_DMA_TAILS") ? atoi(getenv("DALI_HIP_GEMM_DMA_TAILS")) : 1;
    if (!enabled || cus < 8 || M < 1 || N < 4 || K < 32 || K % (tails_on ? 4 : 32) != 0) return 0;
    // 16-byte pieces that start on 16-byte boundaries and never straddle the end of a row; with B stored [K][N] pairs of results
    // are stored as 8 bytes
    if (lda % 4 != 0 || ldb % 4 != 0 || (ta && (M % 4 != 0 || M < 4))) return 0;
    if (!tb && (N % 4 != 0 || ldc % 2 != 0 || !aligned_to(C, 8))) return 0;
    if (!aligned_to(A, 16) || !aligned_to(B, 16)) return 0;
    // per-lane offsets are 32-bit and relative to a pointer that walks along k
    const size_t a_span = ((size_t)(ta ? 32 : M) * lda + (ta ? M : 32)) * sizeof(float);
    const size_t b_span = ((size_t)(tb ? N : 32) * ldb + (tb ? 32 : N)) * sizeof(float);
    if (a_span >= ((size_t)1 << 32) || b_span >= ((size_t)1 << 32)) return 0;
    Args128 g = {};
    g.A = A;
    g.B = B;
    g.slabs = (K + 31) / 32;
    g.ktail = K % 32;
    const bool kt = g.ktail != 0;
    g.lda = lda;
    g.ldb = ldb;
    g.M = M;
    g.N = N;
    g.C = C;
    g.ldc = ldc;
    g.alpha = alpha;
    g.beta = beta;
    const bool low = !ta && !tb && M <= 64;  // one row of 64-row tiles
    g.tiles_m = low ? 1 : (M + 127) / 128;
    g.tiles_n = (N + 127) / 128;
    const long tiles = (long)g.tiles_m * g.tiles_n;
    if (tiles > (1L << 24)) return 0;
    int workgroups = cus - cus % 8;  // every workgroup has a compute unit to itself (its LDS); whole dies keep the bands of tiles
    // Tiles that do not fill a last round are cut along the inner extent into shares, one per workgroup, unless the inner extent
    // is short (fewer than eight
    // slabs (3072x1536 over K = 4096, 288 tiles on 256 compute units: 77 -> 112 TFLOP/s).
    static const int share_env = getenv("DALI_HIP_GEMM_SHARE_REST") ? atoi(getenv("DALI_HIP_GEMM_SHARE_REST")) : 1;
    const int rest = (int)(tiles % workgroups);
    // (a share costs about 5 us to publish and 5 us to add up: with no whole round to hide behind, inner extents under 1536 gain nothing)
    const bool share = share_env && !low && rest > 0 && workgroups <= 256 && g.slabs >= (tiles < workgroups ? 48 : 16) &&
                       (size_t)2 * workgroups * 16384 * sizeof(float) <= kWorkspacePartialBytes && rest <= kWorkspaceCounters;
    if (!share && tiles < workgroups) workgroups = (int)tiles;
    g.rounds = (int)(tiles / workgroups);
    g.rem = (int)(tiles % workgroups);
    // at most four workgroups to a tile (a fifth where the cuts fall unevenly): whoever adds the shares up fetches 64 KiB for each
    g.shares = share ? (4 * rest < workgroups ? 4 * rest : workgroups) : 0;
    g.min_frag = 2;
    g.counters = (unsigned int*)workspace();
    g.partials = (float*)(workspace() + kWorkspaceCounterBytes);
    if (low) return kt ? launch128<false, false, 64, false, true>(g, workgroups) : launch128<false, false, 64, false>(g, workgroups);
    if (kt) {
        // (whole tiles only: a product whose left-over tiles would be cut into shares has its whole slabs done that way and the
        // rest of the inner extent added by the caller)
        if (share) return 0;
        if (!ta && !tb) return launch128<false, false, 128, false, true>(g, workgroups);
        if (ta && !tb) return launch128<true, false, 128, false, true>(g, workgroups);
        if (!ta && tb) return launch128<false, true, 128, false, true>(g, workgroups);
        return launch128<true, true, 128, false, true>(g, workgroups);
    }
    if (share) {
        if (!ta && !tb) return launch128<false, false, 128, true>(g, workgroups);
        if (ta && !tb) return launch128<true, false, 128, true>(g, workgroups);
        if (!ta && tb) return launch128<false, true, 128, true>(g, workgroups);
        return launch128<true, true, 128, true>(g, workgroups);
    }
    if (!ta && !tb) return launch128<false, false, 128, false>(g, workgroups);
    if (ta && !tb) return launch128<true, false, 128, false>(g, workgroups);
    if (!ta && tb) return launch128<false, true, 128, false>(g, workgroups);
    return launch128<true, true, 128, false>(g, workgroups);
}

}  // namespace dali_hip
