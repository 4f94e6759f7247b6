// Stable ordering of int32 keys on the device, for the scatter path
// (assignment through op::gather, dali/array/op/gather.cpp:89-97,126-143).
//
// The reference's GPU code scatters with atomicAdd (gather.cpp:14-28), so the order in which
// duplicates of an index are added varies from run to run. Here the indices are ordered first
// (stable radix sort: equal keys keep their input order) and every destination row then adds its
// contributions one after the other in input order, which is exactly the order of the reference's
// sequential CPU loop.
#include "runtime.h"

#include <cstdlib>
#include <type_traits>

namespace dali_hip {

// A few thousand keys: counting ranks beats any multi-pass sort. The final position of key i is the number of
// (key, position) pairs that order before it. A workgroup counts, for 256 keys, the smaller pairs within one
// segment of the input (staged in LDS, read as wave-wide broadcasts) and publishes the counts; the workgroup that
// finishes last for those 256 keys (a ticket per key block) adds the segments' counts and places the keys.
// n * n comparisons, but spread over the whole chip, in one launch and without an allocation: the counts and the
// tickets live in the library workspace. When key_limit * 2^ceil(log2 n) fits 32 bits a pair is one 32-bit word
// (key in the high bits, position in the low ones), which halves the cost of a comparison.
template <typename W>
__device__ __forceinline__ W rank_pair(int32_t key, int pos, int shift, int limit);
template <>
__device__ __forceinline__ unsigned long long rank_pair<unsigned long long>(int32_t key, int pos, int, int limit) {
    // with a key limit, a key outside [0, limit) is ordered as `limit`: behind every valid key
    if (limit > 0 && (unsigned int)key >= (unsigned int)limit) key = limit;
    return ((unsigned long long)((unsigned int)key ^ 0x80000000u) << 32) | (unsigned int)pos;  // signed key order
}
template <>
__device__ __forceinline__ unsigned int rank_pair<unsigned int>(int32_t key, int pos, int shift, int) {
    // a key outside [0, key_limit) (an invalid index) is ordered behind the largest valid key (the packed form is chosen
    // only when that value fits): whatever the input, the words stay distinct, so the positions computed from them are
    // a permutation, and a run of equal valid keys is never interrupted
    const unsigned int top = (0xFFFFFFFFu >> shift);
    const unsigned int k = (unsigned int)key < top ? (unsigned int)key : top;
    return (k << shift) | (unsigned int)pos;
}

constexpr int kRankSegment = 512;
constexpr int kRankMaxSegments = 32;  // 16384 keys

template <typename W>
__global__ __launch_bounds__(256) void rank_sort_kernel(const int32_t* keys, int n, int shift, int limit, int segments, int32_t* partial,
                                                         unsigned int* tickets, int32_t* sorted_keys, int32_t* perm) {
    __shared__ __attribute__((aligned(16))) W tile[kRankSegment];
    __shared__ int is_last;
    const int i = blockIdx.x * 256 + threadIdx.x;
    const int j0 = blockIdx.y * kRankSegment;
    for (int t = threadIdx.x; t < kRankSegment; t += 256) {
        const int j = j0 + t;
        tile[t] = j < n ? rank_pair<W>(keys[j], j, shift, limit) : ~(W)0;  // padding orders after (or with) every real pair
    }
    __syncthreads();
    const int32_t my_key = i < n ? keys[i] : 0;
    const W mine = rank_pair<W>(my_key, i, shift, limit);
    int count = 0;
#pragma unroll 16
    for (int t = 0; t < kRankSegment; ++t) count += tile[t] < mine ? 1 : 0;
    if (i < n) __hip_atomic_store(partial + (size_t)blockIdx.y * n + i, count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // the counts are acknowledged by memory before the ticket is drawn; the clobber keeps the compiler from moving the stores
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned int ticket = __hip_atomic_fetch_add(tickets + blockIdx.x, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        is_last = ticket == (unsigned int)segments - 1;
    }
    __syncthreads();
    if (!is_last) return;
    if (i < n) {
        // all segments' counts are requested before the first one is waited for (a loop of run-time length would wait
        // for every load in turn)
        int part[kRankMaxSegments];
#pragma unroll
        for (int s = 0; s < kRankMaxSegments; ++s)
            part[s] = s < segments ? __hip_atomic_load(partial + (size_t)s * n + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0;
        int pos = 0;
#pragma unroll
        for (int s = 0; s < kRankMaxSegments; ++s) pos += part[s];
        sorted_keys[pos] = my_key;
        perm[pos] = i;
    }
    if (threadIdx.x == 0) __hip_atomic_store(tickets + blockIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}


// ---------------------------------------------------------------- more than 16384 keys: least-significant-digit radix sort
// Eight bits per pass over (key, position) pairs. A workgroup owns a tile of 2048 consecutive pairs. Pass = three
// launches: (1) a histogram of the tile's digits, stored digit-major [256][tiles]; (2) an exclusive scan over that table,
// which turns every entry into the first output slot of (digit, tile); (3) the move: a pair goes to that slot plus its
// rank among the tile's pairs with the same digit that come before it. The rank is exact, not "whoever gets there
// first", so every pass is stable and equal keys end up in input order: a thread holds eight pairs (one per round of 256),
// a wave finds the lanes with its digit from eight ballots (one per bit), the lowest such lane records how many there
// are per (round, wave, digit), and a scan over the 32 (round, wave) slots of every digit gives each group its offset.
// A workgroup of 256 threads works on a tile of 256 * ROUNDS keys: 8 rounds for long inputs (fewest counters), fewer for
// short ones so that the tiles still cover the chip (65536 keys in tiles of 2048 are 32 workgroups on 256 CUs).
constexpr int kRadixMaxTile = 2048;

// Where a pair's digit comes from. The sort itself only needs "the digit of pair i in this pass":
// IndexDigits: int32 keys. With a key limit, every key outside [0, limit) takes the digits of `limit` itself: such keys (invalid
// indices) end up behind all valid ones, in input order, instead of between the keys that share their low bits.
struct IndexDigits {
    unsigned int flip, limit;
    __device__ __forceinline__ unsigned int operator()(int32_t key, int32_t, int shift) const {
        unsigned int k = (unsigned int)key ^ flip;
        if (limit != 0u && k > limit) k = limit;
        return (k >> shift) & 255u;
    }
};
// WordDigits: unsigned keys ordered as they stand (values of any type mapped to words of the same order beforehand)
struct WordDigits {
    template <typename KEY>
    __device__ __forceinline__ unsigned int operator()(KEY key, int32_t, int shift) const {
        return (unsigned int)(key >> shift) & 255u;
    }
};
// RowDigits: the row of a [rows, cols] matrix that the pair started in (its position / cols): stable passes over these
// digits after the passes over the keys leave every row's pairs together, in key order. The keys are not looked at.
struct RowDigits {
    int cols;
    template <typename KEY>
    __device__ __forceinline__ unsigned int operator()(KEY, int32_t pos, int shift) const {
        return ((unsigned int)(pos / cols) >> shift) & 255u;
    }
};

// keys == nullptr: the digits come from the positions alone; pos_in == nullptr: a pair's position is its index
template <int ROUNDS, typename KEY, typename DIGITS>
__global__ __launch_bounds__(256) void radix_hist_kernel(const KEY* keys, const int32_t* pos_in, int n, int shift, DIGITS digits, unsigned int* hist, int tiles) {
    __shared__ unsigned int h[256];
    h[threadIdx.x] = 0u;
    __syncthreads();
    const long base = (long)blockIdx.x * (256 * ROUNDS);
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
        const long i = base + r * 256 + threadIdx.x;
        if (i < n) atomicAdd(&h[digits(keys ? keys[i] : (KEY)0, pos_in ? pos_in[i] : (int32_t)i, shift)], 1u);
    }
    __syncthreads();
    hist[(long)threadIdx.x * tiles + blockIdx.x] = h[threadIdx.x];
}

// The counters are laid out digit-major ([digit][tile]); a key's slot is (keys with smaller digits) + (keys of its digit in
// earlier tiles) + (its rank within the tile). One workgroup per digit scans that digit's row of counters in place
// (exclusive, coalesced, 256 at a time) and leaves the row's total; the move kernel adds the totals of the smaller digits.
// (A single workgroup walking all 256 * tiles counters took 300 us for 1024 tiles, more than the rest of the sort.)
__global__ __launch_bounds__(256) void radix_row_scan_kernel(unsigned int* hist, int tiles, unsigned int* totals) {
    __shared__ unsigned int wave_sum[4];
    unsigned int* row = hist + (long)blockIdx.x * tiles;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    unsigned int carry = 0;
    for (int base = 0; base < tiles; base += 256) {
        const int i = base + threadIdx.x;
        const unsigned int v = i < tiles ? row[i] : 0u;
        unsigned int incl = v;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const unsigned int o = __shfl_up(incl, d, 64);
            if (lane >= d) incl += o;
        }
        if (lane == 63) wave_sum[wave] = incl;
        __syncthreads();
        unsigned int before = 0, total = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            if (w < wave) before += wave_sum[w];
            total += wave_sum[w];
        }
        if (i < tiles) row[i] = carry + before + incl - v;
        carry += total;
        __syncthreads();
    }
    if (threadIdx.x == 0) totals[blockIdx.x] = carry;
}

template <int ROUNDS, typename KEY, typename DIGITS>
__global__ __launch_bounds__(256) void radix_move_kernel(const KEY* keys_in, const int32_t* pos_in, int n, int shift, DIGITS digits, const unsigned int* hist,
                                                         const unsigned int* totals, int tiles, KEY* keys_out, int32_t* pos_out) {
    __shared__ unsigned short cnt[ROUNDS * 4][256];
    __shared__ unsigned int first_slot[256];
    __shared__ unsigned int wave_total[4];
    for (int t = threadIdx.x; t < ROUNDS * 4 * 256; t += 256) (&cnt[0][0])[t] = 0;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    {
        // keys with smaller digits: exclusive scan of the 256 digit totals, thread d for digit d
        const unsigned int mine = totals[threadIdx.x];
        unsigned int incl = mine;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const unsigned int o = __shfl_up(incl, d, 64);
            if (lane >= d) incl += o;
        }
        if (lane == 63) wave_total[wave] = incl;
        __syncthreads();
        unsigned int before = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w)
            if (w < wave) before += wave_total[w];
        first_slot[threadIdx.x] = before + incl - mine + hist[(long)threadIdx.x * tiles + blockIdx.x];
    }
    __syncthreads();
    const unsigned long long below = (1ull << lane) - 1ull;
    const long base = (long)blockIdx.x * (256 * ROUNDS);
    KEY key[ROUNDS];
    int32_t pos[ROUNDS];
    unsigned int digit[ROUNDS], rank[ROUNDS];
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
        const long i = base + r * 256 + threadIdx.x;
        const bool valid = i < n;
        key[r] = valid && keys_in ? keys_in[i] : (KEY)0;
        pos[r] = valid ? (pos_in ? pos_in[i] : (int32_t)i) : 0;
        digit[r] = digits(key[r], pos[r], shift);
        unsigned long long same = __ballot(valid);
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const unsigned long long m = __ballot((digit[r] >> b) & 1u);
            same &= ((digit[r] >> b) & 1u) ? m : ~m;
        }
        rank[r] = (unsigned int)__popcll(same & below);
        if (valid && rank[r] == 0) cnt[r * 4 + wave][digit[r]] = (unsigned short)__popcll(same);
    }
    __syncthreads();
    {
        unsigned int run = 0;
#pragma unroll
        for (int s = 0; s < ROUNDS * 4; ++s) {
            const unsigned int c = cnt[s][threadIdx.x];
            cnt[s][threadIdx.x] = (unsigned short)run;
            run += c;
        }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
        const long i = base + r * 256 + threadIdx.x;
        if (i < n) {
            const unsigned int dst = first_slot[digit[r]] + cnt[r * 4 + wave][digit[r]] + rank[r];
            if (keys_in) keys_out[dst] = key[r];
            pos_out[dst] = pos[r];
        }
    }
}

// One pass of the radix sort over n pairs in tiles of 256 * rounds: histogram, scan, move (see above)
template <typename KEY, typename DIGITS>
static void radix_pass(int rounds, const KEY* src_keys, const int32_t* src_pos, int n, int shift, DIGITS digits, unsigned int* hist, unsigned int* totals, int tiles,
                       KEY* dst_keys, int32_t* dst_pos, hipStream_t st) {
    auto pass = [&](auto hist_kernel, auto move_kernel) {
        hipLaunchKernelGGL(hist_kernel, dim3(tiles), dim3(256), 0, st, src_keys, src_pos, n, shift, digits, hist, tiles);
        hipLaunchKernelGGL(radix_row_scan_kernel, dim3(256), dim3(256), 0, st, hist, tiles, totals);
        hipLaunchKernelGGL(move_kernel, dim3(tiles), dim3(256), 0, st, src_keys, src_pos, n, shift, digits, (const unsigned int*)hist, (const unsigned int*)totals, tiles,
                           dst_keys, dst_pos);
    };
    switch (rounds) {
        case 1: pass(radix_hist_kernel<1, KEY, DIGITS>, radix_move_kernel<1, KEY, DIGITS>); break;
        case 2: pass(radix_hist_kernel<2, KEY, DIGITS>, radix_move_kernel<2, KEY, DIGITS>); break;
        case 4: pass(radix_hist_kernel<4, KEY, DIGITS>, radix_move_kernel<4, KEY, DIGITS>); break;
        default: pass(radix_hist_kernel<8, KEY, DIGITS>, radix_move_kernel<8, KEY, DIGITS>); break;
    }
}

// tile height for n pairs: 8 rounds for long inputs, fewer while the tiles would not cover the chip
static int radix_rounds(long n) {
    int rounds = kRadixMaxTile / 256;
    while (rounds > 1 && n / (256 * rounds) < 1024) rounds /= 2;
    return rounds;
}

// ---------------------------------------------------------------- ordering along rows (top_k / bottom_k / argsort)
// The values of one dense [rows, cols] matrix become unsigned words whose ascending order is the order asked for: the
// value's bits with the sign bit set for non-negative numbers and all bits inverted for negative ones (two's complement
// integers: the sign bit flipped), everything inverted once more when the largest come first. -0.0 becomes +0.0 first,
// so that the two compare equal, as they do for the reference's comparators. With `reverse` a row is laid out back to
// front, so that the stable sort which follows leaves equal keys in descending column order. The whole matrix is then
// sorted as one sequence by word (stable passes, lowest digit first) and after that by the row a pair started in: every
// row's pairs end up together and in order.
template <typename T>
struct OrderedWord;
template <>
struct OrderedWord<float> {
    typedef unsigned int type;
    static __device__ __forceinline__ type of(float v) {
        const unsigned int b = __float_as_uint(v + 0.f);
        return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
    }
};
template <>
struct OrderedWord<double> {
    typedef unsigned long long type;
    static __device__ __forceinline__ type of(double v) {
        const unsigned long long b = (unsigned long long)__double_as_longlong(v + 0.0);
        return (b >> 63) ? ~b : (b | 0x8000000000000000ull);
    }
};
template <>
struct OrderedWord<int32_t> {
    typedef unsigned int type;
    static __device__ __forceinline__ type of(int32_t v) { return (unsigned int)v ^ 0x80000000u; }
};

template <typename T>
__global__ __launch_bounds__(256) void row_words_kernel(const T* x, long total, int cols, int reverse, int largest, typename OrderedWord<T>::type* words) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const long row = i / cols;
    const int col = (int)(i - row * cols);
    const int src = reverse ? cols - 1 - col : col;
    const typename OrderedWord<T>::type w = OrderedWord<T>::of(x[row * cols + src]);
    words[i] = largest ? ~w : w;
}

// The first k positions of every sorted row, as column numbers of the input
__global__ __launch_bounds__(256) void leading_columns_kernel(const int32_t* pos, long total, int cols, int k, int reverse, int32_t* out) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const long row = i / k;
    const int col = pos[row * cols + (i - row * k)] - (int)(row * cols);
    out[i] = reverse ? cols - 1 - col : col;
}

// A few best entries of long rows: selection instead of a sort. One workgroup per row, read once, coalesced. Every wave
// keeps ONE list of its k best (value, column) pairs, lane i holding the i-th best, and the value of lane k - 1 as a
// wave-wide threshold: after the first few steps almost every element fails the threshold, which costs one comparison,
// and the rare one that passes is inserted by all lanes at once (each lane keeps its entry, takes its neighbour's or
// takes the newcomer). Wave 0 then inserts the other three lists into its own. `better` is the reference's comparator
// (dali/array/op/top_k.cpp:103-135): by value, then by column, ascending columns first unless ties_desc; it is a strict
// total order, so the result does not depend on the order in which elements arrive.
constexpr int kSelectMax = 64;

template <typename T>
struct Candidate {
    T value;
    int32_t column;  // -1: no candidate
};

template <typename T>
__device__ __forceinline__ bool better(const Candidate<T>& a, const Candidate<T>& b, bool largest, bool ties_desc) {
    if (a.column < 0) return false;
    if (b.column < 0) return true;
    if (a.value != b.value) return largest ? a.value > b.value : a.value < b.value;
    return ties_desc ? a.column > b.column : a.column < b.column;
}

// Entry of one lane, the same lane for the whole wave (a scalar read of the register, no trip through the LDS crossbar)
template <typename T>
__device__ __forceinline__ Candidate<T> from_lane(const Candidate<T>& c, int src_lane) {
    Candidate<T> r;
    if constexpr (sizeof(T) == 8) {
        union {
            T v;
            int w[2];
        } u;
        u.v = c.value;
        u.w[0] = __builtin_amdgcn_readlane(u.w[0], src_lane);
        u.w[1] = __builtin_amdgcn_readlane(u.w[1], src_lane);
        r.value = u.v;
    } else {
        union {
            T v;
            int w;
        } u;
        u.v = c.value;
        u.w = __builtin_amdgcn_readlane(u.w, src_lane);
        r.value = u.v;
    }
    r.column = __builtin_amdgcn_readlane(c.column, src_lane);
    return r;
}
// Entry of the lane below (lane 0 keeps its own)
template <typename T>
__device__ __forceinline__ Candidate<T> from_lane_below(const Candidate<T>& c) {
    Candidate<T> r;
    if constexpr (sizeof(T) == 8) {
        union {
            T v;
            int w[2];
        } u;
        u.v = c.value;
        u.w[0] = __shfl_up(u.w[0], 1, 64);
        u.w[1] = __shfl_up(u.w[1], 1, 64);
        r.value = u.v;
    } else {
        r.value = __shfl_up(c.value, 1, 64);
    }
    r.column = __shfl_up(c.column, 1, 64);
    return r;
}

// `cand` is the same in every lane. Lanes whose entry it beats move one place back; the first of them takes it.
template <typename T>
__device__ __forceinline__ void insert_candidate(Candidate<T>& mine, Candidate<T>& worst, const Candidate<T>& cand, int lane, int k, bool largest,
                                                 bool ties_desc) {
    const Candidate<T> prev = from_lane_below(mine);
    const bool beats_here = better(cand, mine, largest, ties_desc);
    const bool beats_prev = lane > 0 && better(cand, prev, largest, ties_desc);
    if (beats_prev)
        mine = prev;
    else if (beats_here)
        mine = cand;
    worst = from_lane(mine, k - 1);
}

template <typename T, bool largest, bool ties_desc>
__global__ __launch_bounds__(256) void select_rows_kernel(const T* x, int cols, int k, int32_t* out) {
    __shared__ Candidate<T> lists[4][64];
    const T* row = x + (size_t)blockIdx.x * cols;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    Candidate<T> mine, worst;
    mine.value = worst.value = (T)0;
    mine.column = worst.column = -1;
    constexpr int BATCH = sizeof(T) == 8 ? 8 : 16;  // loads in flight per lane: four waves per SIMD must cover the memory latency
    for (int base = wave * 64; base < cols; base += 256 * BATCH) {
        Candidate<T> cand[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
            const int c = base + u * 256 + lane;
            cand[u].column = c < cols ? c : -1;
            cand[u].value = c < cols ? row[c] : (T)0;
        }
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
            // the quick test is on the value alone (an equal value may still win on its column); the full comparison
            // is made once per passing element, below
            const bool passes = worst.column < 0 || (largest ? cand[u].value >= worst.value : cand[u].value <= worst.value);
            unsigned long long pending = __ballot(passes && cand[u].column >= 0);
            while (pending) {
                const int src = __ffsll((long long)pending) - 1;
                pending &= pending - 1;
                const Candidate<T> c = from_lane(cand[u], src);
                if (better(c, worst, largest, ties_desc)) insert_candidate(mine, worst, c, lane, k, largest, ties_desc);  // the threshold may have risen
            }
        }
    }
    if (lane >= k) mine.column = -1;
    lists[wave][lane] = mine;
    __syncthreads();
    if (wave != 0) return;
    for (int w = 1; w < 4; ++w)
        for (int i = 0; i < k; ++i) {
            const Candidate<T> c = lists[w][i];
            if (!better(c, worst, largest, ties_desc)) break;  // the lists are ordered: nothing behind it passes either
            insert_candidate(mine, worst, c, lane, k, largest, ties_desc);
        }
    if (lane < k) out[(size_t)blockIdx.x * k + lane] = mine.column;
}

// The same selection for 4-byte keys with a candidate packed into one 64-bit word: the value mapped to an unsigned
// integer of the same order (inverted when the smallest win) in the high half, the column in the low half (inverted when
// the lower column wins ties), 0 = no candidate. "Better" is then one unsigned 64-bit comparison, which is what the
// insertions, the bulk of the work for random rows, are made of.
template <typename T, bool largest, bool ties_desc>
__device__ __forceinline__ unsigned long long pack_candidate(T value, int column) {
    unsigned int u;
    if constexpr (sizeof(T) == 4 && !std::is_integral<T>::value) {
        const float canonical = value + 0.0f;  // -0.0 becomes +0.0
        u = __float_as_uint(canonical);
        u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
    } else {
        u = (unsigned int)value ^ 0x80000000u;
    }
    if (!largest) u = ~u;
    const unsigned int c = ties_desc ? (unsigned int)column + 1u : ~(unsigned int)column;  // never 0 together with u == 0
    return ((unsigned long long)u << 32) | c;
}
template <typename T, bool largest>
__device__ __forceinline__ T unpack_value(unsigned long long bits) {
    unsigned int u = (unsigned int)(bits >> 32);
    if (!largest) u = ~u;
    if constexpr (sizeof(T) == 4 && !std::is_integral<T>::value) {
        u = (u & 0x80000000u) ? (u & 0x7FFFFFFFu) : ~u;
        return __uint_as_float(u);
    } else {
        return (T)(u ^ 0x80000000u);
    }
}
template <bool ties_desc>
__device__ __forceinline__ int packed_column(unsigned long long bits) {
    return ties_desc ? (int)((unsigned int)bits - 1u) : (int)~(unsigned int)bits;
}
__device__ __forceinline__ unsigned long long packed_from_lane(unsigned long long v, int src_lane) {
    const unsigned int lo = (unsigned int)__builtin_amdgcn_readlane((int)(unsigned int)v, src_lane);
    const unsigned int hi = (unsigned int)__builtin_amdgcn_readlane((int)(unsigned int)(v >> 32), src_lane);
    return ((unsigned long long)hi << 32) | lo;
}
__device__ __forceinline__ void insert_packed(unsigned long long& mine, unsigned long long& worst, unsigned long long cand, int lane, int k) {
    const unsigned int lo = (unsigned int)__shfl_up((int)(unsigned int)mine, 1, 64);
    const unsigned int hi = (unsigned int)__shfl_up((int)(unsigned int)(mine >> 32), 1, 64);
    const unsigned long long prev = ((unsigned long long)hi << 32) | lo;
    if (lane > 0 && cand > prev)
        mine = prev;
    else if (cand > mine)
        mine = cand;
    worst = packed_from_lane(mine, k - 1);
}

// WAVES waves share a row: four when there are few rows (more loads in flight per row), one when there are thousands
// (a single list per row sees every element, so it takes a third of the insertions).
template <typename T, bool largest, bool ties_desc, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void select_rows_packed_kernel(const T* x, int cols, int k, int32_t* out) {
    static_assert(sizeof(T) == 4, "packed candidates hold 4-byte values");
    __shared__ unsigned long long lists[WAVES][64];
    const T* row = x + (size_t)blockIdx.x * cols;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    unsigned long long mine = 0, worst = 0;
    constexpr int BATCH = 16;  // loads in flight per lane
    for (int base = wave * 64; base < cols; base += 64 * WAVES * BATCH) {
        T value[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
            const int c = base + u * (64 * WAVES) + lane;
            value[u] = c < cols ? row[c] : (T)0;
        }
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
            // the streaming test is on the raw value against the threshold's value (an equal value may still win on its
            // column); a candidate is packed only once it passes
            const T threshold = unpack_value<T, largest>(worst);
            const bool passes = worst == 0ull || (largest ? value[u] >= threshold : value[u] <= threshold);
            unsigned long long pending = __ballot(passes && base + u * (64 * WAVES) + lane < cols);
            while (pending) {
                const int src = __ffsll((long long)pending) - 1;
                pending &= pending - 1;
                union {
                    T v;
                    int w;
                } raw;
                raw.v = value[u];
                raw.w = __builtin_amdgcn_readlane(raw.w, src);
                const unsigned long long cnd = pack_candidate<T, largest, ties_desc>(raw.v, base + u * (64 * WAVES) + src);
                if (cnd > worst) insert_packed(mine, worst, cnd, lane, k);  // the threshold may have risen
            }
        }
    }
    lists[wave][lane] = lane < k ? mine : 0ull;
    __syncthreads();
    if (wave != 0) return;
    for (int w = 1; w < WAVES; ++w)
        for (int i = 0; i < k; ++i) {
            const unsigned long long cnd = lists[w][i];
            if (!(cnd > worst)) break;  // the lists are ordered: nothing behind it passes either
            insert_packed(mine, worst, cnd, lane, k);
        }
    if (lane < k) out[(size_t)blockIdx.x * k + lane] = packed_column<ties_desc>(mine);
}

template <typename T, bool largest, bool ties_desc>
void launch_select_rows(const T* x, int rows, int cols, int k, int32_t* out, hipStream_t st) {
    if constexpr (sizeof(T) == 4) {
        if (rows >= 4096)
            hipLaunchKernelGGL((select_rows_packed_kernel<T, largest, ties_desc, 1>), dim3((unsigned)rows), dim3(64), 0, st, x, cols, k, out);
        else
            hipLaunchKernelGGL((select_rows_packed_kernel<T, largest, ties_desc, 4>), dim3((unsigned)rows), dim3(256), 0, st, x, cols, k, out);
    }
    else
        hipLaunchKernelGGL((select_rows_kernel<T, largest, ties_desc>), dim3((unsigned)rows), dim3(256), 0, st, x, cols, k, out);
}

template <typename T>
int topk_rows(const void* x, int rows, int cols, int k, bool largest, bool ties_by_descending_column, int32_t* out) {
    hipStream_t st = stream();
    static const int select_off = getenv("DALI_HIP_TOPK_SORT_ONLY") != nullptr;
    if (k <= kSelectMax && cols >= 1024 && !select_off) {
        if (largest && ties_by_descending_column)
            launch_select_rows<T, true, true>((const T*)x, rows, cols, k, out, st);
        else if (largest)
            launch_select_rows<T, true, false>((const T*)x, rows, cols, k, out, st);
        else if (ties_by_descending_column)
            launch_select_rows<T, false, true>((const T*)x, rows, cols, k, out, st);
        else
            launch_select_rows<T, false, false>((const T*)x, rows, cols, k, out, st);
        hipError_t le = hipGetLastError();
        if (le != hipSuccess) return fail("row selection launch failed: %s", hipGetErrorString(le));
        return DALI_HIP_OK;
    }
    // the whole matrix as one stable sort: by word, then by row
    typedef typename OrderedWord<T>::type W;
    const int total = rows * cols;  // (the caller has checked that it fits)
    const int rounds = radix_rounds(total), tiles = (total + 256 * rounds - 1) / (256 * rounds);
    int row_bits = 0;
    while (row_bits < 31 && (1 << row_bits) < rows) ++row_bits;
    const int key_passes = (int)sizeof(W), row_passes = (row_bits + 7) / 8;
    const size_t word_bytes = (size_t)total * sizeof(W), pos_bytes = (size_t)total * sizeof(int32_t), hist_bytes = ((size_t)256 * tiles + 256) * sizeof(unsigned int);
    void *words[2] = {nullptr, nullptr}, *pos[2] = {nullptr, nullptr}, *hist = nullptr;
    int status = DALI_HIP_OK;
    if (dali_hip_bank_allocate(&words[0], word_bytes) || dali_hip_bank_allocate(&words[1], word_bytes) || dali_hip_bank_allocate(&pos[0], pos_bytes) ||
        dali_hip_bank_allocate(&pos[1], pos_bytes) || dali_hip_bank_allocate(&hist, hist_bytes))
        status = DALI_HIP_ERROR;
    if (status == DALI_HIP_OK) {
        unsigned int* h = (unsigned int*)hist;
        unsigned int* totals = h + (size_t)256 * tiles;
        hipLaunchKernelGGL(row_words_kernel<T>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, (const T*)x, (long)total, cols,
                           ties_by_descending_column ? 1 : 0, largest ? 1 : 0, (W*)words[0]);
        int from = 0;
        const int32_t* src_pos = nullptr;  // first pass: a pair's position is its index
        for (int i = 0; i < key_passes; ++i) {
            radix_pass<W, WordDigits>(rounds, (const W*)words[from], src_pos, total, 8 * i, WordDigits(), h, totals, tiles, (W*)words[1 - from], (int32_t*)pos[1 - from], st);
            from = 1 - from;
            src_pos = (const int32_t*)pos[from];
        }
        for (int i = 0; i < row_passes; ++i) {
            radix_pass<W, RowDigits>(rounds, (const W*)nullptr, src_pos, total, 8 * i, RowDigits{cols}, h, totals, tiles, (W*)nullptr, (int32_t*)pos[1 - from], st);
            from = 1 - from;
            src_pos = (const int32_t*)pos[from];
        }
        const long kept = (long)rows * k;
        hipLaunchKernelGGL(leading_columns_kernel, dim3((unsigned)((kept + 255) / 256)), dim3(256), 0, st, src_pos, kept, cols, k, ties_by_descending_column ? 1 : 0, out);
        hipError_t le = hipGetLastError();
        if (le != hipSuccess) status = fail("row sort launch failed: %s", hipGetErrorString(le));
    }
    // back to the bank at once: their next user is ordered behind these launches on the stream
    if (hist) dali_hip_bank_deposit(hist, hist_bytes);
    if (pos[1]) dali_hip_bank_deposit(pos[1], pos_bytes);
    if (pos[0]) dali_hip_bank_deposit(pos[0], pos_bytes);
    if (words[1]) dali_hip_bank_deposit(words[1], word_bytes);
    if (words[0]) dali_hip_bank_deposit(words[0], word_bytes);
    return status;
}

// One launch of the rank sort: `tickets` holds one zeroed counter per block of 256 keys (each is set back to zero by the
// workgroup that consumes it), `partial` room for ceil(n / kRankSegment) * n counts.
static int launch_rank_sort(const int32_t* keys, int ni, int32_t key_limit, unsigned int* tickets, int32_t* partial, int32_t* sorted_keys,
                            int32_t* perm, hipStream_t st) {
    const int segments = (ni + kRankSegment - 1) / kRankSegment, blocks = (ni + 255) / 256;
    int shift = 0;
    while ((1 << shift) < ni) ++shift;
    // (one more key value than the valid ones: invalid keys get a word of their own, behind every valid key)
    const bool packed = key_limit > 0 && (((unsigned long long)key_limit + 1ull) << shift) <= (1ull << 32);
    if (packed)
        hipLaunchKernelGGL(rank_sort_kernel<unsigned int>, dim3(blocks, segments), dim3(256), 0, st, keys, ni, shift, (int)key_limit, segments, partial, tickets,
                           sorted_keys, perm);
    else
        hipLaunchKernelGGL(rank_sort_kernel<unsigned long long>, dim3(blocks, segments), dim3(256), 0, st, keys, ni, shift, (int)key_limit, segments, partial,
                           tickets, sorted_keys, perm);
    hipError_t le = hipGetLastError();
    if (le != hipSuccess) return fail("rank sort launch failed: %s", hipGetErrorString(le));
    return DALI_HIP_OK;
}

// ---------------------------------------------------------------- ordering without any allocation
// dali_hip_argsort_i32_noalloc keeps the tickets and counts of the rank sort in a device array that is part of this
// library's code object instead of the library workspace: callers that must not allocate (stream capture, serving
// loops) get the same kernel with memory that exists from the moment the code object is loaded. Each device holds
// its own copy of the array at its own address; the host-side name below is only a handle for hipGetSymbolAddress,
// the kernels receive the address that call returned for the current device.
constexpr int kNoAllocMaxKeys = kRankSegment * kRankMaxSegments;            // 16384 keys
constexpr size_t kScratchTicketBytes = 256;                                // one ticket per 256 keys: 64 counters
constexpr size_t kScratchPartialBytes = (size_t)kRankMaxSegments * kNoAllocMaxKeys * sizeof(int32_t);  // 2 MiB
static_assert((size_t)(kNoAllocMaxKeys / 256) * sizeof(unsigned int) <= kScratchTicketBytes, "tickets do not fit");
static __device__ __align__(256) unsigned char scratch[kScratchTicketBytes + kScratchPartialBytes];

constexpr int kMaxDevices = 64;
static unsigned char* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each device, 0 = not looked up

int sort_scratch_init(int device) {
    if (device < 0 || device >= kMaxDevices) return fail("sort_scratch_init: device %d out of range", device);
    if (g_scratch_ptr[device]) return DALI_HIP_OK;
    void* ptr = nullptr;
    hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) return fail("hipGetSymbolAddress(scratch) failed on device %d: %s", device, hipGetErrorString(e));
    g_scratch_ptr[device] = (unsigned char*)ptr;  // zero-initialised with the code object: the tickets start at zero
    return DALI_HIP_OK;
}

}  // namespace dali_hip

using namespace dali_hip;

extern "C" int dali_hip_topk_rows(const void* x, int dtype, int64_t rows, int32_t cols, int32_t k, int largest, int ties_by_descending_column,
                                  int32_t* out) {
    if (ensure_init()) return DALI_HIP_ERROR;
    if (rows < 0 || cols < 0) return fail("dali_hip_topk_rows: negative extent");
    if (k < 1 || k > cols) return fail("dali_hip_topk_rows: k = %d must lie in [1, %d]", k, cols);
    if (rows == 0) return DALI_HIP_OK;
    if (rows * (int64_t)cols > 2147483647LL) return fail("dali_hip_topk_rows: %lld keys exceed the int32 position range", (long long)(rows * cols));
    if (!x || !out) return fail("dali_hip_topk_rows: NULL argument");
    switch (dtype) {
        case 0: return topk_rows<float>(x, (int)rows, cols, k, largest != 0, ties_by_descending_column != 0, out);
        case 1: return topk_rows<double>(x, (int)rows, cols, k, largest != 0, ties_by_descending_column != 0, out);
        case 2: return topk_rows<int32_t>(x, (int)rows, cols, k, largest != 0, ties_by_descending_column != 0, out);
    }
    return fail("dali_hip_topk_rows: unknown dtype %d (0 = float, 1 = double, 2 = int32)", dtype);
}

// the outputs are written while other workgroups still read the keys: the three arrays must be distinct
static bool argsort_arrays_overlap(const int32_t* keys, int64_t n, const int32_t* sorted_keys, const int32_t* perm) {
    const size_t bytes = (size_t)n * sizeof(int32_t);
    auto meet = [&](const void* a, const void* b) { return (const char*)a < (const char*)b + bytes && (const char*)b < (const char*)a + bytes; };
    return meet(keys, sorted_keys) || meet(keys, perm) || meet(sorted_keys, perm);
}

extern "C" int dali_hip_argsort_i32(const int32_t* keys, int64_t n, int32_t key_limit, int32_t* sorted_keys, int32_t* perm) {
    if (ensure_init()) return DALI_HIP_ERROR;
    if (n < 0) return fail("dali_hip_argsort_i32: negative length %lld", (long long)n);
    if (n == 0) return DALI_HIP_OK;
    if (n > 2147483647LL) return fail("dali_hip_argsort_i32: %lld keys exceed the int32 position range", (long long)n);
    if (!keys || !sorted_keys || !perm) return fail("dali_hip_argsort_i32: NULL argument");
    if (argsort_arrays_overlap(keys, n, sorted_keys, perm)) return fail("dali_hip_argsort_i32: keys, sorted_keys and perm must not overlap");
    hipStream_t st = stream();
    // keys known to lie in [0, key_limit) need only their low bits sorted
    int end_bit = 32;
    if (key_limit > 0) {
        end_bit = 1;
        while (end_bit < 31 && ((int64_t)1 << end_bit) <= (int64_t)key_limit) ++end_bit;  // the digits of key_limit itself included
    }
    static const int rank_max = getenv("DALI_HIP_RANK_SORT_MAX") ? atoi(getenv("DALI_HIP_RANK_SORT_MAX")) : 16384;
    if (n <= rank_max && n <= (int64_t)kRankSegment * kRankMaxSegments &&
        (size_t)((n + kRankSegment - 1) / kRankSegment) * (size_t)n * sizeof(int32_t) <= kWorkspacePartialBytes &&
        (n + 255) / 256 <= kWorkspaceCounters)
        return launch_rank_sort(keys, (int)n, key_limit, (unsigned int*)workspace(), (int32_t*)(workspace() + kWorkspaceCounterBytes), sorted_keys,
                                perm, st);
    // radix passes over the bits that can differ; arbitrary keys are ordered as signed numbers (the sign bit is flipped in
    // the digit). The pairs bounce between the caller's arrays and one temporary block so that the last pass lands in the
    // caller's.
    const int rounds = radix_rounds(n);
    const int passes = (end_bit + 7) / 8, tiles = (int)((n + 256 * rounds - 1) / (256 * rounds));
    const unsigned int flip = key_limit > 0 ? 0u : 0x80000000u, limit = key_limit > 0 ? (unsigned int)key_limit : 0u;
    const size_t temp_bytes = ((size_t)2 * (size_t)n + (size_t)256 * (size_t)tiles + 256) * sizeof(int32_t);
    void* temp = nullptr;
    if (dali_hip_bank_allocate(&temp, temp_bytes)) return DALI_HIP_ERROR;
    int32_t* tkeys = (int32_t*)temp;
    int32_t* tpos = tkeys + n;
    unsigned int* hist = (unsigned int*)(tpos + n);
    unsigned int* totals = hist + (size_t)256 * (size_t)tiles;
    const int32_t* src_keys = keys;
    const int32_t* src_pos = nullptr;  // first pass: a pair's position is its index
    for (int i = 0; i < passes; ++i) {
        const bool to_caller = (passes - 1 - i) % 2 == 0;
        int32_t* dst_keys = to_caller ? sorted_keys : tkeys;
        int32_t* dst_pos = to_caller ? perm : tpos;
        radix_pass<int32_t, IndexDigits>(rounds, src_keys, src_pos, (int)n, 8 * i, IndexDigits{flip, limit}, hist, totals, tiles, dst_keys, dst_pos, st);
        src_keys = dst_keys;
        src_pos = dst_pos;
    }
    int status = DALI_HIP_OK;
    hipError_t le = hipGetLastError();
    if (le != hipSuccess) status = fail("radix sort launch failed: %s", hipGetErrorString(le));
    // the block goes back to the bank at once: the next user of it is ordered behind the sort on the stream
    dali_hip_bank_deposit(temp, temp_bytes);
    return status;
}

extern "C" int dali_hip_argsort_i32_noalloc(const int32_t* keys, int64_t n, int32_t key_limit, int32_t* sorted_keys, int32_t* perm) {
    const int device = bound_device();
    if (device < 0) return fail("dali_hip_argsort_i32_noalloc: call dali_hip_init first (initialisation allocates, this call must not)");
    if (n < 0) return fail("dali_hip_argsort_i32_noalloc: negative length %lld", (long long)n);
    if (n > kNoAllocMaxKeys)
        return fail("dali_hip_argsort_i32_noalloc: %lld keys exceed the limit of %d keys that the built-in scratch array serves", (long long)n,
                    kNoAllocMaxKeys);
    if (n == 0) return DALI_HIP_OK;
    if (!keys || !sorted_keys || !perm) return fail("dali_hip_argsort_i32_noalloc: NULL argument");
    if (argsort_arrays_overlap(keys, n, sorted_keys, perm)) return fail("dali_hip_argsort_i32_noalloc: keys, sorted_keys and perm must not overlap");
    unsigned char* base = device < kMaxDevices ? g_scratch_ptr[device] : nullptr;
    if (!base) return fail("dali_hip_argsort_i32_noalloc: no scratch address for device %d", device);
    return launch_rank_sort(keys, (int)n, key_limit, (unsigned int*)base, (int32_t*)(base + kScratchTicketBytes), sorted_keys, perm, stream());
}
