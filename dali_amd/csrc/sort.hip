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

#include <hipcub/hipcub.hpp>

namespace dali_hip {

__global__ __launch_bounds__(256) void iota_kernel(int32_t* out, long n) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = (int32_t)i;
}

// A few thousand keys: counting ranks beats any multi-pass sort. The final position of key i is the number of
// (key, position) pairs that order before it. A workgroup counts, for 256 keys, the smaller pairs within one
// segment of the input (staged in LDS, read as wave-wide broadcasts) and publishes the counts; the workgroup that
// finishes last for those 256 keys (a ticket per key block) adds the segments' counts and places the keys.
// n * n comparisons, but spread over the whole chip, in one launch and without an allocation: the counts and the
// tickets live in the library workspace. When key_limit * 2^ceil(log2 n) fits 32 bits a pair is one 32-bit word
// (key in the high bits, position in the low ones), which halves the cost of a comparison.
template <typename W>
__device__ __forceinline__ W rank_pair(int32_t key, int pos, int shift);
template <>
__device__ __forceinline__ unsigned long long rank_pair<unsigned long long>(int32_t key, int pos, int) {
    return ((unsigned long long)((unsigned int)key ^ 0x80000000u) << 32) | (unsigned int)pos;  // signed key order
}
template <>
__device__ __forceinline__ unsigned int rank_pair<unsigned int>(int32_t key, int pos, int shift) {
    // a key outside [0, key_limit) (an invalid index) is ordered as the largest valid key: whatever the input, the
    // words stay distinct, so the positions computed from them are a permutation
    const unsigned int top = (0xFFFFFFFFu >> shift);
    const unsigned int k = (unsigned int)key < top ? (unsigned int)key : top;
    return (k << shift) | (unsigned int)pos;
}

constexpr int kRankSegment = 512;
constexpr int kRankMaxSegments = 32;  // 16384 keys

template <typename W>
__global__ __launch_bounds__(256) void rank_sort_kernel(const int32_t* keys, int n, int shift, int segments, int32_t* partial,
                                                         unsigned int* tickets, int32_t* sorted_keys, int32_t* perm) {
    __shared__ __attribute__((aligned(16))) W tile[kRankSegment];
    __shared__ int is_last;
    const int i = blockIdx.x * 256 + threadIdx.x;
    const int j0 = blockIdx.y * kRankSegment;
    for (int t = threadIdx.x; t < kRankSegment; t += 256) {
        const int j = j0 + t;
        tile[t] = j < n ? rank_pair<W>(keys[j], j, shift) : ~(W)0;  // padding orders after (or with) every real pair
    }
    __syncthreads();
    const int32_t my_key = i < n ? keys[i] : 0;
    const W mine = rank_pair<W>(my_key, i, shift);
    int count = 0;
#pragma unroll 16
    for (int t = 0; t < kRankSegment; ++t) count += tile[t] < mine ? 1 : 0;
    if (i < n) __hip_atomic_store(partial + (size_t)blockIdx.y * n + i, count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_s_waitcnt(0);
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


// ---------------------------------------------------------------- ordering along rows (top_k / bottom_k / argsort)
// Keys of one dense [rows, cols] matrix are copied into a sort buffer beside their column numbers. -0.0 becomes +0.0
// so that the two compare equal, as they do for the reference's comparators; with `reverse` a row is laid out back to
// front, so that the stable sort which follows leaves equal keys in descending column order.
template <typename T>
__global__ __launch_bounds__(256) void row_keys_kernel(const T* x, long total, int cols, int reverse, T* keys, int32_t* columns) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const long row = i / cols;
    const int col = (int)(i - row * cols);
    const int src = reverse ? cols - 1 - col : col;
    keys[i] = x[row * cols + src] + (T)0;
    columns[i] = src;
}

__global__ __launch_bounds__(256) void row_offsets_kernel(int32_t* offsets, int rows, int cols) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i <= rows) offsets[i] = i * cols;
}

__global__ __launch_bounds__(256) void leading_columns_kernel(const int32_t* in, long total, int cols, int k, int32_t* out) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const long row = i / k;
    out[i] = in[row * cols + (i - row * k)];
}

template <typename T>
int topk_rows(const void* x, int rows, int cols, int k, bool largest, bool ties_by_descending_column, int32_t* out) {
    hipStream_t st = stream();
    const long total = (long)rows * cols;
    const size_t key_bytes = (size_t)total * sizeof(T), col_bytes = (size_t)total * sizeof(int32_t), off_bytes = ((size_t)rows + 1) * sizeof(int32_t);
    void *keys = nullptr, *keys_sorted = nullptr, *columns = nullptr, *columns_sorted = nullptr, *offsets = nullptr, *temp = nullptr;
    size_t temp_bytes = 0;
    int status = DALI_HIP_OK;
    if (dali_hip_bank_allocate(&keys, key_bytes) || dali_hip_bank_allocate(&keys_sorted, key_bytes) || dali_hip_bank_allocate(&columns, col_bytes) ||
        dali_hip_bank_allocate(&offsets, off_bytes) || (k < cols && dali_hip_bank_allocate(&columns_sorted, col_bytes)))
        status = DALI_HIP_ERROR;
    int32_t* sorted_columns = k < cols ? (int32_t*)columns_sorted : out;
    if (status == DALI_HIP_OK) {
        hipLaunchKernelGGL(row_keys_kernel<T>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, (const T*)x, total, cols,
                           ties_by_descending_column ? 1 : 0, (T*)keys, (int32_t*)columns);
        hipLaunchKernelGGL(row_offsets_kernel, dim3((unsigned)(rows / 256 + 1)), dim3(256), 0, st, (int32_t*)offsets, rows, cols);
        auto sort = [&](void* t) {
            const int32_t* off = (const int32_t*)offsets;
            return largest ? hipcub::DeviceSegmentedRadixSort::SortPairsDescending(t, temp_bytes, (const T*)keys, (T*)keys_sorted, (const int32_t*)columns,
                                                                                    sorted_columns, (int)total, rows, off, off + 1, 0, (int)sizeof(T) * 8, st)
                           : hipcub::DeviceSegmentedRadixSort::SortPairs(t, temp_bytes, (const T*)keys, (T*)keys_sorted, (const int32_t*)columns,
                                                                          sorted_columns, (int)total, rows, off, off + 1, 0, (int)sizeof(T) * 8, st);
        };
        hipError_t e = sort(nullptr);
        if (e != hipSuccess) {
            status = fail("row sort sizing failed: %s", hipGetErrorString(e));
        } else if (dali_hip_bank_allocate(&temp, temp_bytes ? temp_bytes : 4)) {
            status = DALI_HIP_ERROR;
        } else if ((e = sort(temp)) != hipSuccess) {
            status = fail("row sort failed: %s", hipGetErrorString(e));
        } else if (k < cols) {
            const long kept = (long)rows * k;
            hipLaunchKernelGGL(leading_columns_kernel, dim3((unsigned)((kept + 255) / 256)), dim3(256), 0, st, (const int32_t*)columns_sorted, kept, cols, k, out);
        }
        if (status == DALI_HIP_OK) {
            hipError_t le = hipGetLastError();
            if (le != hipSuccess) status = fail("row sort launch failed: %s", hipGetErrorString(le));
        }
    }
    // back to the bank at once: their next user is ordered behind these launches on the stream
    if (temp) dali_hip_bank_deposit(temp, temp_bytes ? temp_bytes : 4);
    if (columns_sorted) dali_hip_bank_deposit(columns_sorted, col_bytes);
    if (offsets) dali_hip_bank_deposit(offsets, off_bytes);
    if (columns) dali_hip_bank_deposit(columns, col_bytes);
    if (keys_sorted) dali_hip_bank_deposit(keys_sorted, key_bytes);
    if (keys) dali_hip_bank_deposit(keys, key_bytes);
    return status;
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

extern "C" int dali_hip_argsort_i32(const int32_t* keys, int64_t n, int32_t key_limit, int32_t* sorted_keys, int32_t* perm) {
    if (ensure_init()) return DALI_HIP_ERROR;
    if (n < 0) return fail("dali_hip_argsort_i32: negative length %lld", (long long)n);
    if (n == 0) return DALI_HIP_OK;
    if (n > 2147483647LL) return fail("dali_hip_argsort_i32: %lld keys exceed the int32 position range", (long long)n);
    if (!keys || !sorted_keys || !perm) return fail("dali_hip_argsort_i32: NULL argument");
    hipStream_t st = stream();
    // keys known to lie in [0, key_limit) need only their low bits sorted
    int end_bit = 32;
    if (key_limit > 0) {
        end_bit = 1;
        while (end_bit < 31 && ((int64_t)1 << end_bit) < (int64_t)key_limit) ++end_bit;
    }
    static const int rank_max = getenv("DALI_HIP_RANK_SORT_MAX") ? atoi(getenv("DALI_HIP_RANK_SORT_MAX")) : 16384;
    if (n <= rank_max && n <= (int64_t)kRankSegment * kRankMaxSegments &&
        (size_t)((n + kRankSegment - 1) / kRankSegment) * (size_t)n * sizeof(int32_t) <= kWorkspacePartialBytes &&
        (n + 255) / 256 <= kWorkspaceCounters) {
        const int ni = (int)n, segments = (ni + kRankSegment - 1) / kRankSegment, blocks = (ni + 255) / 256;
        unsigned int* tickets = (unsigned int*)workspace();
        int32_t* partial = (int32_t*)(workspace() + kWorkspaceCounterBytes);
        int shift = 0;
        while ((1 << shift) < ni) ++shift;
        const bool packed = key_limit > 0 && ((unsigned long long)key_limit << shift) <= (1ull << 32);
        if (packed)
            hipLaunchKernelGGL(rank_sort_kernel<unsigned int>, dim3(blocks, segments), dim3(256), 0, st, keys, ni, shift, segments, partial, tickets,
                               sorted_keys, perm);
        else
            hipLaunchKernelGGL(rank_sort_kernel<unsigned long long>, dim3(blocks, segments), dim3(256), 0, st, keys, ni, shift, segments, partial,
                               tickets, sorted_keys, perm);
        hipError_t le = hipGetLastError();
        if (le != hipSuccess) return fail("rank sort launch failed: %s", hipGetErrorString(le));
        return DALI_HIP_OK;
    }
    void* positions = nullptr;
    if (dali_hip_bank_allocate(&positions, (size_t)n * sizeof(int32_t))) return DALI_HIP_ERROR;
    hipLaunchKernelGGL(iota_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, (int32_t*)positions, (long)n);
    size_t temp_bytes = 0;
    hipError_t e = hipcub::DeviceRadixSort::SortPairs(nullptr, temp_bytes, keys, sorted_keys, (const int32_t*)positions, perm, (int)n, 0, end_bit, st);
    void* temp = nullptr;
    int status = DALI_HIP_OK;
    if (e != hipSuccess) {
        status = fail("radix sort sizing failed: %s", hipGetErrorString(e));
    } else if (dali_hip_bank_allocate(&temp, temp_bytes ? temp_bytes : 4)) {
        status = DALI_HIP_ERROR;
    } else {
        e = hipcub::DeviceRadixSort::SortPairs(temp, temp_bytes, keys, sorted_keys, (const int32_t*)positions, perm, (int)n, 0, end_bit, st);
        if (e != hipSuccess) status = fail("radix sort failed: %s", hipGetErrorString(e));
    }
    // the blocks go back to the bank at once: the next user of them is ordered behind the sort on the stream
    if (temp) dali_hip_bank_deposit(temp, temp_bytes ? temp_bytes : 4);
    dali_hip_bank_deposit(positions, (size_t)n * sizeof(int32_t));
    return status;
}
