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
// (key, position) pairs that order before it; every workgroup counts, for 256 keys, the smaller pairs within one
// segment of the input (staged in LDS, read as wave-wide broadcasts), and a second kernel adds the per-segment
// counts and places the key. n * n comparisons, but spread over the whole chip and two launches in all.
__device__ __forceinline__ unsigned long long rank_pair(int32_t key, int pos) {
    return ((unsigned long long)((unsigned int)key ^ 0x80000000u) << 32) | (unsigned int)pos;  // signed key order
}

constexpr int kRankSegment = 512;

__global__ __launch_bounds__(256) void rank_count_kernel(const int32_t* keys, int n, int32_t* partial) {
    __shared__ unsigned long long tile[kRankSegment];
    const int i = blockIdx.x * 256 + threadIdx.x;
    const int j0 = blockIdx.y * kRankSegment;
    for (int t = threadIdx.x; t < kRankSegment; t += 256) {
        const int j = j0 + t;
        tile[t] = j < n ? rank_pair(keys[j], j) : ~0ull;  // padding orders after every real pair
    }
    __syncthreads();
    const unsigned long long mine = rank_pair(i < n ? keys[i] : 0, i);
    int count = 0;
#pragma unroll 16
    for (int t = 0; t < kRankSegment; ++t) count += tile[t] < mine ? 1 : 0;
    if (i < n) partial[(size_t)blockIdx.y * n + i] = count;
}

__global__ __launch_bounds__(256) void rank_place_kernel(const int32_t* keys, int n, int segments, const int32_t* partial,
                                                          int32_t* sorted_keys, int32_t* perm) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    int pos = 0;
    for (int s = 0; s < segments; ++s) pos += partial[(size_t)s * n + i];
    sorted_keys[pos] = keys[i];
    perm[pos] = i;
}

}  // namespace dali_hip

using namespace dali_hip;

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
    if (n <= rank_max) {
        const int ni = (int)n, segments = (ni + kRankSegment - 1) / kRankSegment, blocks = (ni + 255) / 256;
        void* partial = nullptr;
        if (dali_hip_bank_allocate(&partial, (size_t)segments * ni * sizeof(int32_t))) return DALI_HIP_ERROR;
        hipLaunchKernelGGL(rank_count_kernel, dim3(blocks, segments), dim3(256), 0, st, keys, ni, (int32_t*)partial);
        hipLaunchKernelGGL(rank_place_kernel, dim3(blocks), dim3(256), 0, st, keys, ni, segments, (const int32_t*)partial, sorted_keys, perm);
        hipError_t le = hipGetLastError();
        dali_hip_bank_deposit(partial, (size_t)segments * ni * sizeof(int32_t));
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
