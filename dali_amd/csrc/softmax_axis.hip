// Softmax along an axis that is not the last one of a contiguous fp32 array, [outer, extent, inner] reduced over `extent`
// (the reference's op::softmax(logits, axis), dali/array/op/softmax.cpp:5-8: exp(x - max) / sum(exp(x - max)) along the axis),
// in one pass over memory: read once, written once.
//
// The generated kernels do this in three passes (maxima and sums of exponentials through the column kernel, then the quotient
// as a strided map: x is read twice). Here a workgroup of 1024 threads owns a strip of W consecutive inner positions of one outer
// index, W * extent values, and holds it in registers, up to 32 values per thread: W = 64 for extents up to 512, 32 up to
// 1024, 16 up to 2048. A row of the strip is W / 4 lanes wide, each with one 16-byte piece, so a wave covers 256 / W rows per
// load and the sixteen waves 4096 / W; a thread keeps every (4096 / W)-th row. Maxima and sums are folded over a thread's
// rows, over the lanes of a wave that share a column (lane bits above the row's width) and over the waves through LDS.
// Neighbouring workgroups take neighbouring strips of the same outer index, so the device as a whole reads whole rows.
#include <hip/hip_runtime.h>

#include "gate_math.h"
#include "runtime.h"

namespace dali_hip {
namespace {

typedef float f4 __attribute__((ext_vector_type(4)));

struct AxisArgs {
    const float* x;
    float* out;
    int extent;       // X
    long inner;       // K (a multiple of 4)
    int strips;       // ceil(K / W)
    int nontemporal;  // loads bypass cache allocation (operands too large to be found in a cache again)
};

// LPR: lanes per row of the strip (W = 4 * LPR)
template <int LPR>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(8, 8))) void softmax_axis_kernel(AxisArgs a) {
    constexpr int RPW = 64 / LPR;     // rows per wave and load
    constexpr int RPS = 16 * RPW;     // rows per workgroup and load
    constexpr int W = 4 * LPR;
    constexpr int EPT = 8;            // loads per thread at most
    __shared__ float red[16][W];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cv = lane % LPR, rw = lane / LPR;
    const long b = blockIdx.x / (unsigned)a.strips;
    const int strip = (int)(blockIdx.x - (unsigned)b * (unsigned)a.strips);
    const long k = (long)strip * W + 4 * cv;
    const bool col_ok = k < a.inner;
    const int X = a.extent;
    const float* src = a.x + (b * X) * a.inner + k;
    float* dst = a.out + (b * X) * a.inner + k;
    const int r0 = wave * RPW + rw;
    f4 v[EPT];
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
        const int r = r0 + e * RPS;
        // (rows past the extent hold the identity of the maximum; their exponentials are never added or stored)
        v[e] = (f4){-INFINITY, -INFINITY, -INFINITY, -INFINITY};
        if (r < X && col_ok) {
            const f4* p = reinterpret_cast<const f4*>(src + (long)r * a.inner);
            v[e] = a.nontemporal ? __builtin_nontemporal_load(p) : *p;
        }
    }
    // one value per column of the strip from one value per thread: lanes that share a column, then the waves
    auto fold = [&](f4 t, auto op) -> f4 {
#pragma unroll
        for (int d = LPR; d < 64; d *= 2) {
            f4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = __shfl_xor(t[j], d, 64);
            t = op(t, o);
        }
        __syncthreads();  // the previous fold's values have been read
        if (rw == 0) {
#pragma unroll
            for (int j = 0; j < 4; ++j) red[wave][4 * cv + j] = t[j];
        }
        __syncthreads();
        f4 r;
#pragma unroll
        for (int j = 0; j < 4; ++j) r[j] = red[0][4 * cv + j];
#pragma unroll
        for (int w = 1; w < 16; ++w) {
            f4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = red[w][4 * cv + j];
            r = op(r, o);
        }
        return r;
    };
    f4 m = v[0];
#pragma unroll
    for (int e = 1; e < EPT; ++e)
#pragma unroll
        for (int j = 0; j < 4; ++j) m[j] = fmaxf(m[j], v[e][j]);
    m = fold(m, [](f4 p, f4 q) {
        f4 r;
#pragma unroll
        for (int j = 0; j < 4; ++j) r[j] = fmaxf(p[j], q[j]);
        return r;
    });
    f4 s = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
        const int r = r0 + e * RPS;
        if (r < X) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v[e][j] = gate_expf(v[e][j] - m[j]);
                s[j] += v[e][j];
            }
        }
    }
    s = fold(s, [](f4 p, f4 q) { return p + q; });
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
        const int r = r0 + e * RPS;
        if (r < X && col_ok) {
            f4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = v[e][j] / s[j];
            __builtin_nontemporal_store(o, reinterpret_cast<f4*>(dst + (long)r * a.inner));
        }
    }
}

// lanes per row for an extent, 0 when the strip would not fit the registers
int lanes_per_row(int extent, long inner) {
    if (extent <= 512 && inner >= 64) return 16;
    if (extent <= 1024 && inner >= 32) return 8;
    if (extent <= 2048) return 4;
    return 0;
}

}  // namespace
}  // namespace dali_hip

using namespace dali_hip;

extern "C" int dali_hip_softmax_axis_supported(long long outer, int extent, long long inner) {
    if (outer < 1 || extent < 2 || inner < 16 || inner % 4 != 0) return 0;
    const int lpr = lanes_per_row(extent, inner);
    if (lpr == 0) return 0;
    const long strips = (inner + 4 * lpr - 1) / (4 * lpr);
    return outer * strips <= 2147483647L ? 1 : 0;
}

extern "C" int dali_hip_softmax_axis(const float* x, float* out, long long outer, int extent, long long inner) {
    if (ensure_init()) return DALI_HIP_ERROR;
    if (!x || !out) return fail("dali_hip_softmax_axis: NULL argument");
    if (!dali_hip_softmax_axis_supported(outer, extent, inner))
        return fail("dali_hip_softmax_axis: [%lld, %d, %lld] is outside what the kernel holds in registers (inner a multiple of 4 and at least 16, extent up to 2048)", outer,
                    extent, inner);
    if ((((uintptr_t)x | (uintptr_t)out) & 15) != 0) return fail("dali_hip_softmax_axis: the arrays must be 16-byte aligned");
    const int lpr = lanes_per_row(extent, inner);
    AxisArgs a;
    a.x = x;
    a.out = out;
    a.extent = extent;
    a.inner = inner;
    a.strips = (int)((inner + 4 * lpr - 1) / (4 * lpr));
    a.nontemporal = (double)outer * extent * (double)inner * 4.0 >= (double)((size_t)64 << 20);
    const dim3 grid((unsigned)(outer * a.strips));
    switch (lpr) {
        case 16: hipLaunchKernelGGL(softmax_axis_kernel<16>, grid, dim3(1024), 0, stream(), a); break;
        case 8: hipLaunchKernelGGL(softmax_axis_kernel<8>, grid, dim3(1024), 0, stream(), a); break;
        default: hipLaunchKernelGGL(softmax_axis_kernel<4>, grid, dim3(1024), 0, stream(), a); break;
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("dali_hip_softmax_axis launch failed: %s", hipGetErrorString(e));
    return DALI_HIP_OK;
}
