// Arithmetic of the LSTM gate epilogue shared by the fused-step kernels.
#ifndef DALI_HIP_GATE_MATH_H
#define DALI_HIP_GATE_MATH_H

#include <hip/hip_runtime.h>

namespace dali_hip {

// exp of the gate epilogue: the same sequence as the exp of the generated kernels (dali_expf in the device prelude of the
// front-end), so that the fused step and the two-launch form round every gate identically.
__device__ __forceinline__ float gate_expf(float x) {
    const float c = 0x1.715476p+0f, cc = 0x1.4ae0bep-26f;
    const float t = x * c;
    float r = __builtin_fmaf(x, c, -t);
    r = __builtin_fmaf(x, cc, r);
    const float e = __builtin_amdgcn_exp2f(t);
    const float fixed = __builtin_fmaf(e, r * 0x1.62e430p-1f, e);
    return __builtin_fabsf(t) < 128.0f ? fixed : e;
}

// the reference's sigmoid (dali/array/functor.h:157-162): 1 / (1 + exp(-x)) in double, rounded to float
__device__ __forceinline__ float gate_sigmoid(float x) { return (float)(1.0 / (1.0 + (double)gate_expf(-x))); }

// One (row, hidden unit) pair of an LSTM step from its four pre-activations (bias not yet added) and the previous cell
// value: gate = pre + bias, i / f / o = sigmoid in double, g = tanh, c' = f * c + i * g, h' = o * tanh(c'), each operation
// rounded on its own like the generated gate kernel (dali/layers/lstm.cpp:238-261).
__device__ __forceinline__ void lstm_gates(float pi, float pf, float po, float pg, const float (&bias)[4], float c_prev, float* c_out, float* h_out) {
#pragma clang fp contract(off)
    const float gi = pi + bias[0];
    const float gf = pf + bias[1];
    const float go = po + bias[2];
    const float gg = pg + bias[3];
    const float iv = (float)(1.0 / (1.0 + (double)gate_expf(-gi)));
    const float fv = (float)(1.0 / (1.0 + (double)gate_expf(-gf)));
    const float ov = (float)(1.0 / (1.0 + (double)gate_expf(-go)));
    const float gv = tanhf(gg);
    const float fc = fv * c_prev;
    const float ig = iv * gv;
    const float cn = fc + ig;
    *c_out = cn;
    *h_out = ov * tanhf(cn);
}

}  // namespace dali_hip

#endif
