/*
 * dali_oracle.c — CPU restatement of the arithmetic of Dali's JIT-fused array
 * expressions. TEST INFRASTRUCTURE ONLY: it is the checker for the HIP path
 * (tests, smoke check, the cpu_baseline leg of the benchmark). Nothing in the
 * product links, imports or calls it.
 *
 * Every function follows the loop structure and rounding points of the
 * reference's generated CPU code (paths relative to the reference repository):
 * single-threaded, fp32 accumulators updated strictly left to right, libm
 * expf/tanhf/logf, sigmoid evaluated in double, no fast-math and no FMA
 * contraction (dali/utils/compiler.cpp:137-145 builds with -O3 -msse2 only).
 * Build with: gcc -O3 -ffp-contract=off (see oracle/Makefile).
 *
 * Pinning status (checked by tests/test_oracle.py):
 *   - functors: closed forms of dali/array/functor.h against libm in fp64 and the
 *     reference's own expectations (dali/array/tests/tests.cpp:1015-1117);
 *   - reducers / axis reduce / all reduce / argmax: closed forms of
 *     dali/array/tests/tests.cpp:1120-1239, brute force with planted ties, and the
 *     reference's reducers compiled from its own header (oracle/_ref);
 *   - gather_from_rows / one_hot: expected tables of dali/array/tests/tests.cpp:1303-1309
 *     and :984-997;
 *   - softmax / cross-entropy: row sums, shift invariance, textbook identities in fp64;
 *   - gemm: known answers of dali/array/tests/dot_tests.cpp:9-118 and an fp64 triple
 *     loop. The reference's fp32 GEMM is an un-vendored BLAS (cblas_sgemm), so its
 *     rounding on random fp32 inputs is PARITY UNPINNED; the fp64-accumulated product
 *     is used as truth with rel 1e-4.
 *   - im2col / col2im / pool2d / conv2d: the slice-and-ravel definition of
 *     dali/array/op/im2col_tests.cpp:7-39 on NHWC, NCHW and WNCH images, the TensorFlow
 *     tables of dali/array/tests/conv_tests.cpp:132-216 (VALID and SAME), a direct
 *     convolution loop, <im2col(x), y> == <x, col2im(y)> on integers, the patch-count
 *     identity col2im(im2col(x)) == x * count, and the window loops of
 *     dali/array/tests/conv_tests.cpp:422-640 for the pooling pair;
 *   - lstm step: composition of the above per dali/layers/lstm.cpp:226-261
 *     (no test in the reference pins LSTM values: PARITY UNPINNED beyond the
 *     composition of pinned parts).
 */
#include <float.h>
#include <limits.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_EPS 1e-6

/* ------------------------------------------------------------------ functors
 * dali/array/functor.h:27-495, non-CUDA branch: EXP_F = std::exp etc., which for
 * a float argument are the float overloads (expf, logf, tanhf, powf). */

static float f_sigmoid(float a) { return (float)(1.0 / (1.0 + (double)expf(-a))); } /* functor.h:157-162 */
static float f_tanh(float a) { return tanhf(a); }                                   /* functor.h:255-264 */
static float f_exp(float a) { return expf(a); }                                     /* functor.h:201-206 */
static float f_log(float a) { return logf(a); }                                     /* functor.h:171-176 */
static float f_negative_log(float a) { return -logf(a); }                           /* functor.h:178-183 */
static float f_square(float a) { return a * a; }                                    /* functor.h:38-43 */
static float f_cube(float a) { return a * a * a; }                                  /* functor.h:45-50 */
static float f_sqrt(float a) { return sqrtf(a); }                                   /* functor.h:101-106 */
static float f_rsqrt(float a) { return (float)(1.0 / sqrt((double)a)); }            /* functor.h:114-119, ::sqrt(double) */
static float f_inv(float a) { return 1.0f / a; }                                    /* functor.h:128-133 */
static float f_identity(float a) { return a; }                                      /* functor.h:164-169 */
static float f_abs(float a) { return fabsf(a); }                                    /* functor.h:330-335 */
static float f_sign(float a) { return (double)a > 0.0 ? 1.0f : -1.0f; }             /* functor.h:348-353 */
static float f_relu(float a) { return (double)a > 0.0 ? a : 0.0f; }                 /* functor.h:390-395 */
static float f_relu_backward(float a) { return (double)a > 0.0 ? 1.0f : 0.0f; }     /* functor.h:404-409 */
static float f_dsigmoid(float a) { return a * (1.0f - a); }                         /* functor.h:248-253 */
static float f_dtanh(float a) { return (float)(1.0 - (double)(a * a)); }            /* functor.h:290-295 */
static float f_round(float a) { return (float)floor((double)a + 0.5); }             /* functor.h:141-147 */
static float f_isnan(float a) { return isnan(a) ? 1.0f : 0.0f; }                    /* functor.h:208-213 */
static float f_isinf(float a) { return isinf(a) ? 1.0f : 0.0f; }                    /* functor.h:227-232 */
static float f_log_or_zero(float a) { return a > 0 ? logf(a) : 0.0f; }              /* functor.h:337-346 */
static float f_inverse_tanh(float a) {                                              /* functor.h:283-288 */
    return (float)((double)(logf(1 + a) - logf(1 - a)) * 0.5);
}
static float f_safe_entropy_log(float a) { /* functor.h:185-199 */
    float s = a;
    const float lo = (float)ORC_EPS, hi = (float)(1.0 - ORC_EPS);
    if (s > hi) s = hi;
    if (s < lo) s = lo;
    return logf(s);
}
static float f_softplus(float x) { /* functor.h:455-464 */
    if ((double)x > 20.0) return x;
    return logf(1.0f + expf(x));
}
static float f_softplus_backward(float x) { /* functor.h:466-475 */
    if ((double)x > 20.0) return 1.0f;
    return expf(x) / (1.0f + expf(x));
}

static float f_add(float a, float b) { return a + b; }                    /* functor.h:59-64 */
static float f_subtract(float a, float b) { return a - b; }               /* functor.h:73-78 */
static float f_eltmul(float a, float b) { return a * b; }                 /* functor.h:80-85 */
static float f_eltdiv(float a, float b) { return a / b; }                 /* functor.h:87-92 */
static float f_equals(float a, float b) { return a == b ? 1.0f : 0.0f; }  /* functor.h:66-71 */
static float f_power(float a, float b) { return powf(a, b); }             /* functor.h:304-308 */
static float f_fill(float a, float b) { (void)a; return b; }              /* functor.h:52-57 */
static float f_div_grad(float a, float b) { return a / (b * b); }         /* functor.h:241-246 */
static float f_threshold(float a, float b) { return a < b ? 1.0f : 0.0f; }  /* functor.h:355-360 */
static float f_max_scalar(float a, float b) { return a > b ? a : b; }       /* functor.h:362-367 */
static float f_min_scalar(float a, float b) { return a < b ? a : b; }       /* functor.h:369-374 */
static float f_lessthanequal(float a, float b) { return a <= b ? 1.0f : 0.0f; }    /* functor.h:425-430 */
static float f_greaterthanequal(float a, float b) { return a >= b ? 1.0f : 0.0f; } /* functor.h:432-437 */
static float f_prelu(float x, float w) { return x > 0 ? x : w * x; }               /* functor.h:477-482 */
static float f_prelu_backward_weights(float x, float g) { return x > 0 ? 0.0f : x * g; } /* functor.h:484-489 */
static float f_prelu_backward_inputs(float x, float w) { return x > 0 ? 1.0f : w; }      /* functor.h:491-496 */
static float f_steep_sigmoid(float x, float agg) {                                      /* functor.h:376-381 */
    return (float)(1.0 / (1.0 + (double)expf(-agg * x)));
}
static float f_steep_sigmoid_backward(float x, float agg) { return agg * (x - x * x); } /* functor.h:383-388 */
static float f_clipped_relu(float x, float c) {                                         /* functor.h:397-402 */
    return (double)x > 0.0 ? (x > c ? c : x) : 0.0f;
}
static float f_clipped_relu_backward(float x, float c) { /* functor.h:411-416 */
    return (double)x > 0.0 ? (x > c ? 0.0f : 1.0f) : 0.0f;
}
static float f_clip(float x, float c) { /* functor.h:418-429 */
    if (x > c) return c;
    if (x < -c) return -c;
    return x;
}
static float f_binary_cross_entropy(float x, float t) { /* functor.h:439-446 */
    float d1 = t * logf(x);
    float d0 = (float)((1.0 - (double)t) * log(1. - (double)x)); /* LOG_F(double) is the double log */
    return -(d1 + d0);
}
static float f_binary_cross_entropy_grad(float x, float t) { /* functor.h:448-455 */
    float num = t - x;
    float den = (float)((double)x * ((double)x - 1.0));
    return num / den;
}

typedef float (*unary_fn)(float);
typedef float (*binary_fn)(float, float);

static const struct { const char* name; unary_fn fn; } UNARY[] = {
    {"sigmoid", f_sigmoid}, {"tanh", f_tanh}, {"exp", f_exp}, {"log", f_log},
    {"negative_log", f_negative_log}, {"square", f_square}, {"cube", f_cube},
    {"sqrt_f", f_sqrt}, {"rsqrt", f_rsqrt}, {"inv", f_inv}, {"identity", f_identity},
    {"abs", f_abs}, {"sign", f_sign}, {"relu", f_relu}, {"relu_backward", f_relu_backward},
    {"dsigmoid", f_dsigmoid}, {"dtanh", f_dtanh}, {"round", f_round},
    {"isnotanumber", f_isnan}, {"isinfinity", f_isinf}, {"log_or_zero", f_log_or_zero},
    {"inverse_tanh", f_inverse_tanh}, {"safe_entropy_log", f_safe_entropy_log},
    {"softplus", f_softplus}, {"softplus_backward", f_softplus_backward}, {0, 0}};

static const struct { const char* name; binary_fn fn; } BINARY[] = {
    {"add", f_add}, {"subtract", f_subtract}, {"eltmul", f_eltmul}, {"eltdiv", f_eltdiv},
    {"equals", f_equals}, {"power", f_power}, {"fill", f_fill}, {"div_grad", f_div_grad},
    {"threshold", f_threshold}, {"max_scalar", f_max_scalar}, {"min_scalar", f_min_scalar},
    {"lessthanequal", f_lessthanequal}, {"greaterthanequal", f_greaterthanequal},
    {"prelu", f_prelu}, {"prelu_backward_weights", f_prelu_backward_weights},
    {"prelu_backward_inputs", f_prelu_backward_inputs}, {"steep_sigmoid", f_steep_sigmoid},
    {"steep_sigmoid_backward", f_steep_sigmoid_backward}, {"clipped_relu", f_clipped_relu},
    {"clipped_relu_backward", f_clipped_relu_backward}, {"clip", f_clip},
    {"binary_cross_entropy", f_binary_cross_entropy},
    {"binary_cross_entropy_grad", f_binary_cross_entropy_grad}, {0, 0}};

/* y[i] = functor::<name><float>::Map(x[i]); returns -1 for an unknown functor.
 * Loop shape: dali/array/jit/jit.cpp:687-715 (one rank-1 loop after collapse). */
int orc_unary(const char* name, const float* x, float* y, int64_t n) {
    for (int k = 0; UNARY[k].name; ++k)
        if (!strcmp(UNARY[k].name, name)) {
            unary_fn f = UNARY[k].fn;
            for (int64_t i = 0; i < n; ++i) y[i] = f(x[i]);
            return 0;
        }
    return -1;
}

/* y[i] = functor::<name><float>::Map(a[i*sa], b[i*sb]); sa/sb = 0 broadcasts a scalar
 * (dali/array/jit/scalar_view.cpp:39-66 passes scalars by pointer). */
int orc_binary(const char* name, const float* a, int64_t sa, const float* b, int64_t sb, float* y, int64_t n) {
    for (int k = 0; BINARY[k].name; ++k)
        if (!strcmp(BINARY[k].name, name)) {
            binary_fn f = BINARY[k].fn;
            for (int64_t i = 0; i < n; ++i) y[i] = f(a[i * sa], b[i * sb]);
            return 0;
        }
    return -1;
}

/* astype float -> int32: round = floor(a + 0.5) then the store converts to int
 * (dali/array/op/elementwise_operation.cpp:137-160, functor.h:141-147). */
void orc_round_to_int(const float* x, int32_t* y, int64_t n) {
    for (int64_t i = 0; i < n; ++i) y[i] = (int32_t)floor((double)x[i] + 0.5);
}

/* Fused elementwise chain y = sigmoid(a)*tanh(b) + c*d - 0.5*a^2, every node
 * rounded to fp32 as ElementWiseKernel nodes of dtype float do
 * (dali/array/jit/elementwise_kernel_utils.cpp:108-119); the double scalar 0.5 is
 * cast to float first (dali/array/op/elementwise_operation.cpp:174-179). */
void orc_chain(const float* a, const float* b, const float* c, const float* d, float* y, int64_t n) {
    const float half = (float)0.5;
    for (int64_t i = 0; i < n; ++i) {
        float t1 = f_eltmul(f_sigmoid(a[i]), f_tanh(b[i]));
        float t2 = f_eltmul(c[i], d[i]);
        float t3 = f_eltmul(half, f_square(a[i]));
        y[i] = f_subtract(f_add(t1, t2), t3);
    }
}

/* ------------------------------------------------------------------ reducers
 * dali/array/jit/reducer_kernels.h:57-169. 0 sum, 1 maximum, 2 minimum, 3 product. */
enum { ORC_SUM = 0, ORC_MAX = 1, ORC_MIN = 2, ORC_PROD = 3 };

static float red_init(int r) {
    switch (r) {
        case ORC_SUM: return 0.0f;       /* reducer_kernels.h:79-82 */
        case ORC_MAX: return -FLT_MAX;   /* reducer_kernels.h:113-116, :19-21 */
        case ORC_MIN: return FLT_MAX;    /* reducer_kernels.h:141-144, :41-43 */
        default: return 1.0f;            /* reducer_kernels.h:165-168 */
    }
}

static inline float red_step(int r, float dst, float src) {
    switch (r) {
        case ORC_SUM: return dst + src;              /* reducer_kernels.h:62-65 */
        case ORC_MAX: return dst > src ? dst : src;  /* reducer_kernels.h:97-103 */
        case ORC_MIN: return dst < src ? dst : src;  /* reducer_kernels.h:122-128 */
        default: return dst * src;                   /* reducer_kernels.h:150-153 */
    }
}

/* AxisReduceKernel: out[i] = reduce over j of x[i*row_stride + j*col_stride],
 * sequential in j (dali/array/jit/all_reduce_kernel_utils.cpp:142-154). A leading
 * axis is reduced by passing the transposed strides (row_stride 1, col_stride =
 * row length), which is the strided view op::axis_reduce builds
 * (dali/array/op/reducer_operation.cpp:642-655). */
void orc_axis_reduce(int reducer, const float* x, int64_t rows, int64_t cols, int64_t row_stride,
                     int64_t col_stride, float* out) {
    for (int64_t i = 0; i < rows; ++i) {
        float res = red_init(reducer);
        const float* p = x + i * row_stride;
        for (int64_t j = 0; j < cols; ++j) res = red_step(reducer, res, p[j * col_stride]);
        out[i] = res;
    }
}

/* AllReduceKernel: nested loops over all dims = one sequential pass for a
 * contiguous array (dali/array/jit/all_reduce_kernel_utils.cpp:105-121). */
float orc_all_reduce(int reducer, const float* x, int64_t n) {
    float res = red_init(reducer);
    for (int64_t i = 0; i < n; ++i) res = red_step(reducer, res, x[i]);
    return res;
}

/* ArgumentAxisReduceKernel: idx = 0; res = init; for j: tmp = res; Reduce(res, x);
 * if (tmp != res) idx = j  -> first index on ties
 * (dali/array/jit/all_reduce_kernel_utils.cpp:210-223); output dtype int32
 * (dali/array/op/reducer_operation.cpp:686-710). */
void orc_arg_axis_reduce(int reducer, const float* x, int64_t rows, int64_t cols, int64_t row_stride,
                         int64_t col_stride, int32_t* out) {
    for (int64_t i = 0; i < rows; ++i) {
        int32_t idx = 0;
        float res = red_init(reducer);
        const float* p = x + i * row_stride;
        for (int64_t j = 0; j < cols; ++j) {
            float tmp = res;
            res = red_step(reducer, res, p[j * col_stride]);
            if (tmp != res) idx = (int32_t)j;
        }
        out[i] = idx;
    }
}

/* ArgumentAllReduceKernel over a contiguous array: flat offset of the extremum
 * (dali/array/jit/all_reduce_kernel_utils.cpp:123-140). The reference stores the
 * index in the INPUT dtype (dali/array/op/reducer_operation.cpp:681-684). */
int64_t orc_arg_all_reduce(int reducer, const float* x, int64_t n) {
    int64_t idx = 0;
    float res = red_init(reducer);
    for (int64_t i = 0; i < n; ++i) {
        float tmp = res;
        res = red_step(reducer, res, x[i]);
        if (tmp != res) idx = i;
    }
    return idx;
}

/* op::mean = sum / identity(count), the int count cast to float
 * (dali/array/op/reducers.cpp:32-41). */
float orc_mean_all(const float* x, int64_t n) { return orc_all_reduce(ORC_SUM, x, n) / (float)(int)n; }

/* ------------------------------------------------------------------- softmax
 * op::softmax(logits, -1) = exped / sum(exped), exped = exp(logits - max(logits))
 * (dali/array/op/softmax.cpp:5-8). The generated CPU code runs four loop nests
 * with three temporaries: temp_0 = max, temp_1 = sum(exp(a - temp_0)),
 * temp_2 = exp(a - temp_0), dst = temp_2 / temp_1 (temporaries per
 * dali/array/jit/jit.cpp:631-652,839-860 and dali/array/jit/reshape.cpp:100-102). */
void orc_softmax(const float* a, float* out, int64_t rows, int64_t cols) {
    float* t0 = (float*)malloc(sizeof(float) * (size_t)rows);
    float* t1 = (float*)malloc(sizeof(float) * (size_t)rows);
    for (int64_t i = 0; i < rows; ++i) {
        float res = -FLT_MAX;
        for (int64_t j = 0; j < cols; ++j) {
            float v = a[i * cols + j];
            res = res > v ? res : v;
        }
        t0[i] = res;
    }
    for (int64_t i = 0; i < rows; ++i) {
        float res = 0.0f;
        for (int64_t j = 0; j < cols; ++j) res += expf(a[i * cols + j] - t0[i]);
        t1[i] = res;
    }
    /* temp_2 is written to `out`, then divided in place: same values as a separate buffer */
    for (int64_t i = 0; i < rows; ++i)
        for (int64_t j = 0; j < cols; ++j) out[i * cols + j] = expf(a[i * cols + j] - t0[i]);
    for (int64_t i = 0; i < rows; ++i)
        for (int64_t j = 0; j < cols; ++j) out[i * cols + j] = out[i * cols + j] / t1[i];
    free(t0);
    free(t1);
}

/* ------------------------------------------------------------- index kernels */

/* out[i] = source[i, indices[i]] (dali/array/op/gather_from_rows.cpp:53-78). */
void orc_gather_from_rows(const float* source, int64_t cols, const int32_t* indices, int64_t n, float* out) {
    for (int64_t i = 0; i < n; ++i) out[i] = source[i * cols + indices[i]];
}

/* out[i, :] = source[indices[i], :] (dali/array/op/gather.cpp:49-52, 2-D form). */
void orc_gather_rows(const float* source, int64_t cols, const int32_t* indices, int64_t n, float* out) {
    for (int64_t i = 0; i < n; ++i)
        for (int64_t j = 0; j < cols; ++j) out[i * cols + j] = source[(int64_t)indices[i] * cols + j];
}

/* Assignment through a gather on the CPU: the generated loop nest walks the destination view in index order
 * and applies `dst (op)= src` element by element (dali/array/op/gather.cpp:89-97 with the non-atomic branch),
 * so duplicates of an index are combined in input order. op: 0 =, 1 +=, 2 -=, 3 *=, 4 /=. values holds n*cols
 * floats, or a single float when value_is_scalar. */
void orc_scatter_rows(float* dest, int64_t cols, const int32_t* indices, int64_t n, const float* values, int value_is_scalar, int op) {
    for (int64_t i = 0; i < n; ++i)
        for (int64_t j = 0; j < cols; ++j) {
            float* d = dest + (int64_t)indices[i] * cols + j;
            const float v = value_is_scalar ? values[0] : values[i * cols + j];
            switch (op) {
                case 0: *d = v; break;
                case 1: *d += v; break;
                case 2: *d -= v; break;
                case 3: *d *= v; break;
                default: *d /= v; break;
            }
        }
}

/* dest[i, indices[i]] (op)= values[i] (dali/array/op/gather_from_rows.cpp:41-51,66-78). */
void orc_scatter_to_rows(float* dest, int64_t cols, const int32_t* indices, int64_t n, const float* values, int value_is_scalar, int op) {
    for (int64_t i = 0; i < n; ++i) {
        float* d = dest + i * cols + indices[i];
        const float v = value_is_scalar ? values[0] : values[i];
        switch (op) {
            case 0: *d = v; break;
            case 1: *d += v; break;
            case 2: *d -= v; break;
            case 3: *d *= v; break;
            default: *d /= v; break;
        }
    }
}

/* Running reduction along the last axis, the CPU loop of dali/array/op/scan.cpp:52-75: so_far starts at the
 * reducer's init value and takes the row's elements one by one. kind: 0 sum, 1 product, 2 maximum, 3 minimum.
 * inclusive: out has `cols` entries per row; exclusive: cols + 1, the first being the init value. */
void orc_axis_scan(int kind, const float* x, int64_t rows, int64_t cols, int inclusive, float* out) {
    const int64_t oc = cols + (inclusive ? 0 : 1);
    for (int64_t r = 0; r < rows; ++r) {
        float so_far = kind == 0 ? 0.0f : (kind == 1 ? 1.0f : (kind == 2 ? -FLT_MAX : FLT_MAX));
        if (!inclusive) out[r * oc] = so_far;
        for (int64_t i = 0; i < cols; ++i) {
            const float v = x[r * cols + i];
            if (kind == 0) so_far += v;
            else if (kind == 1) so_far *= v;
            else if (kind == 2) so_far = so_far > v ? so_far : v;
            else so_far = so_far < v ? so_far : v;
            out[r * oc + i + (inclusive ? 0 : 1)] = so_far;
        }
    }
}

/* out[r, x] = sum over s = 0..n-1 of content[r, (x + s) mod n] * weights[r, s], accumulated in that order
 * (dali/array/op/circular_convolution.cpp:22-38). */
void orc_circular_convolution(const float* content, const float* weights, int64_t rows, int64_t n, float* out) {
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t x = 0; x < n; ++x) {
            float res = 0.0f;
            for (int64_t s = 0; s < n; ++s) {
                int64_t off = x + s;
                if (off >= n) off -= n;
                res += content[r * n + off] * weights[r * n + s];
            }
            out[r * n + x] = res;
        }
}

/* ---- sliding-window nodes ------------------------------------------------------------------
 * Images are dense arrays whose four dimensions come in the order of the letters of `fmt` (a permutation of
 * "NCHW"); dims[k] is the extent of dimension k. */
static int fmt_pos(const char* fmt, char letter) {
    for (int k = 0; k < 4; ++k)
        if (fmt[k] == letter) return k;
    return -1;
}

static int64_t image_index(const int* dims, const char* fmt, int n, int c, int h, int w) {
    int64_t idx = 0;
    for (int k = 0; k < 4; ++k) {
        const int v = fmt[k] == 'N' ? n : (fmt[k] == 'C' ? c : (fmt[k] == 'H' ? h : w));
        idx = idx * dims[k] + v;
    }
    return idx;
}

/* The three letters other than N, last to first: the digits of a patch-row index from the fastest to the
 * slowest (dali/array/op/im2col.cpp:76-80; the same letters for N in position 0 or 1, the positions for which
 * those three lines name three different letters). */
static void row_letters(const char* fmt, char out[3]) {
    int k = 0;
    for (int p = 3; p >= 0; --p)
        if (fmt[p] != 'N') out[k++] = fmt[p];
}

static int letter_extent(char letter, int channels, int fh, int fw) { return letter == 'C' ? channels : (letter == 'H' ? fh : fw); }

/* row -> (c, kh, kw): dali/array/op/im2col.cpp:93-110 (offsets before the dilation factor is applied) */
static void split_row(const char* fmt, int row, int channels, int fh, int fw, int* c, int* kh, int* kw) {
    char l[3];
    row_letters(fmt, l);
    int rest = row;
    for (int k = 0; k < 3; ++k) {
        const int e = letter_extent(l[k], channels, fh, fw);
        const int v = rest % e;
        rest /= e;
        if (l[k] == 'C') *c = v;
        else if (l[k] == 'H') *kh = v;
        else *kw = v;
    }
}

/* (c, kh, kw) -> row: dali/array/op/col2im.cpp:86-94 */
static int join_row(const char* fmt, int channels, int fh, int fw, int c, int kh, int kw) {
    char l[3];
    row_letters(fmt, l);
    int row = 0;
    for (int k = 2; k >= 0; --k) {
        const int v = l[k] == 'C' ? c : (l[k] == 'H' ? kh : kw);
        row = row * letter_extent(l[k], channels, fh, fw) + v;
    }
    return row;
}

/* out[fh*fw*C, N*o_h*o_w]: every column is one patch of the zero-padded image
 * (dali/array/op/im2col.cpp:112-128). geom = {fh, fw, sh, sw, dh, dw, pre_h, pre_w, post_h, post_w}. */
void orc_im2col(const float* image, const int* dims, const char* fmt, const int* geom, float* out) {
    const int fh = geom[0], fw = geom[1], sh = geom[2], sw = geom[3], dh = geom[4], dw = geom[5];
    const int pre_h = geom[6], pre_w = geom[7], post_h = geom[8], post_w = geom[9];
    const int N = dims[fmt_pos(fmt, 'N')], Cc = dims[fmt_pos(fmt, 'C')], H = dims[fmt_pos(fmt, 'H')], W = dims[fmt_pos(fmt, 'W')];
    const int o_h = (H + pre_h + post_h - (dh * (fh - 1) + 1)) / sh + 1;
    const int o_w = (W + pre_w + post_w - (dw * (fw - 1) + 1)) / sw + 1;
    const int64_t rows = (int64_t)fh * fw * Cc, cols = (int64_t)N * o_h * o_w;
    for (int64_t q0 = 0; q0 < rows; ++q0) {
        int c = 0, kh = 0, kw = 0;
        split_row(fmt, (int)q0, Cc, fh, fw, &c, &kh, &kw);
        for (int64_t q1 = 0; q1 < cols; ++q1) {
            const int n = (int)(q1 / ((int64_t)o_h * o_w));
            const int w = (int)(q1 % o_w) * sw + kw * dw - pre_w;
            const int h = (int)((q1 / o_w) % o_h) * sh + kh * dh - pre_h;
            out[q0 * cols + q1] = (0 <= w && w < W && 0 <= h && h < H) ? image[image_index(dims, fmt, n, c, h, w)] : 0.0f;
        }
    }
}

/* The adjoint: every image element collects, patch rows outermost, the entries of the patch matrix that im2col
 * would have copied it to (dali/array/op/col2im.cpp:103-141). `dims` is the shape of the image to form. */
void orc_col2im(const float* input, const int* dims, const char* fmt, const int* geom, float* image) {
    const int fh = geom[0], fw = geom[1], sh = geom[2], sw = geom[3], dh = geom[4], dw = geom[5];
    const int pre_h = geom[6], pre_w = geom[7], post_h = geom[8], post_w = geom[9];
    const int N = dims[fmt_pos(fmt, 'N')], Cc = dims[fmt_pos(fmt, 'C')], H = dims[fmt_pos(fmt, 'H')], W = dims[fmt_pos(fmt, 'W')];
    const int o_h = (H + pre_h + post_h - (dh * (fh - 1) + 1)) / sh + 1;
    const int o_w = (W + pre_w + post_w - (dw * (fw - 1) + 1)) / sw + 1;
    const int64_t cols = (int64_t)N * o_h * o_w;
    const int patch_h = dh * (fh - 1) + 1, patch_w = dw * (fw - 1) + 1;
    for (int n = 0; n < N; ++n)
        for (int c = 0; c < Cc; ++c)
            for (int h0 = 0; h0 < H; ++h0)
                for (int w0 = 0; w0 < W; ++w0) {
                    const int h = h0 + pre_h, w = w0 + pre_w;
                    const int ph_min = h < patch_h ? h % dh : (h - patch_h + sh) / sh;
                    const int pw_min = w < patch_w ? w % dw : (w - patch_w + sw) / sw;
                    const int ph_max = (h + sh) / sh < o_h ? (h + sh) / sh : o_h;
                    const int pw_max = (w + sw) / sw < o_w ? (w + sw) / sw : o_w;
                    float res = 0.0f;
                    for (int ph = ph_min; ph < ph_max; ph += dh)
                        for (int pw = pw_min; pw < pw_max; pw += dw) {
                            const int row = join_row(fmt, Cc, fh, fw, c, (h - ph * sh) / dh, (w - pw * sw) / dw);
                            res += input[(int64_t)row * cols + ((int64_t)n * o_h + ph) * o_w + pw];
                        }
                    image[image_index(dims, fmt, n, c, h0, w0)] = res;
                }
}

/* Pooling over the window clipped to the image, columns outermost (dali/array/op/conv.cpp:66-89).
 * average = 0: maximum from -FLT_MAX; 1: the sum divided by the clipped window's area, converted to float.
 * x has dims (fmt is "NCHW" or "NHWC"); out has the same layout with (out_h, out_w). */
void orc_pool2d(const float* x, const int* dims, const char* fmt, int window_h, int window_w, int stride_h, int stride_w, int prepad_h,
                int prepad_w, int out_h, int out_w, int average, float* out) {
    const int N = dims[fmt_pos(fmt, 'N')], Cc = dims[fmt_pos(fmt, 'C')], H = dims[fmt_pos(fmt, 'H')], W = dims[fmt_pos(fmt, 'W')];
    int odims[4];
    for (int k = 0; k < 4; ++k) odims[k] = fmt[k] == 'H' ? out_h : (fmt[k] == 'W' ? out_w : dims[k]);
    for (int n = 0; n < N; ++n)
        for (int c = 0; c < Cc; ++c)
            for (int i = 0; i < out_h; ++i)
                for (int j = 0; j < out_w; ++j) {
                    int w_start = j * stride_w, w_end = w_start + window_w;
                    w_start = w_start - prepad_w > 0 ? w_start - prepad_w : 0;
                    w_end = w_end - prepad_w < W ? w_end - prepad_w : W;
                    int h_start = i * stride_h, h_end = h_start + window_h;
                    h_start = h_start - prepad_h > 0 ? h_start - prepad_h : 0;
                    h_end = h_end - prepad_h < H ? h_end - prepad_h : H;
                    float res = average ? 0.0f : -FLT_MAX;
                    for (int w = w_start; w < w_end; ++w)
                        for (int h = h_start; h < h_end; ++h) {
                            const float v = x[image_index(dims, fmt, n, c, h, w)];
                            if (average) res += v;
                            else res = res > v ? res : v;
                        }
                    if (average) res = res / (float)((h_end - h_start) * (w_end - w_start));
                    out[image_index(odims, fmt, n, c, i, j)] = res;
                }
}

/* dx[n,c,h,w] = sum over the windows (ph outer, pw inner) that hold (h, w) of PartialGrad(x, y[ph,pw]) *
 * dy[ph,pw], divided by the clipped window area for the average (dali/array/op/conv.cpp:133-172;
 * PartialGrad: jit/reducer_kernels.h:71-73 sum -> 1, :107-109 maximum -> y == x). */
void orc_pool2d_backward(const float* y, const float* dy, const float* x, const int* dims, const char* fmt, int window_h, int window_w,
                         int stride_h, int stride_w, int prepad_h, int prepad_w, int out_h, int out_w, int average, float* dx) {
    const int N = dims[fmt_pos(fmt, 'N')], Cc = dims[fmt_pos(fmt, 'C')], H = dims[fmt_pos(fmt, 'H')], W = dims[fmt_pos(fmt, 'W')];
    int odims[4];
    for (int k = 0; k < 4; ++k) odims[k] = fmt[k] == 'H' ? out_h : (fmt[k] == 'W' ? out_w : dims[k]);
    for (int n = 0; n < N; ++n)
        for (int c = 0; c < Cc; ++c)
            for (int h = 0; h < H; ++h)
                for (int w = 0; w < W; ++w) {
                    const float src = x[image_index(dims, fmt, n, c, h, w)];
                    const int ph_start = (h + prepad_h) < window_h ? 0 : (h + prepad_h - window_h) / stride_h + 1;
                    const int pw_start = (w + prepad_w) < window_w ? 0 : (w + prepad_w - window_w) / stride_w + 1;
                    const int ph_end = (h + prepad_h) / stride_h + 1 < out_h ? (h + prepad_h) / stride_h + 1 : out_h;
                    const int pw_end = (w + prepad_w) / stride_w + 1 < out_w ? (w + prepad_w) / stride_w + 1 : out_w;
                    float grad = 0.0f;
                    for (int ph = ph_start; ph < ph_end; ++ph)
                        for (int pw = pw_start; pw < pw_end; ++pw) {
                            const int64_t q = image_index(odims, fmt, n, c, ph, pw);
                            if (average) {
                                int hstart = ph * stride_h - prepad_h, wstart = pw * stride_w - prepad_w;
                                const int hend = hstart + window_h < H ? hstart + window_h : H;
                                const int wend = wstart + window_w < W ? wstart + window_w : W;
                                hstart = hstart > 0 ? hstart : 0;
                                wstart = wstart > 0 ? wstart : 0;
                                const int pool_size = (hend - hstart) * (wend - wstart);
                                grad += (1.0f * dy[q]) / (float)pool_size;
                            } else {
                                grad += (y[q] == src ? 1.0f : 0.0f) * dy[q];
                            }
                        }
                    dx[image_index(dims, fmt, n, c, h, w)] = grad;
                }
}

/* is_on = (indices[i] == j); on*is_on + (1.0 - is_on)*off, evaluated with T = float
 * for is_on and the 1.0 in double (dali/array/op/one_hot.cpp:38-46). */
void orc_one_hot(const int32_t* indices, int64_t n, int depth, float on, float off, float* out) {
    for (int64_t i = 0; i < n; ++i)
        for (int j = 0; j < depth; ++j) {
            float is_on = (float)(indices[i] == j);
            out[i * depth + j] = (float)((double)(on * is_on) + (1.0 - (double)is_on) * (double)off);
        }
}

/* Softmax cross-entropy in log-sum-exp form, one row at a time:
 *   m = max_j x;  s = sum_j exp(x - m);  lse = log(s) + m;  loss_i = lse - x[i, t_i]
 *   grad = exp(x - m)/s - one_hot(t)           (dout = 1)
 *   mean_loss = sum_i loss_i / (float)rows
 * Built from the reference's own nodes: keepdims max/sum (softmax.cpp:5-8),
 * gather_from_rows, one_hot, op::mean (reducers.cpp:32-41). The gradient is the
 * backward of dali/tensor/op/cost.cpp:122-129 (softmax * dout, then -= dout at
 * the target column) for dout = 1. */
void orc_softmax_cross_entropy(const float* x, const int32_t* t, int64_t rows, int64_t cols, float* loss_rows,
                               float* grad, float* mean_loss) {
    for (int64_t i = 0; i < rows; ++i) {
        const float* r = x + i * cols;
        float m = -FLT_MAX;
        for (int64_t j = 0; j < cols; ++j) m = m > r[j] ? m : r[j];
        float s = 0.0f;
        for (int64_t j = 0; j < cols; ++j) s += expf(r[j] - m);
        float lse = logf(s) + m;
        loss_rows[i] = lse - r[t[i]];
        if (grad) {
            float* g = grad + i * cols;
            for (int64_t j = 0; j < cols; ++j) {
                float is_on = (float)(t[i] == (int32_t)j);
                float oh = (float)((double)(1.0f * is_on) + (1.0 - (double)is_on) * (double)0.0f);
                g[j] = expf(r[j] - m) / s - oh;
            }
        }
    }
    if (mean_loss) *mean_loss = orc_mean_all(loss_rows, rows);
}

/* The reference's own forward: -1.0 * log(gather_from_rows(softmax(x), t))
 * (dali/tensor/op/cost.cpp:121-122); used to cross-check the LSE form. */
void orc_softmax_cross_entropy_via_probs(const float* x, const int32_t* t, int64_t rows, int64_t cols,
                                         float* loss_rows) {
    float* sm = (float*)malloc(sizeof(float) * (size_t)(rows * cols));
    orc_softmax(x, sm, rows, cols);
    for (int64_t i = 0; i < rows; ++i) loss_rows[i] = -1.0f * logf(sm[i * cols + t[i]]);
    free(sm);
}

/* --------------------------------------------------------------------- GEMM
 * Row-major C[M,N] = A[M,K] * B[K,N]; operands addressed through (row, col)
 * strides so that contiguous, transposed and row-strided views are all covered
 * (dali/array/op/dot.cpp:49-67 hands the BLAS contiguous-or-transposed
 * operands; dali/array/gemm/gemm_utils.cpp:7-21 derives (transpose, ld)).
 * Accumulates in double and rounds once: the truth the fp32 results are
 * compared against (the reference's cblas_sgemm rounding is unpinned). */
void orc_gemm_f64acc(const float* A, int64_t a_rs, int64_t a_cs, const float* B, int64_t b_rs, int64_t b_cs,
                     float* C, int64_t ldc, int M, int N, int K) {
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j) {
            double acc = 0.0;
            for (int k = 0; k < K; ++k) acc += (double)A[i * a_rs + k * a_cs] * (double)B[k * b_rs + j * b_cs];
            C[i * ldc + j] = (float)acc;
        }
}

/* Same product with an fp32 accumulator updated sequentially in k: the loop of
 * ReferenceGemm (dali/array/gemm/reference_gemm.h:27-73) instantiated for float.
 * i-k-j order so it runs at memory speed; per output element the additions still
 * happen in increasing k. */
void orc_gemm_f32seq(const float* A, int64_t a_rs, int64_t a_cs, const float* B, int64_t b_rs, int64_t b_cs,
                     float* C, int64_t ldc, int M, int N, int K) {
    for (int i = 0; i < M; ++i) {
        float* c = C + (int64_t)i * ldc;
        for (int j = 0; j < N; ++j) c[j] = 0.0f;
        for (int k = 0; k < K; ++k) {
            float a = A[i * a_rs + k * a_cs];
            const float* b = B + k * b_rs;
            if (b_cs == 1) {
                for (int j = 0; j < N; ++j) c[j] += a * b[j];
            } else {
                for (int j = 0; j < N; ++j) c[j] += a * b[j * b_cs];
            }
        }
    }
}

/* int32 product, the reference's ReferenceGemm<int>
 * (dali/array/gemm/reference_gemm.h:27-73 via dali/array/gemm/cpu_gemm.cpp:14-20). */
void orc_gemm_i32(const int32_t* A, int64_t a_rs, int64_t a_cs, const int32_t* B, int64_t b_rs, int64_t b_cs,
                  int32_t* C, int64_t ldc, int M, int N, int K) {
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j) {
            int32_t acc = 0;
            for (int k = 0; k < K; ++k) acc += A[i * a_rs + k * a_cs] * B[k * b_rs + j * b_cs];
            C[i * ldc + j] = acc;
        }
}

/* ---------------------------------------------------------------- LSTM step
 * gates[B,4H] = b + X*W + H*U (bias assigned first, then one += per product:
 * dali/tensor/op/composite.cpp:41-50); columns packed i, f, o, g;
 * i,f,o = sigmoid, g = tanh (dali/layers/lstm.cpp:226-238);
 * c' = f*c + i*g (lstm.cpp:241-248); h' = o*tanh(c') (lstm.cpp:261).
 * `gates` receives the pre-activation values. use_f64_gemm selects the truth
 * product (double accumulation) or the sequential fp32 one. */
void orc_lstm_step(const float* X, const float* Hprev, const float* Cprev, const float* W, const float* U,
                   const float* bias, int B, int I, int H, int use_f64_gemm, float* gates, float* c_new,
                   float* h_new) {
    int N = 4 * H;
    float* xw = (float*)malloc(sizeof(float) * (size_t)B * N);
    float* hu = (float*)malloc(sizeof(float) * (size_t)B * N);
    if (use_f64_gemm) {
        orc_gemm_f64acc(X, I, 1, W, N, 1, xw, N, B, N, I);
        orc_gemm_f64acc(Hprev, H, 1, U, N, 1, hu, N, B, N, H);
    } else {
        orc_gemm_f32seq(X, I, 1, W, N, 1, xw, N, B, N, I);
        orc_gemm_f32seq(Hprev, H, 1, U, N, 1, hu, N, B, N, H);
    }
    for (int r = 0; r < B; ++r)
        for (int j = 0; j < N; ++j) {
            float g = bias[j];
            g = g + xw[(int64_t)r * N + j];
            g = g + hu[(int64_t)r * N + j];
            gates[(int64_t)r * N + j] = g;
        }
    for (int r = 0; r < B; ++r)
        for (int j = 0; j < H; ++j) {
            const float* g = gates + (int64_t)r * N;
            float ig = f_sigmoid(g[j]);
            float fg = f_sigmoid(g[H + j]);
            float og = f_sigmoid(g[2 * H + j]);
            float cw = f_tanh(g[3 * H + j]);
            float c = f_add(f_eltmul(fg, Cprev[(int64_t)r * H + j]), f_eltmul(ig, cw));
            c_new[(int64_t)r * H + j] = c;
            h_new[(int64_t)r * H + j] = f_eltmul(og, f_tanh(c));
        }
    free(xw);
    free(hu);
}
