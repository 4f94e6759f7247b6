/*
 * dali_front.h — flat C binding of the C++ host front-end (dali_amd/host/dali.h)
 * so that scripting languages can build the same lazy expressions a C++ user of
 * the reference writes with `Array` and `op::` (dali/array/array.h:18-230,
 * dali/array/op.h:1-26). Handles are opaque; every function that can fail
 * returns NULL / non-zero and leaves a message in dali_fe_last_error().
 * The device work itself goes through the C ABI of include/dali_hip.h.
 */
#ifndef DALI_FRONT_H
#define DALI_FRONT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* dali_array_t;

const char* dali_fe_last_error(void);

/* construction (dali/array/array.h:31-62) */
dali_array_t dali_fe_from_host(const void* data, const int* shape, int ndim, int dtype);
/* the same with the host copy in pinned memory, and the non-blocking migration it allows (to_device != 0: host to
 * device, else device to host); replaces the blocking copy of SynchronizedMemory::move_to
 * (dali/array/memory/synchronized_memory.cpp:268-314) where the caller asks for it */
dali_array_t dali_fe_from_host_pinned(const void* data, const int* shape, int ndim, int dtype);
int dali_fe_prefetch(dali_array_t a, int to_device);
dali_array_t dali_fe_empty(const int* shape, int ndim, int dtype);
dali_array_t dali_fe_zeros(const int* shape, int ndim, int dtype);
dali_array_t dali_fe_scalar_double(double v);
dali_array_t dali_fe_scalar_float(float v);
dali_array_t dali_fe_scalar_int(int v);
dali_array_t dali_fe_clone_handle(dali_array_t a);
void dali_fe_release(dali_array_t a);

/* inspection */
int dali_fe_ndim(dali_array_t a);
int dali_fe_shape(dali_array_t a, int* out);   /* writes ndim ints */
int dali_fe_dtype(dali_array_t a);
int dali_fe_is_buffer(dali_array_t a);
int dali_fe_is_contiguous(dali_array_t a);
int dali_fe_strides(dali_array_t a, int* out); /* normalized strides, ndim ints */
int dali_fe_offset(dali_array_t a);

/* views (dali/array/array.h:120-160) */
dali_array_t dali_fe_transpose(dali_array_t a, const int* axes, int naxes); /* naxes == 0: reverse */
dali_array_t dali_fe_pluck_axis(dali_array_t a, int axis, int idx);
dali_array_t dali_fe_slice(dali_array_t a, int axis, int start, int end, int step);
dali_array_t dali_fe_reshape(dali_array_t a, const int* shape, int ndim);
dali_array_t dali_fe_expand_dims(dali_array_t a, int axis);
dali_array_t dali_fe_squeeze(dali_array_t a, int axis);
dali_array_t dali_fe_ascontiguousarray(dali_array_t a);

/* lazy ops (headers under dali/array/op) */
dali_array_t dali_fe_unary(const char* functor_name, dali_array_t a);
dali_array_t dali_fe_binary(const char* functor_name, dali_array_t a, dali_array_t b);
dali_array_t dali_fe_astype(dali_array_t a, int dtype);
dali_array_t dali_fe_all_reduce(const char* reducer_name, dali_array_t a);
dali_array_t dali_fe_axis_reduce(const char* reducer_name, dali_array_t a, const int* axes, int naxes, int keepdims);
dali_array_t dali_fe_arg_all_reduce(const char* reducer_name, dali_array_t a);
dali_array_t dali_fe_arg_axis_reduce(const char* reducer_name, dali_array_t a, int axis);
dali_array_t dali_fe_mean_all(dali_array_t a);
dali_array_t dali_fe_mean_axes(dali_array_t a, const int* axes, int naxes, int keepdims);
dali_array_t dali_fe_softmax(dali_array_t a, int axis);
/* the written-out expression exp(a - max) / sum(exp(a - max)) of dali/array/op/softmax.cpp:5-8, which dali_fe_softmax turns into when it is evaluated */
dali_array_t dali_fe_softmax_naive(dali_array_t a, int axis);
/* op::softmax_temperature (dali/array/op/softmax.cpp:10-13): the reference ignores the temperature, and so does this */
dali_array_t dali_fe_softmax_temperature(dali_array_t a, dali_array_t temperature, int axis);
/* op::ceil (dali/array/op/elementwise_operation.cpp:155-160): int32 result, int32 operands pass through */
dali_array_t dali_fe_ceil(dali_array_t a);
dali_array_t dali_fe_gather_from_rows(dali_array_t source, dali_array_t indices);
/* op::gather (dali/array/op/gather.cpp:163-171); assigning to the lazy result scatters into `source` */
dali_array_t dali_fe_gather(dali_array_t source, dali_array_t indices);
/* op::axis_scan (dali/array/op/scan.cpp:183-194): reducer "reducers::sum" / "reducers::product" / ... along the last axis */
dali_array_t dali_fe_axis_scan(dali_array_t a, const char* reducer, int inclusive);
/* op::arange over 0-d start / stop / step (dali/array/op/arange.cpp:47-57) */
dali_array_t dali_fe_arange(dali_array_t start, dali_array_t stop, dali_array_t step);
/* op::diag / op::eye (dali/array/op/eye.cpp:46-77): `diagonal` is a vector or a 0-d value */
dali_array_t dali_fe_diag(dali_array_t diagonal, int rows, int cols);
/* op::circular_convolution (dali/array/op/circular_convolution.cpp:82-86) */
dali_array_t dali_fe_circular_convolution(dali_array_t x, dali_array_t weights);
/* op::concatenate (dali/array/op/concatenate.cpp:9-73); hstack = axis -1, vstack = axis 0 */
dali_array_t dali_fe_concatenate(dali_array_t* arrays, int n, int axis);
/* Sliding-window operators. data_format is a permutation of "NCHW" naming the order of the image's dimensions
 * (conv2d and the pooling pair accept "NCHW" and "NHWC"); padding: 0 = SAME, 1 = VALID and pooling: 0 = max, 1 = average,
 * the values of dali/array/op/spatial_enums.h.
 * op::im2col (dali/array/op/im2col.cpp:190-267), op::col2im (dali/array/op/col2im.cpp:165-233) */
dali_array_t dali_fe_im2col(dali_array_t image, int filter_h, int filter_w, int stride_h, int stride_w, int padding_h, int padding_w,
                            int postpad_h, int postpad_w, const char* data_format);
dali_array_t dali_fe_col2im(dali_array_t input, const int* image_shape, int image_ndim, int filter_h, int filter_w, int stride_h,
                            int stride_w, const char* data_format);
/* op::conv2d and its three gradients (dali/array/op/conv.cpp:223-401) */
dali_array_t dali_fe_conv2d(dali_array_t input, dali_array_t filters, int stride_h, int stride_w, int padding, const char* data_format);
dali_array_t dali_fe_conv2d_backward_input(dali_array_t filters, dali_array_t out_dw, int stride_h, int stride_w, const int* input_shape,
                                           int padding, const char* data_format);
dali_array_t dali_fe_conv2d_backward_filters(dali_array_t input, dali_array_t out_dw, int stride_h, int stride_w, const int* filters_shape,
                                             int padding, const char* data_format);
dali_array_t dali_fe_conv2d_backward_bias(dali_array_t out_dw, const char* data_format);
/* op::pool2d / op::pool2d_backward (dali/array/op/conv.cpp:403-456) */
dali_array_t dali_fe_pool2d(dali_array_t input, int window_h, int window_w, int stride_h, int stride_w, int pooling, int padding,
                            const char* data_format);
dali_array_t dali_fe_pool2d_backward(dali_array_t out, dali_array_t out_dw, dali_array_t in, int window_h, int window_w, int stride_h,
                                     int stride_w, int pooling, int padding, const char* data_format);
/* op::outer (dali/array/op/outer.cpp:33-36) */
dali_array_t dali_fe_outer(dali_array_t a, dali_array_t b);
/* dest <<= source (dali/array/expression/assignment.cpp:92-126) */
int dali_fe_autoreduce_assign(dali_array_t dest, dali_array_t source);
dali_array_t dali_fe_one_hot(dali_array_t indices, int depth, dali_array_t on_value, dali_array_t off_value);
/* op::dot (dali/array/op/dot.cpp:104-124): scalars multiply, vectors and matrices go to one matrix product, operands of
 * more than two dimensions to tensordot over a's last axis and b's second to last */
dali_array_t dali_fe_dot(dali_array_t a, dali_array_t b);
/* op::tensordot (dali/array/op/dot.cpp:92-98, dali/array/gemm/tensordot_as_dot.h:48-158). With both axis lists NULL the
 * last n_axes axes of a are summed against the first n_axes axes of b; otherwise axis a_reduce_axes[i] of a against axis
 * b_reduce_axes[i] of b. The result holds the kept axes of a, then those of b. */
/* op::top_k (largest != 0) / op::bottom_k (largest == 0): int32 column numbers of the k best entries along the last axis,
 * best first (dali/array/op/top_k.cpp:198-220); op::argsort over the flattened array (flat != 0) or along an axis
 * (dali/array/op/top_k.cpp:222-233) */
dali_array_t dali_fe_top_k(dali_array_t a, int k, int sorted, int largest);
dali_array_t dali_fe_argsort(dali_array_t a, int axis, int flat);
/* op::inner and op::matrix_vector_dot (dali/array/op/dot.cpp:67-90,100-102) */
dali_array_t dali_fe_inner(dali_array_t a, dali_array_t b);
dali_array_t dali_fe_matrix_vector_dot(dali_array_t a, dali_array_t b);
dali_array_t dali_fe_tensordot(dali_array_t a, dali_array_t b, int n_axes, const int* a_reduce_axes, const int* b_reduce_axes);

/* composites evaluated as one fused group */
int dali_fe_softmax_cross_entropy(dali_array_t logits, dali_array_t targets, dali_array_t* mean_loss,
                                  dali_array_t* row_loss, dali_array_t* grad);
int dali_fe_lstm_step(dali_array_t x, dali_array_t h, dali_array_t c, dali_array_t W, dali_array_t U, dali_array_t b,
                      dali_array_t* c_new, dali_array_t* h_new);
/* The LSTM step along xs[T, B, I] (dali/layers/lstm.cpp:294-303): hidden_states [T, B, H], final memory and hidden [B, H] */
int dali_fe_lstm_sequence(dali_array_t xs, dali_array_t h0, dali_array_t c0, dali_array_t W, dali_array_t U, dali_array_t b,
                          dali_array_t* hidden_states, dali_array_t* memory, dali_array_t* hidden);
/* One step of a stack of `layers` LSTM cells (dali/layers/stacked_lstm.cpp:219-283, no dropout): layer l reads the new
 * hidden state of layer l-1; with `shortcut` the layers above the first also read x and their W is
 * [H(l-1) + I, 4 H(l)], hidden-state rows first. c_new and h_new receive `layers` handles each. */
int dali_fe_stacked_lstm_step(dali_array_t x, int layers, const dali_array_t* h, const dali_array_t* c, const dali_array_t* W,
                              const dali_array_t* U, const dali_array_t* b, int shortcut, dali_array_t* c_new, dali_array_t* h_new);
/* The stack along a sequence xs [T, B, I] (AbstractStackedLSTM::activate_sequence, dali/layers/stacked_lstm.cpp:44-51): the
 * final memory and hidden state of every layer and the hidden states [T, B, H] of the top layer */
int dali_fe_stacked_lstm_sequence(dali_array_t xs, int layers, const dali_array_t* h, const dali_array_t* c, const dali_array_t* W,
                                  const dali_array_t* U, const dali_array_t* b, int shortcut, dali_array_t* c_last, dali_array_t* h_last,
                                  dali_array_t* top_states);
/* One GRU step, layers packed reset / update / candidate along the columns of W[I,3H], U[H,3H], b[3H]
 * (dali/layers/gru.cpp:27-44) */
dali_array_t dali_fe_gru_step(dali_array_t x, dali_array_t h, dali_array_t W, dali_array_t U, dali_array_t b);
/* The step along a sequence xs [T, B, I] from the state h0 (GRU::activate_sequence, dali/layers/gru.cpp:59-64): every state
 * [T, B, H] and the last one; the input half of all steps is one product */
int dali_fe_gru_sequence(dali_array_t xs, dali_array_t h0, dali_array_t W, dali_array_t U, dali_array_t b, dali_array_t* states, dali_array_t* last);

/* evaluation, assignment, host access */
int dali_fe_eval(dali_array_t a);
int dali_fe_eval_together(dali_array_t* roots, int n);
int dali_fe_assign(dali_array_t dest, int operator_t, dali_array_t source); /* 0 =, 1 +=, 2 -=, 3 *=, 4 /= */
int dali_fe_to_host(dali_array_t a, void* out);
void* dali_fe_device_ptr(dali_array_t a);

/* observation (dali/utils/scope.h, dali/array/tests/dot_tests.cpp:17-36) */
int dali_fe_stats(uint64_t* kernels, uint64_t* gemms, uint64_t* evals, uint64_t* plans);
/* evaluations that reused a stored plan (same structure: kinds, functors, dtypes, shapes, buffer layouts and sharing)
 * instead of running the planner, and plans stored so far; DALI_HIP_PLAN_CACHE=0 turns the cache off,
 * DALI_HIP_PLAN_CACHE_CHECK=1 runs the planner beside every reuse and raises if the two disagree */
int dali_fe_plan_cache_stats(uint64_t* hits, uint64_t* stored);
/* Named scopes around the front-end's work (dali/utils/scope.h: Scope, ScopeObserver): on_enter / on_exit are called
 * with the scope's name and the number of scopes open (the reported one included) when a scope opens and closes. The
 * front-end opens "JIT[<kernel shape>:<entry point>]" around every generated kernel it launches
 * (dali/array/expression/computation.cpp:19), inside it "get_function" while the kernel is not loaded and, inside that,
 * "compilation" around the build from source (dali/array/jit/jit.cpp:1015,1025), and "gemm" / "gemm_pair" around a
 * product. Either callback may be NULL. Returns the handle dali_fe_scope_unobserve takes. Without observers a scope
 * costs one test. */
typedef void (*dali_fe_scope_callback)(const char* name, int depth, void* user);
int dali_fe_scope_observe(dali_fe_scope_callback on_enter, dali_fe_scope_callback on_exit, void* user);
void dali_fe_scope_unobserve(int handle);
const char* dali_fe_last_kernel_kinds(void);
const char* dali_fe_last_kernel_names(void);
const char* dali_fe_last_source(void);
/* Launch recording: between begin and end every kernel and GEMM launch issued by
 * evaluations is also stored (with the buffers it touches kept alive); replay
 * re-issues the stored launches `times` times on the library stream without
 * rebuilding or re-planning the expressions. */
void* dali_fe_record_begin(void);
int dali_fe_record_end(void* recording); /* number of stored launches */
/* instantiate a HIP graph of the stored launches; later replays launch the graph */
int dali_fe_record_make_graph(void* recording);
int dali_fe_replay(void* recording, int times);
void dali_fe_record_free(void* recording);

/* While on, evaluations and assignments plan and generate their kernels (and compile them with hipRTC when `compile` is set)
 * but launch nothing and touch no device: the way to check code generation for statements that are not plain roots, such as
 * an assignment through a gather. dali_fe_last_source holds the generated text. */
int dali_fe_set_dry_run(int on, int compile);

/* plan + generate (and optionally hipRTC-compile for gfx950) without a device;
 * returns the number of kernels, -1 on error */
int dali_fe_generate_only(dali_array_t* roots, int n, int compile);
/* source of the i-th of those kernels, in launch order ("" outside the range); valid until the next dali_fe_generate_only */
const char* dali_fe_generated_source(int i);

#ifdef __cplusplus
}
#endif
#endif /* DALI_FRONT_H */
