// Flat C binding of the front-end, declared in include/dali_front.h.
#include "../../include/dali_front.h"

#include <cstring>

#include "../../include/dali_hip.h"
#include "expr.h"

using dali::Array;

static thread_local std::string g_err;
static thread_local std::string g_kinds;

#include <functional>

namespace dali {
void set_dry_compile(bool on);
void set_recording(std::vector<std::function<void()>>* rec, std::vector<std::shared_ptr<memory::SynchronizedMemory>>* written);
}

#define FE_TRY(body, failure)               \
    try {                                   \
        body                                \
    } catch (const std::exception& ex) {    \
        g_err = ex.what();                  \
        return failure;                     \
    }

static Array& A(dali_array_t h) {
    if (!h) throw std::runtime_error("NULL array handle");
    return *(Array*)h;
}
static dali_array_t wrap(const Array& a) { return (dali_array_t) new Array(a); }
static std::vector<int> vec(const int* p, int n) { return n > 0 ? std::vector<int>(p, p + n) : std::vector<int>(); }

extern "C" {

const char* dali_fe_last_error(void) { return g_err.c_str(); }

dali_array_t dali_fe_from_host(const void* data, const int* shape, int ndim, int dtype) {
    FE_TRY(return wrap(Array::from_host(data, vec(shape, ndim), (dali::DType)dtype));, nullptr)
}
dali_array_t dali_fe_from_host_pinned(const void* data, const int* shape, int ndim, int dtype) {
    FE_TRY(return wrap(Array::from_host_pinned(data, vec(shape, ndim), (dali::DType)dtype));, nullptr)
}
int dali_fe_prefetch(dali_array_t a, int to_device) {
    FE_TRY(if (to_device) A(a).prefetch_to_device(); else A(a).prefetch_to_host(); return 0;, 1)
}
dali_array_t dali_fe_empty(const int* shape, int ndim, int dtype) {
    FE_TRY(return wrap(Array(vec(shape, ndim), (dali::DType)dtype));, nullptr)
}
dali_array_t dali_fe_zeros(const int* shape, int ndim, int dtype) {
    FE_TRY(return wrap(Array::zeros(vec(shape, ndim), (dali::DType)dtype));, nullptr)
}
dali_array_t dali_fe_scalar_double(double v) { FE_TRY(return wrap(Array(v));, nullptr) }
dali_array_t dali_fe_scalar_float(float v) { FE_TRY(return wrap(Array(v));, nullptr) }
dali_array_t dali_fe_scalar_int(int v) { FE_TRY(return wrap(Array(v));, nullptr) }
dali_array_t dali_fe_clone_handle(dali_array_t a) { FE_TRY(return wrap(A(a));, nullptr) }
void dali_fe_release(dali_array_t a) { delete (Array*)a; }

int dali_fe_ndim(dali_array_t a) { FE_TRY(return A(a).ndim();, -1) }
int dali_fe_shape(dali_array_t a, int* out) {
    FE_TRY(const auto& s = A(a).shape(); for (size_t i = 0; i < s.size(); ++i) out[i] = s[i]; return 0;, 1)
}
int dali_fe_dtype(dali_array_t a) { FE_TRY(return (int)A(a).dtype();, -1) }
int dali_fe_is_buffer(dali_array_t a) { FE_TRY(return A(a).is_buffer() ? 1 : 0;, -1) }
int dali_fe_is_contiguous(dali_array_t a) { FE_TRY(return A(a).contiguous_memory() ? 1 : 0;, -1) }
int dali_fe_strides(dali_array_t a, int* out) {
    FE_TRY(auto s = A(a).normalized_strides(); for (size_t i = 0; i < s.size(); ++i) out[i] = s[i]; return 0;, 1)
}
int dali_fe_offset(dali_array_t a) { FE_TRY(return A(a).offset();, -1) }

dali_array_t dali_fe_transpose(dali_array_t a, const int* axes, int naxes) {
    FE_TRY(return wrap(naxes ? A(a).transpose(vec(axes, naxes)) : A(a).transpose());, nullptr)
}
dali_array_t dali_fe_pluck_axis(dali_array_t a, int axis, int idx) { FE_TRY(return wrap(A(a).pluck_axis(axis, idx));, nullptr) }
dali_array_t dali_fe_slice(dali_array_t a, int axis, int start, int end, int step) {
    FE_TRY(return wrap(A(a).slice(axis, start, end, step));, nullptr)
}
dali_array_t dali_fe_reshape(dali_array_t a, const int* shape, int ndim) { FE_TRY(return wrap(A(a).reshape(vec(shape, ndim)));, nullptr) }
dali_array_t dali_fe_expand_dims(dali_array_t a, int axis) { FE_TRY(return wrap(A(a).expand_dims(axis));, nullptr) }
dali_array_t dali_fe_squeeze(dali_array_t a, int axis) { FE_TRY(return wrap(A(a).squeeze(axis));, nullptr) }
dali_array_t dali_fe_ascontiguousarray(dali_array_t a) { FE_TRY(return wrap(A(a).ascontiguousarray());, nullptr) }

static std::string qualified(const char* name, const char* ns) {
    std::string s(name);
    return s.find("::") == std::string::npos ? std::string(ns) + "::" + s : s;
}

dali_array_t dali_fe_unary(const char* functor_name, dali_array_t a) {
    FE_TRY(return wrap(dali::op::elementwise(A(a), qualified(functor_name, "functor")));, nullptr)
}
dali_array_t dali_fe_binary(const char* functor_name, dali_array_t a, dali_array_t b) {
    FE_TRY(return wrap(dali::op::elementwise(A(a), A(b), qualified(functor_name, "functor")));, nullptr)
}
dali_array_t dali_fe_ceil(dali_array_t a) { FE_TRY(return wrap(dali::op::ceil(A(a)));, nullptr) }
dali_array_t dali_fe_astype(dali_array_t a, int dtype) { FE_TRY(return wrap(dali::op::astype(A(a), (dali::DType)dtype));, nullptr) }
dali_array_t dali_fe_all_reduce(const char* r, dali_array_t a) {
    FE_TRY(return wrap(dali::op::all_reduce(A(a), qualified(r, "reducers")));, nullptr)
}
dali_array_t dali_fe_axis_reduce(const char* r, dali_array_t a, const int* axes, int naxes, int keepdims) {
    FE_TRY(return wrap(dali::op::axis_reduce(A(a), qualified(r, "reducers"), vec(axes, naxes), keepdims != 0));, nullptr)
}
dali_array_t dali_fe_arg_all_reduce(const char* r, dali_array_t a) {
    FE_TRY(return wrap(dali::op::argument_all_reduce(A(a), qualified(r, "reducers")));, nullptr)
}
dali_array_t dali_fe_arg_axis_reduce(const char* r, dali_array_t a, int axis) {
    FE_TRY(return wrap(dali::op::argument_axis_reduce(A(a), qualified(r, "reducers"), axis));, nullptr)
}
dali_array_t dali_fe_mean_all(dali_array_t a) { FE_TRY(return wrap(dali::op::mean(A(a)));, nullptr) }
dali_array_t dali_fe_mean_axes(dali_array_t a, const int* axes, int naxes, int keepdims) {
    FE_TRY(return wrap(dali::op::mean(A(a), vec(axes, naxes), keepdims != 0));, nullptr)
}
dali_array_t dali_fe_softmax(dali_array_t a, int axis) { FE_TRY(return wrap(dali::op::softmax(A(a), axis));, nullptr) }
dali_array_t dali_fe_softmax_naive(dali_array_t a, int axis) { FE_TRY(return wrap(dali::op::softmax_naive(A(a), axis));, nullptr) }
dali_array_t dali_fe_softmax_temperature(dali_array_t a, dali_array_t temperature, int axis) {
    FE_TRY(return wrap(dali::op::softmax_temperature(A(a), A(temperature), axis));, nullptr)
}
dali_array_t dali_fe_gather_from_rows(dali_array_t s, dali_array_t i) { FE_TRY(return wrap(dali::op::gather_from_rows(A(s), A(i)));, nullptr) }
dali_array_t dali_fe_gather(dali_array_t s, dali_array_t i) { FE_TRY(return wrap(dali::op::gather(A(s), A(i)));, nullptr) }
int dali_fe_autoreduce_assign(dali_array_t dest, dali_array_t source) { FE_TRY(dali::op::autoreduce_assign(A(dest), A(source)); return 0;, 1) }
dali_array_t dali_fe_axis_scan(dali_array_t a, const char* reducer, int inclusive) {
    FE_TRY(return wrap(dali::op::axis_scan(A(a), reducer, inclusive != 0));, nullptr)
}
dali_array_t dali_fe_arange(dali_array_t start, dali_array_t stop, dali_array_t step) {
    FE_TRY(return wrap(dali::op::arange(A(start), A(stop), A(step)));, nullptr)
}
dali_array_t dali_fe_diag(dali_array_t diagonal, int rows, int cols) { FE_TRY(return wrap(dali::op::diag(A(diagonal), rows, cols));, nullptr) }
dali_array_t dali_fe_circular_convolution(dali_array_t x, dali_array_t w) { FE_TRY(return wrap(dali::op::circular_convolution(A(x), A(w)));, nullptr) }
dali_array_t dali_fe_concatenate(dali_array_t* arrays, int n, int axis) {
    FE_TRY(std::vector<Array> v; for (int i = 0; i < n; ++i) v.push_back(A(arrays[i])); return wrap(dali::op::concatenate(v, axis));, nullptr)
}
dali_array_t dali_fe_im2col(dali_array_t image, int filter_h, int filter_w, int stride_h, int stride_w, int padding_h, int padding_w,
                            int postpad_h, int postpad_w, const char* data_format) {
    FE_TRY(return wrap(dali::op::im2col(A(image), filter_h, filter_w, stride_h, stride_w, padding_h, padding_w, postpad_h, postpad_w, data_format));
           , nullptr)
}
dali_array_t dali_fe_col2im(dali_array_t input, const int* image_shape, int image_ndim, int filter_h, int filter_w, int stride_h,
                            int stride_w, const char* data_format) {
    FE_TRY(return wrap(dali::op::col2im(A(input), std::vector<int>(image_shape, image_shape + image_ndim), filter_h, filter_w, stride_h, stride_w,
                                        data_format));
           , nullptr)
}
dali_array_t dali_fe_conv2d(dali_array_t input, dali_array_t filters, int stride_h, int stride_w, int padding, const char* data_format) {
    FE_TRY(return wrap(dali::op::conv2d(A(input), A(filters), stride_h, stride_w, (dali::PADDING_T)padding, data_format));, nullptr)
}
dali_array_t dali_fe_conv2d_backward_input(dali_array_t filters, dali_array_t out_dw, int stride_h, int stride_w, const int* input_shape,
                                           int padding, const char* data_format) {
    FE_TRY(return wrap(dali::op::conv2d_backward_input(A(filters), A(out_dw), stride_h, stride_w, std::vector<int>(input_shape, input_shape + 4),
                                                       (dali::PADDING_T)padding, data_format));
           , nullptr)
}
dali_array_t dali_fe_conv2d_backward_filters(dali_array_t input, dali_array_t out_dw, int stride_h, int stride_w, const int* filters_shape,
                                             int padding, const char* data_format) {
    FE_TRY(return wrap(dali::op::conv2d_backward_filters(A(input), A(out_dw), stride_h, stride_w,
                                                         std::vector<int>(filters_shape, filters_shape + 4), (dali::PADDING_T)padding, data_format));
           , nullptr)
}
dali_array_t dali_fe_conv2d_backward_bias(dali_array_t out_dw, const char* data_format) {
    FE_TRY(return wrap(dali::op::conv2d_backward_bias(A(out_dw), data_format));, nullptr)
}
dali_array_t dali_fe_pool2d(dali_array_t input, int window_h, int window_w, int stride_h, int stride_w, int pooling, int padding,
                            const char* data_format) {
    FE_TRY(return wrap(dali::op::pool2d(A(input), window_h, window_w, stride_h, stride_w, (dali::POOLING_T)pooling, (dali::PADDING_T)padding,
                                        data_format));
           , nullptr)
}
dali_array_t dali_fe_pool2d_backward(dali_array_t out, dali_array_t out_dw, dali_array_t in, int window_h, int window_w, int stride_h,
                                     int stride_w, int pooling, int padding, const char* data_format) {
    FE_TRY(return wrap(dali::op::pool2d_backward(A(out), A(out_dw), A(in), window_h, window_w, stride_h, stride_w, (dali::POOLING_T)pooling,
                                                 (dali::PADDING_T)padding, data_format));
           , nullptr)
}
dali_array_t dali_fe_outer(dali_array_t a, dali_array_t b) { FE_TRY(return wrap(dali::op::outer(A(a), A(b)));, nullptr) }
dali_array_t dali_fe_one_hot(dali_array_t indices, int depth, dali_array_t on_value, dali_array_t off_value) {
    FE_TRY(return wrap(dali::op::one_hot(A(indices), depth, A(on_value), A(off_value)));, nullptr)
}
dali_array_t dali_fe_dot(dali_array_t a, dali_array_t b) { FE_TRY(return wrap(dali::op::dot(A(a), A(b)));, nullptr) }
dali_array_t dali_fe_inner(dali_array_t a, dali_array_t b) { FE_TRY(return wrap(dali::op::inner(A(a), A(b)));, nullptr) }
dali_array_t dali_fe_matrix_vector_dot(dali_array_t a, dali_array_t b) { FE_TRY(return wrap(dali::op::matrix_vector_dot(A(a), A(b)));, nullptr) }
dali_array_t dali_fe_top_k(dali_array_t a, int k, int sorted, int largest) {
    FE_TRY(return wrap(largest ? dali::op::top_k(A(a), k, sorted != 0) : dali::op::bottom_k(A(a), k, sorted != 0));, nullptr)
}
dali_array_t dali_fe_argsort(dali_array_t a, int axis, int flat) {
    FE_TRY(return wrap(flat ? dali::op::argsort(A(a)) : dali::op::argsort(A(a), axis));, nullptr)
}
dali_array_t dali_fe_tensordot(dali_array_t a, dali_array_t b, int n_axes, const int* a_reduce_axes, const int* b_reduce_axes) {
    FE_TRY(if (!a_reduce_axes || !b_reduce_axes) return wrap(dali::op::tensordot(A(a), A(b), n_axes));
           return wrap(dali::op::tensordot(A(a), A(b), std::vector<int>(a_reduce_axes, a_reduce_axes + n_axes),
                                           std::vector<int>(b_reduce_axes, b_reduce_axes + n_axes)));
           , nullptr)
}

int dali_fe_softmax_cross_entropy(dali_array_t logits, dali_array_t targets, dali_array_t* mean_loss, dali_array_t* row_loss,
                                  dali_array_t* grad) {
    FE_TRY(auto r = dali::op::softmax_cross_entropy(A(logits), A(targets)); *mean_loss = wrap(r.mean_loss); *row_loss = wrap(r.row_loss);
           *grad = wrap(r.grad); return 0;
           , 1)
}
int dali_fe_lstm_step(dali_array_t x, dali_array_t h, dali_array_t c, dali_array_t W, dali_array_t U, dali_array_t b,
                      dali_array_t* c_new, dali_array_t* h_new) {
    FE_TRY(auto r = dali::op::lstm_step(A(x), A(h), A(c), A(W), A(U), A(b)); *c_new = wrap(r.memory); *h_new = wrap(r.hidden); return 0;, 1)
}

int dali_fe_lstm_sequence(dali_array_t xs, dali_array_t h0, dali_array_t c0, dali_array_t W, dali_array_t U, dali_array_t b,
                          dali_array_t* hidden_states, dali_array_t* memory, dali_array_t* hidden) {
    FE_TRY(auto r = dali::op::lstm_sequence(A(xs), A(h0), A(c0), A(W), A(U), A(b)); *hidden_states = wrap(r.hidden_states);
           *memory = wrap(r.memory); *hidden = wrap(r.hidden); return 0;
           , 1)
}
static int stacked_lstm_step_impl(dali_array_t x, int layers, const dali_array_t* h, const dali_array_t* c, const dali_array_t* W, const dali_array_t* U,
                                  const dali_array_t* b, int shortcut, dali_array_t* c_new, dali_array_t* h_new) {
    std::vector<Array> hv, cv, Wv, Uv, bv;
    for (int l = 0; l < layers; ++l) {
        hv.push_back(A(h[l]));
        cv.push_back(A(c[l]));
        Wv.push_back(A(W[l]));
        Uv.push_back(A(U[l]));
        bv.push_back(A(b[l]));
    }
    auto r = dali::op::stacked_lstm_step(A(x), hv, cv, Wv, Uv, bv, shortcut != 0);
    for (int l = 0; l < layers; ++l) {
        c_new[l] = wrap(r.memory[l]);
        h_new[l] = wrap(r.hidden[l]);
    }
    return 0;
}
int dali_fe_stacked_lstm_step(dali_array_t x, int layers, const dali_array_t* h, const dali_array_t* c, const dali_array_t* W, const dali_array_t* U,
                              const dali_array_t* b, int shortcut, dali_array_t* c_new, dali_array_t* h_new) {
    FE_TRY(return stacked_lstm_step_impl(x, layers, h, c, W, U, b, shortcut, c_new, h_new);, 1)
}
static int stacked_lstm_sequence_impl(dali_array_t xs, int layers, const dali_array_t* h, const dali_array_t* c, const dali_array_t* W,
                                      const dali_array_t* U, const dali_array_t* b, int shortcut, dali_array_t* c_last, dali_array_t* h_last,
                                      dali_array_t* top_states) {
    std::vector<Array> hv, cv, Wv, Uv, bv;
    for (int l = 0; l < layers; ++l) {
        hv.push_back(A(h[l]));
        cv.push_back(A(c[l]));
        Wv.push_back(A(W[l]));
        Uv.push_back(A(U[l]));
        bv.push_back(A(b[l]));
    }
    auto r = dali::op::stacked_lstm_sequence(A(xs), hv, cv, Wv, Uv, bv, shortcut != 0);
    for (int l = 0; l < layers; ++l) {
        c_last[l] = wrap(r.memory[l]);
        h_last[l] = wrap(r.hidden[l]);
    }
    *top_states = wrap(r.top_hidden_states);
    return 0;
}
int dali_fe_stacked_lstm_sequence(dali_array_t xs, int layers, const dali_array_t* h, const dali_array_t* c, const dali_array_t* W,
                                  const dali_array_t* U, const dali_array_t* b, int shortcut, dali_array_t* c_last, dali_array_t* h_last,
                                  dali_array_t* top_states) {
    FE_TRY(return stacked_lstm_sequence_impl(xs, layers, h, c, W, U, b, shortcut, c_last, h_last, top_states);, 1)
}
int dali_fe_gru_sequence(dali_array_t xs, dali_array_t h0, dali_array_t W, dali_array_t U, dali_array_t b, dali_array_t* states, dali_array_t* last) {
    FE_TRY(auto r = dali::op::gru_sequence(A(xs), A(h0), A(W), A(U), A(b)); *states = wrap(r.states); *last = wrap(r.last); return 0;, -1)
}

dali_array_t dali_fe_gru_step(dali_array_t x, dali_array_t h, dali_array_t W, dali_array_t U, dali_array_t b) {
    FE_TRY(return wrap(dali::op::gru_step(A(x), A(h), A(W), A(U), A(b)));, nullptr)
}

int dali_fe_eval(dali_array_t a) { FE_TRY(A(a).eval(); return 0;, 1) }
int dali_fe_eval_together(dali_array_t* roots, int n) {
    FE_TRY(std::vector<Array> r; for (int i = 0; i < n; ++i) r.push_back(A(roots[i])); Array::eval_together(r); return 0;, 1)
}
int dali_fe_assign(dali_array_t dest, int operator_t, dali_array_t source) {
    FE_TRY(dali::evaluate_into(A(dest), (dali::OPERATOR_T)operator_t, A(source)); return 0;, 1)
}
int dali_fe_to_host(dali_array_t a, void* out) { FE_TRY(A(a).to_host(out); return 0;, 1) }
void* dali_fe_device_ptr(dali_array_t a) { FE_TRY(return A(a).device_ptr();, nullptr) }

int dali_fe_stats(uint64_t* kernels, uint64_t* gemms, uint64_t* evals, uint64_t* plans) {
    auto& s = dali::jit_stats();
    if (kernels) *kernels = s.kernels_launched;
    if (gemms) *gemms = s.gemms_launched;
    if (evals) *evals = s.evals;
    if (plans) *plans = s.plans_built;
    return 0;
}
int dali_fe_plan_cache_stats(uint64_t* hits, uint64_t* stored) {
    auto& s = dali::jit_stats();
    if (hits) *hits = s.plan_cache_hits;
    if (stored) *stored = s.plan_cache_stored;
    return 0;
}
const char* dali_fe_last_kernel_kinds(void) {
    g_kinds = dali::jit_stats().last_kernel_kinds;
    return g_kinds.c_str();
}
const char* dali_fe_last_kernel_names(void) {
    static thread_local std::string names;
    names = dali::jit_stats().last_kernel_names;
    return names.c_str();
}
const char* dali_fe_last_source(void) { return dali::last_generated_source().c_str(); }

struct Recording {
    std::vector<std::function<void()>> launches;
    std::vector<std::shared_ptr<dali::memory::SynchronizedMemory>> written;
    void* graph = nullptr;  // hipGraphExec_t once instantiated
    // the replayed kernels write device memory behind the front-end's back: host copies become stale
    void invalidate_host_copies() {
        for (auto& m : written) m->mutable_data(dali::memory::DEVICE_T_GPU);
    }
};

void* dali_fe_record_begin(void) {
    auto* rec = new Recording();
    dali::set_recording(&rec->launches, &rec->written);
    return rec;
}
int dali_fe_record_end(void* recording) {
    dali::set_recording(nullptr, nullptr);
    return recording ? (int)((Recording*)recording)->launches.size() : -1;
}
int dali_fe_record_make_graph(void* recording) {
    FE_TRY(auto* rec = (Recording*)recording; if (!rec) throw std::runtime_error("NULL recording");
           if (rec->graph) return 0;
           if (rec->launches.empty()) throw std::runtime_error("recording holds no launches");
           dali::check_hip(dali_hip_capture_begin(), "graph capture begin");
           try { for (auto& f : rec->launches) f(); } catch (...) { void* junk = nullptr; dali_hip_capture_end(&junk); if (junk) dali_hip_graph_destroy(junk); throw; }
           dali::check_hip(dali_hip_capture_end(&rec->graph), "graph capture end");
           return 0;
           , 1)
}
int dali_fe_replay(void* recording, int times) {
    FE_TRY(auto* rec = (Recording*)recording; if (!rec) throw std::runtime_error("NULL recording");
           if (times > 0) rec->invalidate_host_copies();
           if (rec->graph) { for (int t = 0; t < times; ++t) dali::check_hip(dali_hip_graph_launch(rec->graph), "graph launch"); return 0; }
           for (int t = 0; t < times; ++t) for (auto& f : rec->launches) f(); return 0;
           , 1)
}
void dali_fe_record_free(void* recording) {
    auto* rec = (Recording*)recording;
    if (rec && rec->graph) dali_hip_graph_destroy(rec->graph);
    delete rec;
}

int dali_fe_set_dry_run(int on, int compile) {
    dali::set_dry_run(on != 0);
    dali::set_dry_compile(on != 0 && compile != 0);
    return 0;
}
int dali_fe_scope_observe(dali_fe_scope_callback on_enter, dali_fe_scope_callback on_exit, void* user) {
    // the depth counts the scopes this observer has seen open, the one reported included
    auto depth = std::make_shared<int>(0);
    dali::Scope::callback_t enter, leave;
    enter = [on_enter, user, depth](dali::Scope::name_t n) {
        ++*depth;
        if (on_enter) on_enter(n->c_str(), *depth, user);
    };
    leave = [on_exit, user, depth](dali::Scope::name_t n) {
        if (on_exit) on_exit(n->c_str(), *depth, user);
        if (*depth > 0) --*depth;
    };
    return dali::Scope::add_observer(enter, leave);
}

void dali_fe_scope_unobserve(int id) { dali::Scope::remove_observer(id); }

// every kernel source of the last dali_fe_generate_only call, in the order of the launches they stand for
static std::vector<std::string> g_generated;
const char* dali_fe_generated_source(int i) { return i >= 0 && i < (int)g_generated.size() ? g_generated[i].c_str() : ""; }

int dali_fe_generate_only(dali_array_t* roots, int n, int compile) {
    dali::set_dry_compile(compile != 0);
    try {
        std::vector<Array> r;
        for (int i = 0; i < n; ++i) r.push_back(A(roots[i]));
        g_generated = dali::generate_only(r);
        dali::set_dry_compile(false);
        return (int)g_generated.size();
    } catch (const std::exception& ex) {
        dali::set_dry_compile(false);
        g_err = ex.what();
        return -1;
    }
}

}  // extern "C"
