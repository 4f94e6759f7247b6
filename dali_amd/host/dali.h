// Host front-end: lazy `Array` expressions and the `op::` factories for the
// JIT-fused path, mirroring the subset of the reference's public API that the
// fused-expression hot path needs (dali/array/array.h:18-230, dali/array/op.h).
// Building an expression computes nothing; `eval()` (or any host read) plans the
// fused subgraph, generates HIP source for it, has libdali_hip compile/cache it
// and launches it through the six-array C ABI.
#ifndef DALI_AMD_HOST_DALI_H
#define DALI_AMD_HOST_DALI_H

#include <cstdint>
#include <functional>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace dali {

// numbering as in dali/array/dtype.h:6-10
enum DType { DTYPE_FLOAT = 0, DTYPE_DOUBLE = 1, DTYPE_INT32 = 2 };
int size_of_dtype(DType dtype);
std::string dtype_to_cpp_name(DType dtype);

// dali/array/expression/operator.h
enum OPERATOR_T {
    OPERATOR_T_EQL = 0,
    OPERATOR_T_ADD = 1,
    OPERATOR_T_SUB = 2,
    OPERATOR_T_MUL = 3,
    OPERATOR_T_DIV = 4
};

namespace memory {
// dali/array/memory/access_modes.h:6-10
enum AM { AM_READONLY = 0, AM_MUTABLE = 1, AM_OVERWRITE = 2 };
enum DeviceT { DEVICE_T_CPU = 0, DEVICE_T_GPU = 1 };

// Host + device copies of one allocation with freshness flags and lazy
// migration on access (dali/array/memory/synchronized_memory.h:35-133).
class SynchronizedMemory {
  public:
    // pinned_host: the host copy lives in page-locked memory, which lets prefetch() migrate without blocking
    explicit SynchronizedMemory(size_t bytes, bool pinned_host = false);
    ~SynchronizedMemory();
    SynchronizedMemory(const SynchronizedMemory&) = delete;
    SynchronizedMemory& operator=(const SynchronizedMemory&) = delete;

    size_t bytes() const { return bytes_; }
    void* data(DeviceT device, AM mode);
    const void* readonly_data(DeviceT device);
    void* mutable_data(DeviceT device);
    void* overwrite_data(DeviceT device);
    bool is_fresh(DeviceT device) const { return device == DEVICE_T_CPU ? host_fresh_ : device_fresh_; }
    bool is_allocated(DeviceT device) const { return device == DEVICE_T_CPU ? host_ != nullptr : device_ != nullptr; }
    void lazy_clear();  // zero on first allocation (dali/array/memory/synchronized_memory.cpp:237-266)
    // Start bringing the other side's fresh copy to `device` without waiting for it. With a pinned host copy the
    // transfer runs beside the compute stream and the next access waits only for this block; otherwise it is the
    // blocking migration of data().
    void prefetch(DeviceT device);

  private:
    void allocate(DeviceT device);
    void move_to(DeviceT device);
    void settle(DeviceT device, bool host_will_write);
    size_t bytes_;
    bool pinned_host_ = false;
    void* to_device_event_ = nullptr;  // an h2d transfer in flight: the compute stream has not been told to wait yet
    void* to_host_event_ = nullptr;    // a d2h transfer in flight
    void* host_ = nullptr;
    void* device_ = nullptr;
    bool host_fresh_ = false, device_fresh_ = false;
    bool clear_on_allocation_ = false;
};
}  // namespace memory

struct Expr;
struct ArrayState;

// dali/array/op/spatial_enums.h
enum PADDING_T { PADDING_T_SAME = 0, PADDING_T_VALID = 1 };
enum POOLING_T { POOLING_T_MAX = 0, POOLING_T_AVG = 1 };

class Array {
  public:
    Array();
    Array(const std::vector<int>& shape, DType dtype = DTYPE_FLOAT);
    Array(double scalar);
    Array(float scalar);
    Array(int scalar);
    explicit Array(std::shared_ptr<Expr> expr);

    static Array zeros(const std::vector<int>& shape, DType dtype = DTYPE_FLOAT);
    static Array ones(const std::vector<int>& shape, DType dtype = DTYPE_FLOAT);
    static Array arange(int n, DType dtype = DTYPE_FLOAT);
    // copies `data` (contiguous, row-major) into a new buffer
    static Array from_host(const void* data, const std::vector<int>& shape, DType dtype);
    // the same with the host copy in pinned memory (needs an initialised device): prefetch_to_device() then returns at once
    static Array from_host_pinned(const void* data, const std::vector<int>& shape, DType dtype);
    void prefetch_to_device() const;
    void prefetch_to_host() const;

    bool is_stateless() const;
    bool is_buffer() const;
    bool is_scalar() const;  // ndim == 0
    const std::vector<int>& shape() const;
    int ndim() const;
    DType dtype() const;
    int number_of_elements() const;
    // empty for a contiguous buffer, as in the reference
    const std::vector<int>& strides() const;
    std::vector<int> normalized_strides() const;
    int offset() const;
    bool contiguous_memory() const;
    std::shared_ptr<Expr> expression() const;

    // views: exact on buffers; a lazy node is evaluated first
    Array transpose() const;
    Array transpose(const std::vector<int>& axes) const;
    Array swapaxes(int a, int b) const;
    Array pluck_axis(int axis, int idx) const;
    Array operator[](int idx) const { return pluck_axis(0, idx); }
    Array slice(int axis, int start, int end, int step = 1) const;
    Array reshape(const std::vector<int>& shape) const;
    Array expand_dims(int axis) const;
    Array squeeze(int axis) const;
    Array insert_broadcast_axis(int axis) const { return expand_dims(axis); }
    Array ascontiguousarray() const;

    // evaluation (dali/array/array.cpp:232-245)
    void eval() const;
    // evaluate several roots over the same index domain in as few kernels as the
    // planner can form (shared subexpressions are computed once)
    static void eval_together(const std::vector<Array>& roots);

    // dst (op)= expression, into this array's existing buffer
    Array& assign(const Array& other);
    Array& operator+=(const Array& other);
    Array& operator-=(const Array& other);
    Array& operator*=(const Array& other);
    Array& operator/=(const Array& other);
    // dst += sum of `other` over the axes where dst has extent 1 (dali/array/array.h, operator<<=)
    Array& operator<<=(const Array& other);
    // rows picked by an int32 index array; assigning to the result scatters into this array
    // (dali/array/array.h:139, dali/array/op/gather.cpp)
    Array operator[](const Array& indices) const;
    Array gather_from_rows(const Array& indices) const;

    // host access: evaluates, migrates and writes the elements row-major
    void to_host(void* out) const;
    double scalar_value() const;  // first element as double

    // device pointer of an evaluated buffer (base + offset applied), for interop
    void* device_ptr(memory::AM mode = memory::AM_READONLY) const;

    // method sugar used by the reference's expressions (dali/array/array.h:196-230)
    Array sum() const;
    Array sum(const std::vector<int>& axes, bool keepdims = false) const;
    Array max() const;
    Array max(const std::vector<int>& axes, bool keepdims = false) const;
    Array min() const;
    Array min(const std::vector<int>& axes, bool keepdims = false) const;
    Array mean() const;
    Array mean(const std::vector<int>& axes, bool keepdims = false) const;
    Array argmax() const;
    Array argmax(int axis) const;
    Array argmin() const;
    Array argmin(int axis) const;
    Array exp() const;
    Array log() const;
    Array tanh() const;
    Array sigmoid() const;
    Array square() const;
    Array dot(const Array& other) const;

    std::shared_ptr<ArrayState> state_;
};

Array operator+(const Array& a, const Array& b);
Array operator-(const Array& a, const Array& b);
Array operator*(const Array& a, const Array& b);
Array operator/(const Array& a, const Array& b);
Array operator-(const Array& a);

namespace op {
// dali/array/op/elementwise_operation.h, unary.h, binary.h
Array elementwise(Array a, const std::string& functor_name);
Array elementwise(Array a, Array b, const std::string& functor_name);
Array astype(Array a, DType dtype);
Array unsafe_cast(Array a, DType dtype);
Array round(Array a);
Array ceil(Array a);
Array add(const Array& a, const Array& b);
Array subtract(const Array& a, const Array& b);
Array eltmul(const Array& a, const Array& b);
Array eltdiv(const Array& a, const Array& b);
Array pow(const Array& a, const Array& b);
Array equals(const Array& a, const Array& b);
Array prelu(const Array& x, const Array& weights);
Array clip(const Array& x, const Array& clipping_value);
Array identity(const Array& x);
Array sigmoid(const Array& x);
Array tanh(const Array& x);
Array exp(const Array& x);
Array log(const Array& x);
Array softplus(const Array& x);
Array relu(const Array& x);
Array abs(const Array& x);
Array sign(const Array& x);
Array square(const Array& x);
Array cube(const Array& x);
Array sqrt(const Array& x);
Array rsqrt(const Array& x);
Array eltinv(const Array& x);
Array negate(const Array& x);
Array isnan(const Array& x);
Array isinf(const Array& x);
Array dsigmoid(const Array& x);
Array dtanh(const Array& x);
Array softplus_backward(const Array& x);
Array relu_backward(const Array& x);
Array log_or_zero(const Array& x);
Array inverse_tanh(const Array& x);
Array clipped_relu(const Array& x, const Array& upper_bound);
Array clipped_relu_backward(const Array& x, const Array& upper_bound);
Array steep_sigmoid(const Array& x, const Array& aggressiveness);
Array steep_sigmoid_backward(const Array& x, const Array& aggressiveness);
Array prelu_backward_weights(const Array& a, const Array& grad);
Array prelu_backward_inputs(const Array& a, const Array& weights);
Array lessthanequal(const Array& a, const Array& b);
Array greaterthanequal(const Array& a, const Array& b);
Array maximum(const Array& a, const Array& b);
Array minimum(const Array& a, const Array& b);
Array binary_cross_entropy(const Array& a, const Array& b);
Array binary_cross_entropy_grad(const Array& a, const Array& b);
Array close(const Array& left, const Array& right, const Array& atolerance);
Array add(const std::vector<Array>& arrays);

// dali/array/op/reducers.h, reducer_operation.h
Array all_reduce(const Array& a, const std::string& reducer_name);
Array axis_reduce(const Array& a, const std::string& reducer_name, const std::vector<int>& axes, bool keepdims);
Array argument_all_reduce(const Array& a, const std::string& reducer_name);
Array argument_axis_reduce(const Array& a, const std::string& reducer_name, int axis);
Array sum(const Array& x);
Array sum(const Array& x, const std::vector<int>& axes, bool keepdims = false);
Array prod(const Array& x);
Array prod(const Array& x, const std::vector<int>& axes, bool keepdims = false);
Array max(const Array& x);
Array max(const Array& x, const std::vector<int>& axes, bool keepdims = false);
Array min(const Array& x);
Array min(const Array& x, const std::vector<int>& axes, bool keepdims = false);
Array mean(const Array& x);
Array mean(const Array& x, const std::vector<int>& axes, bool keepdims = false);
Array L2_norm(const Array& x);
Array L2_norm(const Array& x, const std::vector<int>& axes, bool keepdims = false);
Array argmax(const Array& x);
Array argmax(const Array& x, int axis);
Array argmin(const Array& x);
Array argmin(const Array& x, int axis);
Array any_isnan(const Array& x);
Array any_isinf(const Array& x);
Array any_isnan(const Array& x, const std::vector<int>& axes, bool keepdims = false);
Array any_isinf(const Array& x, const std::vector<int>& axes, bool keepdims = false);
Array all_equals(const Array& left, const Array& right);
Array all_close(const Array& left, const Array& right, const Array& atolerance);

// dali/array/op/softmax.h, gather_from_rows.h, one_hot.h, dot.h
Array softmax(const Array& logits, int axis = -1);
// the written-out expression of dali/array/op/softmax.cpp:5-8 (what op::softmax becomes when it is evaluated)
Array softmax_naive(const Array& logits, int axis = -1);
Array softmax_temperature(const Array& logits, const Array& temperature, int axis = -1);
Array gather_from_rows(const Array& source, const Array& indices);
Array gather(const Array& source, const Array& indices);
// dali/array/op/scan.h, arange.h, eye.h, outer.h
Array axis_scan(const Array& a, const std::string& reducer_name, bool inclusive = true);
Array cumsum(const Array& a, bool inclusive = true);
Array cumprod(const Array& a, bool inclusive = true);
Array arange(int size);
Array arange(int start, int stop);
Array arange(const Array& start, const Array& stop, const Array& step);
Array eye(int size);
Array eye(int rows, int cols);
Array diag(const Array& diagonal);
Array diag(const Array& diagonal, int rows);
Array diag(const Array& diagonal, int rows, int cols);
Array outer(const Array& a, const Array& b);
// dali/array/op/circular_convolution.h
Array circular_convolution(Array x, Array weights);

// dali/array/op/concatenate.h
Array concatenate(const std::vector<Array>& arrays, int axis);
Array hstack(const std::vector<Array>& arrays);
Array vstack(const std::vector<Array>& arrays);

// dali/array/op/spatial_utils.h: geometry of sliding-window operators
void check_data_format(const std::string& data_format, int* n_dim, int* c_dim, int* h_dim, int* w_dim);
struct SlidingWindowFunctionInfo {
    int out_w, out_h, batch_size, in_channels, in_h, in_w;
    int padding_h, padding_w, odd_padding_h, odd_padding_w, stride_h, stride_w;
};
struct PoolFunctionInfo : SlidingWindowFunctionInfo {
    int window_h, window_w;
};
struct ConvFunctionInfo : SlidingWindowFunctionInfo {
    int filter_h, filter_w, out_channels;
};
PoolFunctionInfo compute_pool_info(const std::vector<int>& input_shape, int window_h, int window_w, int stride_h, int stride_w,
                                   PADDING_T padding, const std::string& data_format);
ConvFunctionInfo compute_conv2d_info(const std::vector<int>& input_shape, const std::vector<int>& filters_shape, int stride_h,
                                     int stride_w, PADDING_T padding, const std::string& data_format);
// dali/array/op/im2col.h, col2im.h: the patch matrix [filter_h * filter_w * C, N * out_h * out_w] of an image whose
// dimensions come in the order of the letters of data_format, and its adjoint
std::vector<int> im2col_shape(const std::vector<int>& src_shape, int filter_h, int filter_w, int stride_h, int stride_w, int dilate_h,
                              int dilate_w, int prepad_h, int prepad_w, int postpad_h, int postpad_w, const std::string& data_format);
Array im2col(const Array& image, int filter_h, int filter_w, int stride_h, int stride_w, int padding_h, int padding_w, int postpad_h,
             int postpad_w, const std::string& data_format);
Array col2im(const Array& input, const std::vector<int>& image_shape, int filter_h, int filter_w, int stride_h, int stride_w,
             const std::string& data_format);
// dali/array/op/conv.h: convolution as im2col + one matrix product, and pooling
Array conv2d(const Array& input, const Array& filters, int stride_h, int stride_w, PADDING_T padding, const std::string& data_format);
Array conv2d_backward_input(Array filters, Array out_dw, int stride_h, int stride_w, const std::vector<int>& input_shape,
                            PADDING_T padding, const std::string& data_format);
Array conv2d_backward_filters(Array input, Array out_dw, int stride_h, int stride_w, const std::vector<int>& filters_shape,
                              PADDING_T padding, const std::string& data_format);
Array conv2d_backward_bias(Array out_dw, const std::string& data_format);
Array pool2d(const Array& input, int window_h, int window_w, int stride_h, int stride_w, POOLING_T pooling_mode, PADDING_T padding,
             const std::string& data_format);
Array pool2d_backward(const Array& out, const Array& out_dw, const Array& in, int window_h, int window_w, int stride_h, int stride_w,
                      POOLING_T pooling_mode, PADDING_T padding, const std::string& data_format);
Array& autoreduce_assign(Array& left, const Array& right);
Array one_hot(Array indices, int depth, Array on_value, Array off_value);
Array matmul(Array a, Array b);
Array dot(const Array& a, const Array& b);
Array inner(const Array& a, const Array& b);
Array top_k(const Array& array, int k, bool sorted = true);
Array bottom_k(const Array& array, int k, bool sorted = true);
Array argsort(const Array& array);
Array argsort(const Array& array, int axis);
Array matrix_vector_dot(const Array& a, const Array& b);
Array tensordot(const Array& a, const Array& b, int axis);
Array tensordot(const Array& a, const Array& b, const std::vector<int>& a_reduce_axes, const std::vector<int>& b_reduce_axes);

// Softmax cross-entropy with integer targets in log-sum-exp form
// (definition: dali/tensor/op/cost.cpp:115-133). Returns {mean loss (scalar),
// per-row loss [N], gradient [N, V] = softmax - one_hot}; the three are evaluated
// together so the logits are read once.
struct CrossEntropyResult {
    Array mean_loss, row_loss, grad;
};
CrossEntropyResult softmax_cross_entropy(const Array& logits, const Array& targets);

// One LSTM cell step with the four gates packed i, f, o, g along the columns of
// W[I,4H], U[H,4H], b[4H] (definition: dali/layers/lstm.cpp:226-261 with
// StackedInputLayer::activate, dali/layers/layers.cpp:159-161). Returns {c', h'},
// already evaluated: one accumulating GEMM pair plus one fused gate kernel.
struct LSTMState {
    Array memory, hidden;
};
LSTMState lstm_step(const Array& x, const Array& h, const Array& c, const Array& W, const Array& U,
                    const Array& b);
// The step along a sequence xs[T, B, I] (dali/layers/lstm.cpp:294-303): all hidden states [T, B, H], the final
// cell state and the final hidden state (a view of the last slice).
struct LSTMSequence {
    Array hidden_states, memory, hidden;
};
LSTMSequence lstm_sequence(const Array& xs, const Array& h0, const Array& c0, const Array& W, const Array& U, const Array& b);
// One step of a stack of LSTM cells (dali/layers/stacked_lstm.cpp:219-283, forward_LSTMs and shortcut_forward_LSTMs
// without dropout): layer l reads the new hidden state of layer l-1, the first layer reads x. With `shortcut` every
// layer above the first also reads x; its W[l] is then [H(l-1) + I, 4 H(l)], the rows for the hidden state below
// first, the rows for x after them (the order LSTM::activate_shortcut passes its inputs, dali/layers/lstm.cpp:281-289).
struct StackedLSTMState {
    std::vector<Array> memory, hidden;
};
StackedLSTMState stacked_lstm_step(const Array& x, const std::vector<Array>& h, const std::vector<Array>& c, const std::vector<Array>& W,
                                   const std::vector<Array>& U, const std::vector<Array>& b, bool shortcut);
// The stack along a whole sequence xs [T, B, I] (AbstractStackedLSTM::activate_sequence, dali/layers/stacked_lstm.cpp:44-51,
// which returns the final state of every layer): final memory and hidden state per layer and the hidden states of the top
// layer [T, B, H], already evaluated. Layer by layer, each over the whole sequence.
struct StackedLSTMSequence {
    std::vector<Array> memory, hidden;
    Array top_hidden_states;
};
StackedLSTMSequence stacked_lstm_sequence(const Array& xs, const std::vector<Array>& h, const std::vector<Array>& c, const std::vector<Array>& W,
                                          const std::vector<Array>& U, const std::vector<Array>& b, bool shortcut);
// One GRU step with reset, update and candidate layers packed along the columns of W[I,3H], U[H,3H], b[3H]
// (dali/layers/gru.cpp:27-44). Returns h', already evaluated.
Array gru_step(const Array& x, const Array& h, const Array& W, const Array& U, const Array& b);
// The step along a whole sequence xs [T, B, I] from the state h0 (GRU::activate_sequence, dali/layers/gru.cpp:59-64, which
// returns the last state): every state [T, B, H] and the last one (a view of it), already evaluated.
struct GRUSequence {
    Array states, last;
};
GRUSequence gru_sequence(const Array& xs, const Array& h0, const Array& W, const Array& U, const Array& b);
}  // namespace op

// Named scopes (dali/utils/scope.h:11-34): DALI_SCOPE(name) opens a scope that lasts to the end of the block when
// somebody observes and costs one test otherwise. The front-end opens "JIT[<kernel shape>:<entry point>]" around every
// generated kernel it launches (the name dali/array/expression/computation.cpp:19 gives a computation), inside it
// "get_function" when the kernel is not loaded yet and, inside that, "compilation" around the call that builds it from
// source unless the code-object cache on disk holds it (dali/array/jit/jit.cpp:1015,1025), and "gemm" around a product.
struct Scope {
    typedef std::shared_ptr<std::string> name_t;
    typedef std::function<void(name_t)> callback_t;
    static bool has_observers();
    // returns the handle remove_observer takes; either callback may be empty
    static int add_observer(callback_t on_enter, callback_t on_exit);
    static void remove_observer(int id);
    name_t name;
    explicit Scope(name_t name_);
    ~Scope();
    Scope(const Scope&) = delete;
    Scope& operator=(const Scope&) = delete;
};
#define DALI_SCOPE(str)                                                              \
    std::unique_ptr<::dali::Scope> dali_scope_guard;                                 \
    if (::dali::Scope::has_observers()) dali_scope_guard.reset(new ::dali::Scope(std::make_shared<std::string>(str)))

// Keeps the stack of open scopes and hands it to two callbacks (dali/utils/scope.h:37-63); observes for as long as it lives.
struct ScopeObserver {
    struct State {
        std::vector<Scope::name_t> trace;  // outermost first; on_exit sees the scope that is being left as the last entry
    };
    typedef std::function<void(const State&)> callback_t;
    ScopeObserver(callback_t on_enter_, callback_t on_exit_);
    ~ScopeObserver();
    ScopeObserver(const ScopeObserver&) = delete;
    ScopeObserver& operator=(const ScopeObserver&) = delete;
  private:
    callback_t on_enter, on_exit;
    State state;
    int id;
};

// Counts of executed computations, used by tests to assert laziness and fusion.
struct JitStats {
    uint64_t kernels_launched = 0;  // generated kernels
    uint64_t gemms_launched = 0;
    uint64_t evals = 0;
    uint64_t plans_built = 0;       // planner invocations that had to generate source
    uint64_t plan_cache_hits = 0;   // evaluations that reused a stored plan instead of planning
    uint64_t plan_cache_stored = 0; // plans stored so far
    std::string last_kernel_kinds;  // e.g. "row" or "row,all" for the last eval
    std::string last_kernel_names;  // entry-point names of the generated kernels of the last eval
};
JitStats& jit_stats();
// HIP source of the kernels generated for the last eval (concatenated)
const std::string& last_generated_source();

// Plan + generate the HIP source for `roots` without touching a device; returns
// the sources of the kernels the planner would launch. Used to check code
// generation on machines without a GPU.
std::vector<std::string> generate_only(const std::vector<Array>& roots);

}  // namespace dali

#endif
