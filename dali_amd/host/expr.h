// Expression nodes of the lazy graph (internal to the front-end).
#ifndef DALI_AMD_HOST_EXPR_H
#define DALI_AMD_HOST_EXPR_H

#include <sstream>

#include "dali.h"

namespace dali {

enum class Kind {
    BUFFER,            // dali/array/expression/buffer.h
    SCALAR,            // dali/array/jit/scalar_view.cpp:15-71
    ELEMENTWISE,       // dali/array/op/elementwise_operation.cpp:35-124
    AXIS_REDUCE,       // dali/array/op/reducer_operation.cpp:98-156 (reduces the LAST axis)
    ALL_REDUCE,        // dali/array/op/reducer_operation.cpp:41-88
    ARG_AXIS_REDUCE,   // dali/array/op/reducer_operation.cpp:193-228
    ARG_ALL_REDUCE,    // dali/array/op/reducer_operation.cpp:158-191
    EXPAND_DIMS,       // dali/array/jit/reshape.cpp:156-209
    BROADCAST,         // dali/array/jit/reshape.cpp:62-154 (BroadcastedReshape)
    GATHER_FROM_ROWS,  // dali/array/op/gather_from_rows.cpp:21-127
    GATHER,            // dali/array/op/gather.cpp:31-160 (rows of a 2-D source picked by a 1-D index)
    AXIS_SCAN,         // dali/array/op/scan.cpp:19-194 (name = reducer, depth = 1 when inclusive)
    ARANGE,            // dali/array/op/arange.cpp:8-39 (args: start, step scalars)
    DIAG,              // dali/array/op/eye.cpp:8-44 (args: diagonal vector or scalar)
    CIRCULAR_CONV,     // dali/array/op/circular_convolution.cpp:8-86 (args: content, weights, both of the node's shape)
    IM2COL,            // dali/array/op/im2col.cpp:11-148 (args: image; geom, data_format)
    COL2IM,            // dali/array/op/col2im.cpp:27-162 (args: patch matrix; shape = image shape)
    POOL2D,            // dali/array/op/conv.cpp:12-112 (name = reducer, depth = 1 for the average)
    POOL2D_BACKWARD,   // dali/array/op/conv.cpp:114-212 (args: y, dy, x)
    ONE_HOT,           // dali/array/op/one_hot.cpp:16-74
    MATMUL,            // dali/array/op/dot.cpp:18-47
    SOFTMAX            // dali/array/op/softmax.cpp:5-8 as one node (axis = the normalised axis); written out when evaluated
};

struct Expr {
    Kind kind;
    DType dtype = DTYPE_FLOAT;
    std::vector<int> shape;
    std::vector<Array> args;
    std::string name;  // functor or reducer, e.g. "functor::exp", "reducers::sum"

    // BUFFER
    std::shared_ptr<memory::SynchronizedMemory> memory;
    std::vector<int> strides;  // empty = contiguous row-major
    int offset = 0;            // in elements

    // SCALAR
    double dvalue = 0.0;
    int ivalue = 0;

    // GATHER over a source of more than two dimensions whose trailing axes do not merge into one (a strided view): args[0]
    // is then a dense copy, good for reading; an assignment through the node must reach the view itself, kept here
    std::vector<Array> origin;

    int axis = 0;   // EXPAND_DIMS
    int depth = 0;  // ONE_HOT

    // sliding-window nodes. IM2COL / COL2IM: filter_h, filter_w, stride_h, stride_w, dilate_h, dilate_w, prepad_h,
    // prepad_w, postpad_h, postpad_w; POOL2D / POOL2D_BACKWARD: window_h, window_w, stride_h, stride_w, prepad_h, prepad_w
    std::vector<int> geom;
    std::string data_format;  // a permutation of "NCHW": the order of the image's dimensions

    int numel() const {
        int64_t n = 1;
        for (int s : shape) n *= s;
        return (int)n;
    }
};

struct ArrayState {
    std::shared_ptr<Expr> expr;
};

template <typename... Args>
std::string make_message(const Args&... args) {
    std::ostringstream ss;
    using expander = int[];
    (void)expander{0, ((void)(ss << args), 0)...};
    return ss.str();
}

std::string shape_str(const std::vector<int>& shape);

#define DALI_ASSERT(cond, msg)                         \
    do {                                               \
        if (!(cond)) throw std::runtime_error(msg);    \
    } while (0)

// C-ABI status -> exception
void check_hip(int status, const char* what);

std::vector<int> contiguous_strides(const std::vector<int>& shape);

// evaluation driver (jit.cpp)
void evaluate(const std::vector<Array>& roots);
void evaluate_into(const Array& dest, OPERATOR_T op, const Array& source);
void evaluate_into_together(const std::vector<Array>& dests, const std::vector<Array>& sources);
// Maximum and sum of exp(x - maximum) of every row, evaluated, as [rows, 1], for rows that are few for their length (cut into
// pieces that fill the device); *x comes back as the contiguous buffer they were taken from. False for any other shape.
bool few_long_rows_softmax_statistics(Array* x, Array* maxima, Array* sums);
bool dry_run();
// one fused launch for the LSTM cell step (records itself like any other launch)
void lstm_step_fused(const Array& x, const Array& h, const Array& c, const Array& W, const Array& U, const Array& b, const Array& c_new,
                     const Array& h_new);
void lstm_step_small(const Array& x, const Array& h, const Array& c, const Array& W, const Array& U, const Array& b, const Array& c_new,
                     const Array& h_new);
// the recurrent half of an LSTM over a whole sequence in one launch: pre [T, B, 4H] = x.W + bias for every step
void lstm_recurrent_persistent(const Array& pre, const Array& U, const Array& h0, const Array& c0, const Array& hs, const Array& c_out);
void gru_recurrent_persistent(const Array& pre, const Array& U, const Array& h0, const Array& hs, const Array& scratch);
// softmax of a contiguous fp32 buffer seen as [outer, extent, inner] along `extent`, one pass over memory (records itself like any other launch)
void softmax_axis_launch(const Array& x, const Array& out, long long outer, int extent, long long inner);
// stride-1 convolution of a dense float NHWC image [N,H,W,C] (C a multiple of 4) with filters [O,fh,fw,C], fh <= 8:
// one padding copy and one multi-term product, no patch matrix; returns [N, out_h, out_w, O]
Array conv2d_direct_nhwc(const Array& x, const Array& filters, int pad_top, int pad_left, int pad_bottom, int pad_right);
// column numbers of the k best entries of every row of a [rows, cols] matrix, best first (evaluates its argument)
Array topk_rows(const Array& x2d, int k, bool largest, bool ties_by_descending_column);
void set_dry_run(bool on);
bool dry_run();

}  // namespace dali

#endif
