"""``op``: the lazy operator factories (``dali/array/op.h`` of the reference)."""
import ctypes as C

from ._native import front, fe_error, DaliError
from .array import Array, as_array, _ints, _wrap, DTYPE_FLOAT, DTYPE_DOUBLE, DTYPE_INT32  # noqa: F401


def elementwise(functor_name, a, b=None):
    a = as_array(a)
    if b is None:
        return _wrap(front.dali_fe_unary(functor_name.encode(), a._h), functor_name)
    b = as_array(b)
    return _wrap(front.dali_fe_binary(functor_name.encode(), a._h, b._h), functor_name)


def _unary(name):
    def f(x):
        return elementwise(name, x)
    f.__name__ = name
    return f


def _binary(name):
    def f(a, b):
        return elementwise(name, a, b)
    f.__name__ = name
    return f


# dali/array/op/unary.h
identity = _unary("identity")
sigmoid = _unary("sigmoid")
tanh = _unary("tanh")
exp = _unary("exp")
log = _unary("log")
softplus = _unary("softplus")
relu = _unary("relu")
abs = _unary("abs")
sign = _unary("sign")
square = _unary("square")
cube = _unary("cube")
sqrt = _unary("sqrt_f")
rsqrt = _unary("rsqrt")
eltinv = _unary("inv")
isnan = _unary("isnotanumber")
isinf = _unary("isinfinity")
dsigmoid = _unary("dsigmoid")
dtanh = _unary("dtanh")
softplus_backward = _unary("softplus_backward")
relu_backward = _unary("relu_backward")
log_or_zero = _unary("log_or_zero")
inverse_tanh = _unary("inverse_tanh")
# dali/array/op/binary.h
add = _binary("add")
subtract = _binary("subtract")
eltmul = _binary("eltmul")
eltdiv = _binary("eltdiv")
pow = _binary("power")
equals = _binary("equals")
prelu = _binary("prelu")
clip = _binary("clip")
clipped_relu = _binary("clipped_relu")
clipped_relu_backward = _binary("clipped_relu_backward")
steep_sigmoid = _binary("steep_sigmoid")
steep_sigmoid_backward = _binary("steep_sigmoid_backward")
prelu_backward_weights = _binary("prelu_backward_weights")
prelu_backward_inputs = _binary("prelu_backward_inputs")
lessthanequal = _binary("lessthanequal")
greaterthanequal = _binary("greaterthanequal")
maximum = _binary("max_scalar")
minimum = _binary("min_scalar")
binary_cross_entropy = _binary("binary_cross_entropy")
binary_cross_entropy_grad = _binary("binary_cross_entropy_grad")


def close(left, right, atolerance):
    """|left - right| <= atolerance, elementwise (dali/array/op/binary.cpp:16-18)."""
    return lessthanequal(abs(subtract(left, right)), atolerance)


def astype(a, dtype):
    a = as_array(a)
    return _wrap(front.dali_fe_astype(a._h, dtype), "astype")


def _reduce(reducer, x, axes, keepdims):
    x = as_array(x)
    if axes is None:
        return _wrap(front.dali_fe_all_reduce(reducer.encode(), x._h), reducer)
    if isinstance(axes, int):
        axes = [axes]
    a, n = _ints(axes)
    return _wrap(front.dali_fe_axis_reduce(reducer.encode(), x._h, a, n, 1 if keepdims else 0), reducer)


def sum(x, axes=None, keepdims=False):
    return _reduce("sum", x, axes, keepdims)


def prod(x, axes=None, keepdims=False):
    return _reduce("product", x, axes, keepdims)


def max(x, axes=None, keepdims=False):
    return _reduce("maximum", x, axes, keepdims)


def min(x, axes=None, keepdims=False):
    return _reduce("minimum", x, axes, keepdims)


def mean(x, axes=None, keepdims=False):
    x = as_array(x)
    if axes is None:
        return _wrap(front.dali_fe_mean_all(x._h), "mean")
    if isinstance(axes, int):
        axes = [axes]
    a, n = _ints(axes)
    return _wrap(front.dali_fe_mean_axes(x._h, a, n, 1 if keepdims else 0), "mean")


def _arg(reducer, x, axis):
    x = as_array(x)
    if axis is None:
        return _wrap(front.dali_fe_arg_all_reduce(reducer.encode(), x._h), "arg " + reducer)
    return _wrap(front.dali_fe_arg_axis_reduce(reducer.encode(), x._h, axis), "arg " + reducer)


def argmax(x, axis=None):
    return _arg("maximum", x, axis)


def argmin(x, axis=None):
    return _arg("minimum", x, axis)


# Converted operands are bound to local names for the duration of each native
# call: a temporary Array would release its handle before the call reads it.
def softmax(x, axis=-1):
    x = as_array(x)
    return _wrap(front.dali_fe_softmax(x._h, axis), "softmax")


def softmax_naive(x, axis=-1):
    """exp(x - max) / sum(exp(x - max)) written out (what ``softmax`` becomes when it is evaluated, except for shapes that
    get their statistics from a pass of their own)."""
    x = as_array(x)
    return _wrap(front.dali_fe_softmax_naive(x._h, axis), "softmax_naive")


def gather(source, indices):
    """source[indices[...], ...]; assigning to the lazy result scatters into ``source``."""
    source, indices = as_array(source), as_array(indices)
    return _wrap(front.dali_fe_gather(source._h, indices._h), "gather")


def gather_from_rows(source, indices):
    source, indices = as_array(source), as_array(indices)
    return _wrap(front.dali_fe_gather_from_rows(source._h, indices._h), "gather_from_rows")


def one_hot(indices, depth, on_value, off_value):
    indices, on_value, off_value = as_array(indices), as_array(on_value), as_array(off_value)
    return _wrap(front.dali_fe_one_hot(indices._h, depth, on_value._h, off_value._h), "one_hot")


def dot(a, b):
    a, b = as_array(a), as_array(b)
    return _wrap(front.dali_fe_dot(a._h, b._h), "dot")


def inner(a, b):
    a, b = as_array(a), as_array(b)
    return _wrap(front.dali_fe_inner(a._h, b._h), "inner")


def matrix_vector_dot(a, b):
    a, b = as_array(a), as_array(b)
    return _wrap(front.dali_fe_matrix_vector_dot(a._h, b._h), "matrix_vector_dot")


def ceil(a):
    """Rounds up to int32 (dali/array/op/elementwise_operation.cpp:155-160)."""
    return _wrap(front.dali_fe_ceil(as_array(a)._h), "ceil")


def softmax_temperature(x, temperature, axis=-1):
    """The reference's softmax_temperature does not read its temperature (dali/array/op/softmax.cpp:10-13); neither does this."""
    return _wrap(front.dali_fe_softmax_temperature(as_array(x)._h, as_array(temperature)._h, axis), "softmax_temperature")


def top_k(a, k, sorted=True):
    """int32 positions of the k largest entries along the last axis, largest first, lower position first among equals
    (dali/array/op/top_k.cpp:198-208)."""
    return _wrap(front.dali_fe_top_k(as_array(a)._h, k, 1 if sorted else 0, 1), "top_k")


def bottom_k(a, k, sorted=True):
    """int32 positions of the k smallest entries along the last axis, smallest first (dali/array/op/top_k.cpp:210-220)."""
    return _wrap(front.dali_fe_top_k(as_array(a)._h, k, 1 if sorted else 0, 0), "bottom_k")


def argsort(a, axis=None):
    """Stable ascending order of the flattened array, or along ``axis`` (dali/array/op/top_k.cpp:222-233)."""
    if axis is None:
        return _wrap(front.dali_fe_argsort(as_array(a)._h, 0, 1), "argsort")
    return _wrap(front.dali_fe_argsort(as_array(a)._h, axis, 0), "argsort")


def tensordot(a, b, axes):
    """``axes`` = a count (the last axes of a against the first of b) or a pair of axis lists (dali/array/op/dot.cpp:92-98)."""
    a, b = as_array(a), as_array(b)
    if isinstance(axes, int):
        return _wrap(front.dali_fe_tensordot(a._h, b._h, axes, None, None), "tensordot")
    a_axes, b_axes = axes
    if len(a_axes) != len(b_axes):
        raise DaliError("tensordot_as_dot must have as many reduction axes for a than b")
    pa, n = _ints(a_axes)
    pb, _ = _ints(b_axes)
    return _wrap(front.dali_fe_tensordot(a._h, b._h, n, pa, pb), "tensordot")


def softmax_cross_entropy(logits, targets):
    """(mean loss, per-row loss, gradient) of the LSE-form softmax cross-entropy, evaluated together."""
    outs = [C.c_void_p() for _ in range(3)]
    logits, targets = as_array(logits), as_array(targets)
    if front.dali_fe_softmax_cross_entropy(logits._h, targets._h, *[C.byref(o) for o in outs]) != 0:
        raise fe_error("softmax_cross_entropy")
    return tuple(Array(o.value) for o in outs)


def lstm_step(x, h, c, W, U, b):
    """One LSTM cell step; returns (c', h') already evaluated."""
    outs = [C.c_void_p() for _ in range(2)]
    keep = [as_array(v) for v in (x, h, c, W, U, b)]
    if front.dali_fe_lstm_step(*[k._h for k in keep], *[C.byref(o) for o in outs]) != 0:
        raise fe_error("lstm_step")
    return tuple(Array(o.value) for o in outs)


def lstm_sequence(xs, h0, c0, W, U, b):
    """The LSTM step along xs[T, B, I]; returns (hidden_states [T, B, H], final memory, final hidden), evaluated."""
    outs = [C.c_void_p() for _ in range(3)]
    keep = [as_array(v) for v in (xs, h0, c0, W, U, b)]
    if front.dali_fe_lstm_sequence(*[k._h for k in keep], *[C.byref(o) for o in outs]) != 0:
        raise fe_error("lstm_sequence")
    return tuple(Array(o.value) for o in outs)


def stacked_lstm_step(x, h, c, W, U, b, shortcut=False):
    """One step of a stack of LSTM cells (dali/layers/stacked_lstm.cpp:219-283, no dropout); h, c, W, U, b are lists with
    one entry per layer. Returns (list of c', list of h'), evaluated."""
    layers = len(W)
    xa = as_array(x)
    groups = [[as_array(v) for v in g] for g in (h, c, W, U, b)]
    if any(len(g) != layers for g in groups[2:]):
        raise ValueError("stacked_lstm_step: every layer needs its W, U and b")
    if len(groups[0]) != layers or len(groups[1]) != layers:
        states = len(groups[0]) if len(groups[0]) != layers else len(groups[1])  # (min / max in this module are the reductions)
        raise DaliError("Activating LSTM stack of size %d with different number of states %d" % (layers, states))
    handles = [(C.c_void_p * layers)(*[k._h for k in g]) for g in groups]
    c_new, h_new = (C.c_void_p * layers)(), (C.c_void_p * layers)()
    if front.dali_fe_stacked_lstm_step(xa._h, layers, *handles, 1 if shortcut else 0, c_new, h_new) != 0:
        raise fe_error("stacked_lstm_step")
    return [Array(v) for v in c_new], [Array(v) for v in h_new]


def stacked_lstm_sequence(xs, h, c, W, U, b, shortcut=False):
    """The stack of LSTM layers along xs [T, B, I] (AbstractStackedLSTM::activate_sequence): h, c, W, U, b are lists with
    one entry per layer. Returns (list of final c, list of final h, hidden states [T, B, H] of the top layer), evaluated."""
    layers = len(W)
    xa = as_array(xs)
    groups = [[as_array(v) for v in g] for g in (h, c, W, U, b)]
    if any(len(g) != layers for g in groups[2:]) or layers < 1:
        raise ValueError("stacked_lstm_sequence: every layer needs its W, U and b")
    if len(groups[0]) != layers or len(groups[1]) != layers:
        states = len(groups[0]) if len(groups[0]) != layers else len(groups[1])
        raise DaliError("Activating LSTM stack of size %d with different number of states %d" % (layers, states))
    handles = [(C.c_void_p * layers)(*[k._h for k in g]) for g in groups]
    c_last, h_last, top = (C.c_void_p * layers)(), (C.c_void_p * layers)(), C.c_void_p()
    if front.dali_fe_stacked_lstm_sequence(xa._h, layers, *handles, 1 if shortcut else 0, c_last, h_last, C.byref(top)) != 0:
        raise fe_error("stacked_lstm_sequence")
    return [Array(v) for v in c_last], [Array(v) for v in h_last], Array(top.value)


def gru_sequence(xs, h0, W, U, b):
    """The GRU step along xs [T, B, I] from the state h0 (GRU::activate_sequence): (states [T, B, H], last state)."""
    keep = [as_array(v) for v in (xs, h0, W, U, b)]
    outs = [C.c_void_p(), C.c_void_p()]
    if front.dali_fe_gru_sequence(*[k._h for k in keep], *[C.byref(o) for o in outs]) != 0:
        raise fe_error("gru_sequence")
    return Array(outs[0].value), Array(outs[1].value)


def gru_step(x, h, W, U, b):
    """One GRU step; reset / update / candidate layers packed along the columns of W[I,3H], U[H,3H], b[3H]."""
    keep = [as_array(v) for v in (x, h, W, U, b)]
    return _wrap(front.dali_fe_gru_step(*[k._h for k in keep]), "gru_step")


# dali/array/op/reducers.cpp:61-72, binary.cpp:7-12
def any_isnan(x, axes=None, keepdims=False):
    return max(isnan(x), axes, keepdims)


def any_isinf(x, axes=None, keepdims=False):
    return max(isinf(x), axes, keepdims)


def all_equals(left, right):
    return prod(equals(left, right))


def all_close(left, right, atolerance):
    return prod(close(left, right, atolerance))


# dali/array/op/scan.h, arange.h, eye.h, outer.h
def axis_scan(a, reducer, inclusive=True):
    a = as_array(a)
    return _wrap(front.dali_fe_axis_scan(a._h, reducer.encode(), 1 if inclusive else 0), "axis_scan")


def cumsum(a, inclusive=True):
    return axis_scan(a, "reducers::sum", inclusive)


def cumprod(a, inclusive=True):
    return axis_scan(a, "reducers::product", inclusive)


def arange(*args):
    """arange(size), arange(start, stop) or arange(start, stop, step) over python scalars."""
    if len(args) == 1:
        start, stop, step = 0, args[0], 1
    elif len(args) == 2:
        start, stop, step = args[0], args[1], 1
    else:
        start, stop, step = args
    s0, s1, s2 = as_array(start), as_array(stop), as_array(step)
    return _wrap(front.dali_fe_arange(s0._h, s1._h, s2._h), "arange")


def diag(diagonal, rows=None, cols=None):
    d = as_array(diagonal)
    if rows is None:
        rows = d.shape[0]
    if cols is None:
        cols = rows
    return _wrap(front.dali_fe_diag(d._h, int(rows), int(cols)), "diag")


def eye(rows, cols=None):
    return diag(1.0, rows, rows if cols is None else cols)


def outer(a, b):
    a, b = as_array(a), as_array(b)
    return _wrap(front.dali_fe_outer(a._h, b._h), "outer")


def circular_convolution(x, weights):
    """out[..., i] = sum_s x[..., (i + s) mod n] * weights[..., s] (dali/array/op/circular_convolution.cpp)."""
    x, weights = as_array(x), as_array(weights)
    return _wrap(front.dali_fe_circular_convolution(x._h, weights._h), "circular_convolution")


def concatenate(arrays, axis):
    """The arrays one after the other along ``axis`` (dali/array/op/concatenate.cpp:9-73)."""
    keep = [as_array(a) for a in arrays]
    hs = (C.c_void_p * len(keep))(*[k._h for k in keep])
    return _wrap(front.dali_fe_concatenate(hs, len(keep), axis), "concatenate")


def hstack(arrays):
    return concatenate(arrays, -1)


def vstack(arrays):
    return concatenate(arrays, 0)


# dali/array/op/spatial_enums.h
PADDING_T_SAME, PADDING_T_VALID = 0, 1
POOLING_T_MAX, POOLING_T_AVG = 0, 1


def _padding(p):
    return {"same": PADDING_T_SAME, "valid": PADDING_T_VALID}.get(p.lower(), None) if isinstance(p, str) else int(p)


def _pooling(p):
    return {"max": POOLING_T_MAX, "avg": POOLING_T_AVG}.get(p.lower(), None) if isinstance(p, str) else int(p)


def im2col(image, filter_h, filter_w, stride_h, stride_w, padding_h=0, padding_w=0, postpad_h=0, postpad_w=0, data_format="NCHW"):
    """Patch matrix [filter_h*filter_w*C, N*out_h*out_w] of a 3-D or 4-D image (dali/array/op/im2col.cpp:190-267)."""
    image = as_array(image)
    return _wrap(front.dali_fe_im2col(image._h, filter_h, filter_w, stride_h, stride_w, padding_h, padding_w, postpad_h, postpad_w,
                                      data_format.encode()), "im2col")


def col2im(patches, image_shape, filter_h, filter_w, stride_h, stride_w, data_format="NCHW"):
    """The adjoint of im2col: sums the patch matrix back into an image of ``image_shape`` (dali/array/op/col2im.cpp:165-233)."""
    patches = as_array(patches)
    s, n = _ints(image_shape)
    return _wrap(front.dali_fe_col2im(patches._h, s, n, filter_h, filter_w, stride_h, stride_w, data_format.encode()), "col2im")


def conv2d(x, filters, stride_h=1, stride_w=1, padding="valid", data_format="NCHW"):
    x, filters = as_array(x), as_array(filters)
    return _wrap(front.dali_fe_conv2d(x._h, filters._h, stride_h, stride_w, _padding(padding), data_format.encode()), "conv2d")


def conv2d_backward_input(filters, out_dw, stride_h, stride_w, input_shape, padding="valid", data_format="NCHW"):
    filters, out_dw = as_array(filters), as_array(out_dw)
    s, n = _ints(input_shape)
    if n != 4:
        raise ValueError("conv2d_backward_input's result shape must be of size 4")
    return _wrap(front.dali_fe_conv2d_backward_input(filters._h, out_dw._h, stride_h, stride_w, s, _padding(padding), data_format.encode()),
                 "conv2d_backward_input")


def conv2d_backward_filters(x, out_dw, stride_h, stride_w, filters_shape, padding="valid", data_format="NCHW"):
    x, out_dw = as_array(x), as_array(out_dw)
    s, n = _ints(filters_shape)
    if n != 4:
        raise ValueError("conv2d_backward_filters's filters shape must be of size 4")
    return _wrap(front.dali_fe_conv2d_backward_filters(x._h, out_dw._h, stride_h, stride_w, s, _padding(padding), data_format.encode()),
                 "conv2d_backward_filters")


def conv2d_backward_bias(out_dw, data_format="NCHW"):
    out_dw = as_array(out_dw)
    return _wrap(front.dali_fe_conv2d_backward_bias(out_dw._h, data_format.encode()), "conv2d_backward_bias")


def pool2d(x, window_h, window_w, stride_h, stride_w, pooling="max", padding="valid", data_format="NCHW"):
    x = as_array(x)
    return _wrap(front.dali_fe_pool2d(x._h, window_h, window_w, stride_h, stride_w, _pooling(pooling), _padding(padding), data_format.encode()),
                 "pool2d")


def pool2d_backward(y, dy, x, window_h, window_w, stride_h, stride_w, pooling="max", padding="valid", data_format="NCHW"):
    y, dy, x = as_array(y), as_array(dy), as_array(x)
    return _wrap(front.dali_fe_pool2d_backward(y._h, dy._h, x._h, window_h, window_w, stride_h, stride_w, _pooling(pooling), _padding(padding),
                                               data_format.encode()), "pool2d_backward")
