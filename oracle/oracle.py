"""ctypes loader for the checker libraries (test infrastructure only).

``liboracle.so`` is the CPU restatement (oracle/dali_oracle.c); ``_ref/libdali_ref.so``
is built from the reference's own headers when the reference checkout is present.
Only tests, the smoke check and the benchmark's cpu_baseline leg import this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
SUM, MAX, MIN, PROD = 0, 1, 2, 3

_f = C.POINTER(C.c_float)
_i32 = C.POINTER(C.c_int32)
_i64 = C.c_int64


def build(force=False):
    """Compile the checker libraries (gcc only; no GPU toolchain involved)."""
    so = os.path.join(_HERE, "liboracle.so")
    if force or not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(os.path.join(_HERE, "dali_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "liboracle.so"], stdout=subprocess.DEVNULL)
    ref = os.path.join(_HERE, "_ref", "libdali_ref.so")
    if os.path.isdir("/root/reference") and (force or not os.path.exists(ref)):
        subprocess.check_call(["make", "-C", _HERE, "ref"], stdout=subprocess.DEVNULL)


def _load():
    path = os.path.join(_HERE, "liboracle.so")
    if not os.path.exists(path):
        build()
    lib = C.CDLL(path)
    lib.orc_unary.argtypes = [C.c_char_p, _f, _f, _i64]
    lib.orc_binary.argtypes = [C.c_char_p, _f, _i64, _f, _i64, _f, _i64]
    lib.orc_round_to_int.argtypes = [_f, _i32, _i64]
    lib.orc_chain.argtypes = [_f, _f, _f, _f, _f, _i64]
    lib.orc_axis_reduce.argtypes = [C.c_int, _f, _i64, _i64, _i64, _i64, _f]
    lib.orc_all_reduce.argtypes = [C.c_int, _f, _i64]
    lib.orc_all_reduce.restype = C.c_float
    lib.orc_arg_axis_reduce.argtypes = [C.c_int, _f, _i64, _i64, _i64, _i64, _i32]
    lib.orc_arg_all_reduce.argtypes = [C.c_int, _f, _i64]
    lib.orc_arg_all_reduce.restype = _i64
    lib.orc_mean_all.argtypes = [_f, _i64]
    lib.orc_mean_all.restype = C.c_float
    lib.orc_softmax.argtypes = [_f, _f, _i64, _i64]
    lib.orc_gather_from_rows.argtypes = [_f, _i64, _i32, _i64, _f]
    lib.orc_gather_rows.argtypes = [_f, _i64, _i32, _i64, _f]
    lib.orc_scatter_rows.argtypes = [_f, _i64, _i32, _i64, _f, C.c_int, C.c_int]
    lib.orc_scatter_to_rows.argtypes = [_f, _i64, _i32, _i64, _f, C.c_int, C.c_int]
    lib.orc_axis_scan.argtypes = [C.c_int, _f, _i64, _i64, C.c_int, _f]
    lib.orc_circular_convolution.argtypes = [_f, _f, _i64, _i64, _f]
    lib.orc_one_hot.argtypes = [_i32, _i64, C.c_int, C.c_float, C.c_float, _f]
    _ip = C.POINTER(C.c_int)
    lib.orc_im2col.argtypes = [_f, _ip, C.c_char_p, _ip, _f]
    lib.orc_col2im.argtypes = [_f, _ip, C.c_char_p, _ip, _f]
    lib.orc_pool2d.argtypes = [_f, _ip, C.c_char_p] + [C.c_int] * 9 + [_f]
    lib.orc_pool2d_backward.argtypes = [_f, _f, _f, _ip, C.c_char_p] + [C.c_int] * 9 + [_f]
    lib.orc_softmax_cross_entropy.argtypes = [_f, _i32, _i64, _i64, _f, _f, _f]
    lib.orc_softmax_cross_entropy_via_probs.argtypes = [_f, _i32, _i64, _i64, _f]
    for name in ("orc_gemm_f64acc", "orc_gemm_f32seq"):
        getattr(lib, name).argtypes = [_f, _i64, _i64, _f, _i64, _i64, _f, _i64, C.c_int, C.c_int, C.c_int]
    lib.orc_gemm_i32.argtypes = [_i32, _i64, _i64, _i32, _i64, _i64, _i32, _i64, C.c_int, C.c_int, C.c_int]
    lib.orc_lstm_step.argtypes = [_f, _f, _f, _f, _f, _f, C.c_int, C.c_int, C.c_int, C.c_int, _f, _f, _f]
    return lib


lib = _load()


def _ref_load():
    path = os.path.join(_HERE, "_ref", "libdali_ref.so")
    if not os.path.exists(path):
        return None
    r = C.CDLL(path)
    r.ref_axis_reduce.argtypes = [C.c_int, _f, C.c_int, C.c_int, C.c_int, C.c_int, _f]
    r.ref_arg_axis_reduce.argtypes = [C.c_int, _f, C.c_int, C.c_int, C.c_int, C.c_int, _i32]
    r.ref_all_reduce.argtypes = [C.c_int, _f, C.c_int]
    r.ref_all_reduce.restype = C.c_float
    r.ref_index_to_dim3.argtypes = [C.c_int, _i32, _i32]
    r.ref_indices_to_offset3.argtypes = [_i32, _i32]
    r.ref_indices_to_offset3.restype = C.c_int
    r.ref_gemm_i32.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _i32, C.c_int, _i32, C.c_int, _i32, C.c_int]
    r.ref_gemm_f32.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _f, C.c_int, _f, C.c_int, _f, C.c_int]
    return r


ref = _ref_load()


def fp(a):
    return a.ctypes.data_as(_f)


def ip(a):
    return a.ctypes.data_as(_i32)


def _c32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def unary(name, x):
    x = _c32(x)
    y = np.empty_like(x)
    if lib.orc_unary(name.encode(), fp(x), fp(y), x.size) != 0:
        raise KeyError(name)
    return y


def binary(name, a, b):
    """a, b: same-shape arrays or Python/NumPy scalars (broadcast with stride 0)."""
    a_arr = _c32(a)
    b_arr = _c32(b)
    out_shape = a_arr.shape if a_arr.size >= b_arr.size else b_arr.shape
    n = max(a_arr.size, b_arr.size)
    sa = 0 if a_arr.size == 1 and n > 1 else 1
    sb = 0 if b_arr.size == 1 and n > 1 else 1
    y = np.empty(out_shape, dtype=np.float32)
    if lib.orc_binary(name.encode(), fp(a_arr), sa, fp(b_arr), sb, fp(y), n) != 0:
        raise KeyError(name)
    return y


def round_to_int(x):
    x = _c32(x)
    y = np.empty(x.shape, dtype=np.int32)
    lib.orc_round_to_int(fp(x), ip(y), x.size)
    return y


def chain(a, b, c, d):
    a, b, c, d = map(_c32, (a, b, c, d))
    y = np.empty_like(a)
    lib.orc_chain(fp(a), fp(b), fp(c), fp(d), fp(y), a.size)
    return y


def axis_reduce(reducer, x, axis):
    """Reduce a 2-D array along `axis` (0 walks the transposed strided view, as the reference does)."""
    x = _c32(x)
    rows, cols = x.shape
    if axis in (1, -1):
        out = np.empty(rows, dtype=np.float32)
        lib.orc_axis_reduce(reducer, fp(x), rows, cols, cols, 1, fp(out))
    else:
        out = np.empty(cols, dtype=np.float32)
        lib.orc_axis_reduce(reducer, fp(x), cols, rows, 1, cols, fp(out))
    return out


def all_reduce(reducer, x):
    x = _c32(x)
    return np.float32(lib.orc_all_reduce(reducer, fp(x), x.size))


def arg_axis_reduce(reducer, x, axis):
    x = _c32(x)
    rows, cols = x.shape
    if axis in (1, -1):
        out = np.empty(rows, dtype=np.int32)
        lib.orc_arg_axis_reduce(reducer, fp(x), rows, cols, cols, 1, ip(out))
    else:
        out = np.empty(cols, dtype=np.int32)
        lib.orc_arg_axis_reduce(reducer, fp(x), cols, rows, 1, cols, ip(out))
    return out


def arg_all_reduce(reducer, x):
    x = _c32(x)
    return int(lib.orc_arg_all_reduce(reducer, fp(x), x.size))


def mean_all(x):
    x = _c32(x)
    return np.float32(lib.orc_mean_all(fp(x), x.size))


def softmax(a):
    a = _c32(a)
    rows = int(np.prod(a.shape[:-1])) if a.ndim > 1 else 1
    cols = a.shape[-1]
    out = np.empty_like(a)
    lib.orc_softmax(fp(a), fp(out), rows, cols)
    return out


def gather_from_rows(source, indices):
    source = _c32(source)
    indices = np.ascontiguousarray(indices, dtype=np.int32)
    out = np.empty(indices.shape[0], dtype=np.float32)
    lib.orc_gather_from_rows(fp(source), source.shape[1], ip(indices), indices.shape[0], fp(out))
    return out


def one_hot(indices, depth, on=1.0, off=0.0):
    indices = np.ascontiguousarray(indices, dtype=np.int32)
    out = np.empty(indices.shape + (depth,), dtype=np.float32)
    lib.orc_one_hot(ip(indices), indices.size, depth, on, off, fp(out))
    return out


def softmax_cross_entropy(x, t, want_grad=True):
    x = _c32(x)
    t = np.ascontiguousarray(t, dtype=np.int32)
    rows, cols = x.shape
    loss_rows = np.empty(rows, dtype=np.float32)
    grad = np.empty_like(x) if want_grad else None
    mean = C.c_float()
    lib.orc_softmax_cross_entropy(fp(x), ip(t), rows, cols, fp(loss_rows), fp(grad) if want_grad else None, C.byref(mean))
    return np.float32(mean.value), loss_rows, grad


def softmax_cross_entropy_via_probs(x, t):
    x = _c32(x)
    t = np.ascontiguousarray(t, dtype=np.int32)
    out = np.empty(x.shape[0], dtype=np.float32)
    lib.orc_softmax_cross_entropy_via_probs(fp(x), ip(t), x.shape[0], x.shape[1], fp(out))
    return out


def axis_scan(kind, x, inclusive=True):
    """kind: 'sum' | 'product' | 'maximum' | 'minimum'; scans the last axis."""
    x = _c32(x)
    cols = x.shape[-1] if x.ndim else 1
    rows = x.size // cols if cols else 0
    out_shape = x.shape[:-1] + (cols + (0 if inclusive else 1),) if x.ndim else ((), (2,))[0 if inclusive else 1]
    out = np.empty(out_shape, dtype=np.float32)
    lib.orc_axis_scan({"sum": 0, "product": 1, "maximum": 2, "minimum": 3}[kind], fp(x), rows, cols, 1 if inclusive else 0, fp(out))
    return out


def circular_convolution(content, weights):
    content, weights = np.broadcast_arrays(np.asarray(content, np.float32), np.asarray(weights, np.float32))
    content, weights = _c32(content), _c32(weights)
    n = content.shape[-1]
    out = np.empty_like(content)
    lib.orc_circular_convolution(fp(content), fp(weights), content.size // n, n, fp(out))
    return out


def gather_rows(source, indices):
    source = _c32(source)
    idx = np.ascontiguousarray(indices, dtype=np.int32).ravel()
    cols = source.shape[1]
    out = np.empty((idx.size, cols), dtype=np.float32)
    lib.orc_gather_rows(fp(source), cols, ip(idx), idx.size, fp(out))
    return out


def scatter_rows(dest, indices, values, op=1):
    """dest[indices[i], :] (op)= values[i, :] in input order; returns the updated copy of ``dest``."""
    dest = _c32(dest).copy()
    idx = np.ascontiguousarray(indices, dtype=np.int32).ravel()
    vals = _c32(np.asarray(values, dtype=np.float32))
    scalar = vals.size == 1
    lib.orc_scatter_rows(fp(dest), dest.shape[1], ip(idx), idx.size, fp(vals), 1 if scalar else 0, op)
    return dest


def scatter_to_rows(dest, indices, values, op=1):
    dest = _c32(dest).copy()
    idx = np.ascontiguousarray(indices, dtype=np.int32).ravel()
    vals = _c32(np.asarray(values, dtype=np.float32))
    scalar = vals.size == 1
    lib.orc_scatter_to_rows(fp(dest), dest.shape[1], ip(idx), idx.size, fp(vals), 1 if scalar else 0, op)
    return dest


def _ints(values):
    return (C.c_int * len(values))(*[int(v) for v in values])


def _out_extent(size, pre, post, filt, stride, dilate=1):
    return (size + pre + post - (dilate * (filt - 1) + 1)) // stride + 1


def im2col(image, filter_h, filter_w, stride_h, stride_w, prepad_h=0, prepad_w=0, postpad_h=0, postpad_w=0, data_format="NCHW",
           dilate_h=1, dilate_w=1):
    """Patch matrix [filter_h*filter_w*C, N*out_h*out_w] of a 4-D image laid out as ``data_format`` says."""
    image = _c32(image)
    H, W = image.shape[data_format.index("H")], image.shape[data_format.index("W")]
    Cc, N = image.shape[data_format.index("C")], image.shape[data_format.index("N")]
    o_h = _out_extent(H, prepad_h, postpad_h, filter_h, stride_h, dilate_h)
    o_w = _out_extent(W, prepad_w, postpad_w, filter_w, stride_w, dilate_w)
    out = np.empty((filter_h * filter_w * Cc, N * o_h * o_w), dtype=np.float32)
    geom = _ints([filter_h, filter_w, stride_h, stride_w, dilate_h, dilate_w, prepad_h, prepad_w, postpad_h, postpad_w])
    lib.orc_im2col(fp(image), _ints(image.shape), data_format.encode(), geom, fp(out))
    return out


def col2im(patches, image_shape, filter_h, filter_w, stride_h, stride_w, data_format="NCHW"):
    patches = _c32(patches)
    out = np.empty(tuple(image_shape), dtype=np.float32)
    geom = _ints([filter_h, filter_w, stride_h, stride_w, 1, 1, 0, 0, 0, 0])
    lib.orc_col2im(fp(patches), _ints(image_shape), data_format.encode(), geom, fp(out))
    return out


def sliding_window_info(in_h, in_w, window_h, window_w, stride_h, stride_w, padding):
    """out_h, out_w, padding_h, padding_w, odd_padding_h, odd_padding_w (dali/array/op/spatial_utils.cpp:64-91)."""
    ceil = lambda a, b: (a + b - 1) // b
    if padding == "same":
        out_h, out_w = ceil(in_h, stride_h), ceil(in_w, stride_w)
        pad_h = max(0, (out_h - 1) * stride_h + window_h - in_h)
        pad_w = max(0, (out_w - 1) * stride_w + window_w - in_w)
    else:
        out_h, out_w = ceil(in_h - window_h + 1, stride_h), ceil(in_w - window_w + 1, stride_w)
        pad_h = pad_w = 0
    return out_h, out_w, pad_h // 2, pad_w // 2, pad_h % 2, pad_w % 2


def conv2d(x, filters, stride_h, stride_w, padding="valid", data_format="NCHW", gemm_mode="f64"):
    """im2col followed by one matrix product, laid out as dali/array/op/conv.cpp:223-276 does."""
    x, filters = _c32(x), _c32(filters)
    n_dim, c_dim, h_dim, w_dim = (data_format.index(l) for l in "NCHW")
    fh, fw, oc = filters.shape[h_dim], filters.shape[w_dim], filters.shape[n_dim]
    out_h, out_w, ph, pw, odd_h, odd_w = sliding_window_info(x.shape[h_dim], x.shape[w_dim], fh, fw, stride_h, stride_w, padding)
    patches = im2col(x, fh, fw, stride_h, stride_w, ph, pw, ph + odd_h, pw + odd_w, data_format)
    f2 = np.ascontiguousarray(np.swapaxes(filters, n_dim, 0)).reshape(oc, -1)
    batch = x.shape[n_dim]
    if data_format == "NCHW":
        return np.ascontiguousarray(gemm(f2, patches, gemm_mode).reshape(oc, batch, out_h, out_w).swapaxes(0, 1))
    return gemm(np.ascontiguousarray(patches.T), np.ascontiguousarray(f2.T), gemm_mode).reshape(batch, out_h, out_w, oc)


def pool2d(x, window_h, window_w, stride_h, stride_w, mode="max", padding="valid", data_format="NCHW"):
    x = _c32(x)
    H, W = x.shape[data_format.index("H")], x.shape[data_format.index("W")]
    out_h, out_w, ph, pw, _, _ = sliding_window_info(H, W, window_h, window_w, stride_h, stride_w, padding)
    oshape = list(x.shape)
    oshape[data_format.index("H")], oshape[data_format.index("W")] = out_h, out_w
    out = np.empty(tuple(oshape), dtype=np.float32)
    lib.orc_pool2d(fp(x), _ints(x.shape), data_format.encode(), window_h, window_w, stride_h, stride_w, ph, pw, out_h, out_w,
                   1 if mode == "avg" else 0, fp(out))
    return out


def pool2d_backward(y, dy, x, window_h, window_w, stride_h, stride_w, mode="max", padding="valid", data_format="NCHW"):
    y, dy, x = _c32(y), _c32(dy), _c32(x)
    H, W = x.shape[data_format.index("H")], x.shape[data_format.index("W")]
    out_h, out_w, ph, pw, _, _ = sliding_window_info(H, W, window_h, window_w, stride_h, stride_w, padding)
    dx = np.empty_like(x)
    lib.orc_pool2d_backward(fp(y), fp(dy), fp(x), _ints(x.shape), data_format.encode(), window_h, window_w, stride_h, stride_w, ph, pw,
                            out_h, out_w, 1 if mode == "avg" else 0, fp(dx))
    return dx


def _strides(a):
    return a.strides[0] // a.itemsize, a.strides[1] // a.itemsize


def gemm(A, B, mode="f64"):
    """C = A @ B for 2-D float32 arrays of any (row, col) strides."""
    assert A.dtype == np.float32 and B.dtype == np.float32
    M, K = A.shape
    N = B.shape[1]
    Cm = np.empty((M, N), dtype=np.float32)
    ars, acs = _strides(A)
    brs, bcs = _strides(B)
    fn = lib.orc_gemm_f64acc if mode == "f64" else lib.orc_gemm_f32seq
    fn(A.ctypes.data_as(_f), ars, acs, B.ctypes.data_as(_f), brs, bcs, fp(Cm), N, M, N, K)
    return Cm


def gemm_i32(A, B):
    M, K = A.shape
    N = B.shape[1]
    Cm = np.empty((M, N), dtype=np.int32)
    ars, acs = _strides(A)
    brs, bcs = _strides(B)
    lib.orc_gemm_i32(A.ctypes.data_as(_i32), ars, acs, B.ctypes.data_as(_i32), brs, bcs, ip(Cm), N, M, N, K)
    return Cm


def lstm_step(X, H, Cm, W, U, b, f64_gemm=True):
    X, H, Cm, W, U, b = map(_c32, (X, H, Cm, W, U, b))
    B, I = X.shape
    Hd = H.shape[1]
    gates = np.empty((B, 4 * Hd), dtype=np.float32)
    c_new = np.empty((B, Hd), dtype=np.float32)
    h_new = np.empty((B, Hd), dtype=np.float32)
    lib.orc_lstm_step(fp(X), fp(H), fp(Cm), fp(W), fp(U), fp(b), B, I, Hd, 1 if f64_gemm else 0, fp(gates), fp(c_new), fp(h_new))
    return gates, c_new, h_new


def lstm_sequence(Xs, H0, C0, W, U, b, f64_gemm=True):
    """lstm_step along Xs[T, B, I] (dali/layers/lstm.cpp:294-303): (all hidden states, final memory)."""
    h, c, hs = H0, C0, []
    for t in range(Xs.shape[0]):
        _, c, h = lstm_step(Xs[t], h, c, W, U, b, f64_gemm)
        hs.append(h)
    return np.stack(hs), c


def stacked_lstm_step(X, Hs, Cs, Ws, Us, bs, shortcut=False, f64_gemm=True):
    """forward_LSTMs / shortcut_forward_LSTMs without dropout (dali/layers/stacked_lstm.cpp:219-283): layer l reads
    the new hidden state of layer l-1; a shortcut layer above the first reads [hidden below, X]
    (LSTM::activate_shortcut, dali/layers/lstm.cpp:281-289). Returns (list of c', list of h')."""
    if not (len(Hs) == len(Cs) == len(Ws)):
        raise ValueError("Activating LSTM stack of size %d with different number of states %d" % (len(Ws), min(len(Hs), len(Cs))))
    cs, hs = [], []
    layer_input = np.ascontiguousarray(X, np.float32)
    for l in range(len(Ws)):
        inp = np.concatenate([layer_input, X], 1) if (shortcut and l > 0) else layer_input
        _, c, h = lstm_step(np.ascontiguousarray(inp, np.float32), Hs[l], Cs[l], Ws[l], Us[l], bs[l], f64_gemm)
        cs.append(c)
        hs.append(h)
        layer_input = h
    return cs, hs


def gru_step(X, Hs, W, U, b):
    """dali/layers/gru.cpp:27-44 with the layers packed reset / update / candidate: products accumulated in fp64, the
    gate arithmetic through the checker's functors (sigmoid in double, libm tanhf), every operation rounded to fp32.
    No test of the reference pins GRU values: PARITY UNPINNED beyond the composition of pinned parts."""
    X, Hs, W, U, b = map(_c32, (X, Hs, W, U, b))
    Hn = Hs.shape[1]
    px, ph = gemm(X, W), gemm(Hs, np.ascontiguousarray(U[:, :2 * Hn]))
    f32 = np.float32
    pre = lambda k, rec: ((px[:, k * Hn:(k + 1) * Hn] + rec).astype(f32) + b[k * Hn:(k + 1) * Hn]).astype(f32)
    r = unary("sigmoid", pre(0, ph[:, :Hn]))
    reset_state = (r * Hs).astype(f32)
    pc = gemm(reset_state, np.ascontiguousarray(U[:, 2 * Hn:]))
    z = unary("sigmoid", pre(1, ph[:, Hn:]))
    m = unary("tanh", pre(2, pc))
    one_minus = (np.float32(1.0) - z).astype(f32)
    return ((Hs * one_minus).astype(f32) + (m * z).astype(f32)).astype(f32)


def gru_sequence(Xs, H0, W, U, b):
    """GRU::activate_sequence (dali/layers/gru.cpp:59-64): the step applied to every Xs[t] in turn, the state carried along.
    Returns every state [T, B, H]."""
    h = _c32(H0)
    out = []
    for x in Xs:
        h = gru_step(x, h, W, U, b)
        out.append(h)
    return np.stack(out)


def k_best(x, k, largest):
    """int32 positions of the k best entries along the last axis, best first (dali/array/op/top_k.cpp:96-220).
    k = 1 is argmax / argmin (first position on ties, :205,:217); k = the whole axis is the full sort with runs of equal
    values in ascending position (:139-158); otherwise the heap's comparator decides (:103-135): top_k breaks ties
    towards the lower position, bottom_k towards the HIGHER one. Stable sorts of (value, position) pairs."""
    x = np.asarray(x)
    if x.size == 1:
        return np.zeros(x.shape, np.int32)
    n = x.shape[-1]
    rows = x.reshape(-1, n)
    out = np.empty((rows.shape[0], k), np.int32)
    pos = np.arange(n)
    for r, row in enumerate(rows):
        if largest:
            order = np.lexsort((-pos, row))[::-1]  # value descending, position ascending
        elif k < n and k > 1:
            order = np.lexsort((-pos, row))  # value ascending, position descending
        else:
            order = np.lexsort((pos, row))  # value ascending, position ascending
        out[r] = order[:k]
    return out.reshape(x.shape[:-1] + (k,))


def argsort(x, axis=None):
    """dali/array/op/top_k.cpp:222-233: bottom_k over the whole (flattened, or swapped-to-last) axis."""
    x = np.asarray(x)
    if axis is None:
        return k_best(x.reshape(-1), x.size, False)
    return np.swapaxes(k_best(np.swapaxes(x, axis, -1), x.shape[axis], False), axis, -1)
