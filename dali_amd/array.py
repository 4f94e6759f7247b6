"""``Array``: Python handle on a lazy front-end array (``dali::Array``)."""
import ctypes as C

import numpy as np

from ._native import front, fe_error

DTYPE_FLOAT, DTYPE_DOUBLE, DTYPE_INT32 = 0, 1, 2
_NP = {DTYPE_FLOAT: np.float32, DTYPE_DOUBLE: np.float64, DTYPE_INT32: np.int32}
_FROM_NP = {np.dtype(np.float32): DTYPE_FLOAT, np.dtype(np.float64): DTYPE_DOUBLE, np.dtype(np.int32): DTYPE_INT32}


def _ints(seq):
    seq = [int(v) for v in seq]
    return (C.c_int * max(1, len(seq)))(*seq), len(seq)


def _wrap(handle, what):
    if not handle:
        raise fe_error(what)
    return Array(handle)


def as_array(x):
    """Array, numpy array or Python scalar -> Array (scalars become literals)."""
    if isinstance(x, Array):
        return x
    if isinstance(x, (bool, int, np.integer)):
        return _wrap(front.dali_fe_scalar_int(int(x)), "scalar")
    if isinstance(x, np.float32):
        return _wrap(front.dali_fe_scalar_float(float(x)), "scalar")
    if isinstance(x, (float, np.floating)):
        return _wrap(front.dali_fe_scalar_double(float(x)), "scalar")
    return Array.from_numpy(np.asarray(x))


class Array(object):
    __array_priority__ = 100

    def __init__(self, handle):
        self._h = handle

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h and front is not None:
            front.dali_fe_release(h)

    # ---- construction
    @staticmethod
    def from_numpy(a, pinned=False):
        """Copy ``a`` into a new buffer. ``pinned=True`` keeps the host copy in page-locked memory (needs an initialised
        device), so that ``prefetch("gpu")`` / ``prefetch("cpu")`` migrate it without blocking."""
        a = np.ascontiguousarray(a)
        if a.dtype not in _FROM_NP:
            raise TypeError("dtype %s is not one of float32, float64, int32" % a.dtype)
        shape, nd = _ints(a.shape)
        make = front.dali_fe_from_host_pinned if pinned else front.dali_fe_from_host
        return _wrap(make(a.ctypes.data_as(C.c_void_p), shape, nd, _FROM_NP[a.dtype]), "from_numpy")

    def prefetch(self, device="gpu"):
        """Start migrating the buffer's fresh copy to ``device`` ("gpu" or "cpu"); blocking unless the host copy is pinned."""
        if front.dali_fe_prefetch(self._h, 1 if device == "gpu" else 0) != 0:
            raise fe_error("prefetch")
        return self

    @staticmethod
    def empty(shape, dtype=DTYPE_FLOAT):
        s, nd = _ints(shape)
        return _wrap(front.dali_fe_empty(s, nd, dtype), "empty")

    @staticmethod
    def zeros(shape, dtype=DTYPE_FLOAT):
        s, nd = _ints(shape)
        return _wrap(front.dali_fe_zeros(s, nd, dtype), "zeros")

    # ---- inspection
    @property
    def ndim(self):
        return front.dali_fe_ndim(self._h)

    @property
    def shape(self):
        nd = self.ndim
        out = (C.c_int * max(1, nd))()
        front.dali_fe_shape(self._h, out)
        return tuple(out[i] for i in range(nd))

    @property
    def dtype(self):
        return front.dali_fe_dtype(self._h)

    @property
    def strides(self):
        nd = self.ndim
        out = (C.c_int * max(1, nd))()
        front.dali_fe_strides(self._h, out)
        return tuple(out[i] for i in range(nd))

    @property
    def offset(self):
        return front.dali_fe_offset(self._h)

    def is_buffer(self):
        return bool(front.dali_fe_is_buffer(self._h))

    def contiguous_memory(self):
        return bool(front.dali_fe_is_contiguous(self._h))

    # ---- views
    def transpose(self, *axes):
        if len(axes) == 1 and isinstance(axes[0], (tuple, list)):
            axes = axes[0]
        a, n = _ints(axes)
        return _wrap(front.dali_fe_transpose(self._h, a, n), "transpose")

    @property
    def T(self):
        return self.transpose()

    def pluck_axis(self, axis, idx):
        return _wrap(front.dali_fe_pluck_axis(self._h, axis, idx), "pluck_axis")

    def slice(self, axis, start, end, step=1):
        return _wrap(front.dali_fe_slice(self._h, axis, start, end, step), "slice")

    def reshape(self, *shape):
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = shape[0]
        s, nd = _ints(shape)
        return _wrap(front.dali_fe_reshape(self._h, s, nd), "reshape")

    def expand_dims(self, axis):
        return _wrap(front.dali_fe_expand_dims(self._h, axis), "expand_dims")

    def squeeze(self, axis):
        return _wrap(front.dali_fe_squeeze(self._h, axis), "squeeze")

    def ascontiguousarray(self):
        return _wrap(front.dali_fe_ascontiguousarray(self._h), "ascontiguousarray")

    def __getitem__(self, key):
        """Integers pluck an axis, slices make strided views (buffers only evaluate lazily built nodes first)."""
        if isinstance(key, Array):
            from . import op
            return op.gather(self, key)
        if not isinstance(key, tuple):
            key = (key,)
        out, axis = self, 0
        for k in key:
            if isinstance(k, (int, np.integer)):
                out = out.pluck_axis(axis, int(k))
            elif isinstance(k, slice):
                n = out.shape[axis]
                start, stop, step = k.indices(n)
                if step < 0:
                    # numpy walks start, start + step, ... down to above stop; the native slice names the same elements by
                    # their range [stop + 1, start + 1) and walks it from its last element (dali/array/slice.cpp:27-37)
                    start, stop = stop + 1, start + 1
                if stop < start:
                    stop = start
                if (start, stop, step) != (0, n, 1):
                    out = out.slice(axis, start, stop, step)
                axis += 1
            elif k is None:
                out = out.expand_dims(axis)
                axis += 1
            else:
                raise IndexError("unsupported index %r" % (k,))
        return out

    # ---- evaluation
    def eval(self):
        if front.dali_fe_eval(self._h) != 0:
            raise fe_error("eval")
        return self

    def numpy(self):
        out = np.empty(self.shape, dtype=_NP[self.dtype])
        if front.dali_fe_to_host(self._h, out.ctypes.data_as(C.c_void_p)) != 0:
            raise fe_error("to_host")
        return out

    def device_ptr(self):
        p = front.dali_fe_device_ptr(self._h)
        if not p:
            raise fe_error("device_ptr")
        return p

    def assign(self, other, operator_t=0):
        other = as_array(other)
        if front.dali_fe_assign(self._h, operator_t, other._h) != 0:
            raise fe_error("assign")
        return self

    def __iadd__(self, other):
        return self.assign(other, 1)

    def __isub__(self, other):
        return self.assign(other, 2)

    def __imul__(self, other):
        return self.assign(other, 3)

    def __itruediv__(self, other):
        return self.assign(other, 4)

    def __ilshift__(self, other):
        """dst <<= src: add the sum of ``src`` over the axes where ``dst`` has extent 1."""
        other = as_array(other)
        if front.dali_fe_autoreduce_assign(self._h, other._h) != 0:
            raise fe_error("autoreduce_assign")
        return self

    def gather_from_rows(self, indices):
        from . import op
        return op.gather_from_rows(self, indices)

    # ---- arithmetic sugar
    def __add__(self, o):
        from . import op
        return op.add(self, o)

    def __radd__(self, o):
        from . import op
        return op.add(o, self)

    def __sub__(self, o):
        from . import op
        return op.subtract(self, o)

    def __rsub__(self, o):
        from . import op
        return op.subtract(o, self)

    def __mul__(self, o):
        from . import op
        return op.eltmul(self, o)

    def __rmul__(self, o):
        from . import op
        return op.eltmul(o, self)

    def __truediv__(self, o):
        from . import op
        return op.eltdiv(self, o)

    def __rtruediv__(self, o):
        from . import op
        return op.eltdiv(o, self)

    def __neg__(self):
        from . import op
        return op.eltmul(-1, self)

    def sum(self, axes=None, keepdims=False):
        from . import op
        return op.sum(self, axes, keepdims)

    def max(self, axes=None, keepdims=False):
        from . import op
        return op.max(self, axes, keepdims)

    def min(self, axes=None, keepdims=False):
        from . import op
        return op.min(self, axes, keepdims)

    def mean(self, axes=None, keepdims=False):
        from . import op
        return op.mean(self, axes, keepdims)

    def argmax(self, axis=None):
        from . import op
        return op.argmax(self, axis)

    def argmin(self, axis=None):
        from . import op
        return op.argmin(self, axis)

    def dot(self, other):
        from . import op
        return op.dot(self, other)


def eval_together(arrays):
    hs = (C.c_void_p * len(arrays))(*[a._h for a in arrays])
    if front.dali_fe_eval_together(hs, len(arrays)) != 0:
        raise fe_error("eval_together")


def jit_stats():
    vals = [C.c_uint64() for _ in range(4)]
    front.dali_fe_stats(*[C.byref(v) for v in vals])
    pc = [C.c_uint64() for _ in range(2)]
    front.dali_fe_plan_cache_stats(*[C.byref(v) for v in pc])
    return {"kernels": vals[0].value, "gemms": vals[1].value, "evals": vals[2].value, "plans": vals[3].value,
            "plan_cache_hits": pc[0].value, "plan_cache_stored": pc[1].value}


def last_kernel_kinds():
    return front.dali_fe_last_kernel_kinds().decode()


def last_kernel_names():
    return front.dali_fe_last_kernel_names().decode()


def last_source():
    return front.dali_fe_last_source().decode()


def generated_source(i):
    """Source of the i-th kernel of the last ``generate_only`` call."""
    return front.dali_fe_generated_source(i).decode()


def generate_only(arrays, compile=False):
    """Plan and generate HIP source for ``arrays`` without touching a device."""
    hs = (C.c_void_p * len(arrays))(*[a._h for a in arrays])
    n = front.dali_fe_generate_only(hs, len(arrays), 1 if compile else 0)
    if n < 0:
        raise fe_error("generate_only")
    return n


_SCOPE_CB = C.CFUNCTYPE(None, C.c_char_p, C.c_int, C.c_void_p)


class ScopeObserver(object):
    """Calls ``on_enter(name, trace)`` / ``on_exit(name, trace)`` for every named scope the front-end opens inside the
    ``with`` block (dali/utils/scope.h: ScopeObserver); ``trace`` lists the open scopes, outermost first, the reported
    one included. ``events`` collects ("enter" | "exit", name, depth) in order."""

    def __init__(self, on_enter=None, on_exit=None):
        self.events, self.trace = [], []
        self._on_enter, self._on_exit, self._id = on_enter, on_exit, 0

        def enter(name, depth, _user):
            name = name.decode()
            self.trace.append(name)
            self.events.append(("enter", name, depth))
            if self._on_enter:
                self._on_enter(name, list(self.trace))

        def leave(name, depth, _user):
            name = name.decode()
            self.events.append(("exit", name, depth))
            if self._on_exit:
                self._on_exit(name, list(self.trace))
            if self.trace and self.trace[-1] == name:
                self.trace.pop()

        self._enter_cb, self._exit_cb = _SCOPE_CB(enter), _SCOPE_CB(leave)  # kept alive as long as the observer

    def __enter__(self):
        self._id = front.dali_fe_scope_observe(C.cast(self._enter_cb, C.c_void_p), C.cast(self._exit_cb, C.c_void_p), None)
        return self

    def __exit__(self, *exc):
        front.dali_fe_scope_unobserve(self._id)
        self._id = 0
        return False


class Recording(object):
    """Stores the launches issued inside the ``with`` block; ``replay(n)`` re-issues them."""

    def __init__(self):
        self._rec = None
        self.launches = 0

    def __enter__(self):
        self._rec = front.dali_fe_record_begin()
        return self

    def __exit__(self, *exc):
        self.launches = front.dali_fe_record_end(self._rec)
        return False

    def make_graph(self):
        """Instantiate a HIP graph of the stored launches; later replays launch the graph."""
        if front.dali_fe_record_make_graph(self._rec) != 0:
            raise fe_error("make_graph")
        return self

    def replay(self, times=1):
        if front.dali_fe_replay(self._rec, times) != 0:
            raise fe_error("replay")

    def __del__(self):
        rec, self._rec = getattr(self, "_rec", None), None
        if rec and front is not None:
            front.dali_fe_record_free(rec)
