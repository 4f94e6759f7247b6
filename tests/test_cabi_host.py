"""CPU-side checks: the C-ABI libraries load and export every declared symbol,
the host front-end's shape/dtype logic and error behaviour, and the planner +
code generator for the five benchmark configurations (generated HIP is compiled
for gfx950 with hipRTC; nothing is launched)."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dali_(?:hip|fe)_[a-z0-9_]+)\s*\(", text)))


def test_hip_library_exports_every_declared_symbol(D):
    from dali_amd._native import hip, HIP_SYMBOLS
    names = declared_functions("dali_hip.h")
    assert len(names) >= 29
    for n in names:
        assert hasattr(hip, n), "libdali_hip.so does not export %s" % n
        assert n in HIP_SYMBOLS, "binding table misses %s" % n


def test_front_library_exports_every_declared_symbol(D):
    from dali_amd._native import front, FRONT_SYMBOLS
    names = declared_functions("dali_front.h")
    assert len(names) >= 45
    for n in names:
        assert hasattr(front, n), "libdali_front.so does not export %s" % n
        assert n in FRONT_SYMBOLS, "binding table misses %s" % n


def test_launch_plan_struct_layout_matches_header(D):
    from dali_amd._native import LaunchPlan
    text = open(os.path.join(ROOT, "include", "dali_hip.h")).read()
    body = re.search(r"typedef struct dali_hip_launch_plan \{(.*?)\} dali_hip_launch_plan;", text, re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = re.findall(r"(?:const\s+)?int32_t\s*\*?\s*([a-z0-9_]+);", body)
    assert fields == [f[0] for f in LaunchPlan._fields_]


def test_compile_only_reports_errors_without_exiting(D):
    from dali_amd._native import hip
    size = C.c_size_t()
    ok = b'extern "C" __global__ void k(float* a) { a[threadIdx.x] = 1.0f; }'
    assert hip.dali_hip_compile_only(ok, C.byref(size)) == 0 and size.value > 0
    bad = b'extern "C" __global__ void k(float* a) { a[0] = functor::nope<float>::Map(1.0f); }'
    assert hip.dali_hip_compile_only(bad, C.byref(size)) != 0
    msg = hip.dali_hip_last_error().decode()
    assert "hipRTC" in msg and "nope" in msg  # the compiler log travels with the error (compiler.h:147-150 keeps only a log path)


# ------------------------------------------------------------ host front-end
def test_lazy_until_evaluated_and_shapes(D, rng):
    op = D.op
    a = D.Array.from_numpy(rng.randn(3, 5).astype(np.float32))
    before = D.jit_stats()
    e = op.exp(a - op.max(a, [-1], True))
    s = e / op.sum(e, [-1], True)
    assert not s.is_buffer() and s.shape == (3, 5) and s.dtype == D.DTYPE_FLOAT
    assert op.sum(a, [0]).shape == (5,) and op.sum(a, [1], True).shape == (3, 1) and op.sum(a).shape == ()
    assert op.argmax(a, 1).dtype == D.DTYPE_INT32 and op.argmax(a, 0).shape == (5,)
    assert op.argmax(a).dtype == D.DTYPE_FLOAT  # flat argmax keeps the input dtype (reducer_operation.cpp:681-684)
    assert op.dot(a, a.T).shape == (3, 3)
    assert op.one_hot(D.Array.from_numpy(np.zeros(4, np.int32)), 7, 1.0, 0.0).shape == (4, 7)
    assert D.jit_stats() == before  # nothing ran


def test_type_promotion_and_errors(D, rng):
    op = D.op
    f = D.Array.from_numpy(rng.randn(2, 3).astype(np.float32))
    i = D.Array.from_numpy(np.arange(6, dtype=np.int32).reshape(2, 3))
    d = D.Array.from_numpy(rng.randn(2, 3))
    assert (f + i).dtype == D.DTYPE_FLOAT and (f + d).dtype == D.DTYPE_DOUBLE and (i + i).dtype == D.DTYPE_INT32
    assert (i * 2.5).dtype == D.DTYPE_INT32  # array (op) scalar keeps the array dtype (array.cpp:845-865)
    assert op.mean(i).dtype == D.DTYPE_DOUBLE  # reducers.cpp:32-36
    with pytest.raises(D.DaliError, match="same rank"):
        f + D.Array.from_numpy(rng.randn(3).astype(np.float32))
    with pytest.raises(D.DaliError, match="common shape"):
        f + D.Array.from_numpy(rng.randn(2, 4).astype(np.float32))
    with pytest.raises(D.DaliError, match="duplicate axes"):
        op.sum(f, [0, 0])
    with pytest.raises(D.DaliError, match="Reduction axis"):
        op.sum(f, [2])
    with pytest.raises(D.DaliError, match="indices must be integers"):
        op.gather_from_rows(f, f)
    with pytest.raises(D.DaliError, match="not aligned"):
        op.dot(f, f)
    with pytest.raises(D.DaliError, match="depth must be strictly positive"):
        op.one_hot(i, 0, 1.0, 0.0)


def test_view_algebra_matches_numpy_strides(D, rng):
    x = rng.randn(4, 6, 5).astype(np.float32)
    a = D.Array.from_numpy(x)

    def same(view, ref):
        assert view.shape == ref.shape
        assert [s * 4 for s in view.strides] == [st if n > 1 else view.strides[k] * 4 for k, (st, n) in enumerate(zip(ref.strides, ref.shape))]
        assert view.offset * 4 == ref.__array_interface__["data"][0] - x.__array_interface__["data"][0]

    same(a.transpose(), x.transpose())
    same(a.transpose(1, 0, 2), x.transpose(1, 0, 2))
    same(a[1], x[1])
    same(a[:, 2:5], x[:, 2:5])
    same(a[:, ::2, 1:4], x[:, ::2, 1:4])
    same(a.reshape(24, 5), x.reshape(24, 5))
    assert a[:, 2:5].contiguous_memory() is False and a[1].contiguous_memory() is True
    assert a.expand_dims(1).shape == (4, 1, 6, 5)


# ------------------------------------------------- planner + code generation
def _cfg_roots(D, rng, small=True):
    op = D.op
    f = lambda *s: D.Array.from_numpy(rng.randn(*s).astype(np.float32))
    cfgs = {}
    a, b, c, d = f(4096), f(4096), f(4096), f(4096)
    cfgs["c2_chain"] = ([op.sigmoid(a) * op.tanh(b) + c * d - 0.5 * op.square(a)], "flat")
    cfgs["c1_softmax"] = ([op.softmax(f(64, 1024))], "row")
    m = f(128, 256)
    cfgs["c3_sum_axis1"] = ([op.sum(m, [1])], "row")
    cfgs["c3_max_axis0"] = ([op.max(m, [0])], "col")
    cfgs["c3_sum_all"] = ([op.sum(m)], "all")
    cfgs["c3_argmax_axis1"] = ([op.argmax(m, 1)], "row")
    x, t = f(16, 32000), D.Array.from_numpy(rng.randint(0, 32000, 16).astype(np.int32))
    mx = op.max(x, [-1], True)
    ex = op.exp(x - mx)
    s = op.sum(ex, [-1], True)
    grad = ex / s - op.one_hot(t, 32000, np.float32(1), np.float32(0))
    row_loss = (op.log(s) + mx) - op.gather_from_rows(x, t).expand_dims(1)
    cfgs["c4_cross_entropy"] = ([grad, row_loss], "row")
    pre, bias, cell = f(8, 4 * 64), f(4 * 64), f(8, 64)
    g = lambda k: pre[:, k * 64:(k + 1) * 64] + bias[k * 64:(k + 1) * 64].expand_dims(0)
    cn = op.sigmoid(g(1)) * cell + op.sigmoid(g(0)) * op.tanh(g(3))
    cfgs["c5_lstm_gates"] = ([cn, op.sigmoid(g(2)) * op.tanh(cn)], "map2d")
    return cfgs


def test_five_configs_plan_into_single_fused_kernels_that_compile(D, rng):
    for name, (roots, kind) in _cfg_roots(D, rng).items():
        n = D.generate_only(roots, compile=True)  # hipRTC for gfx950, no device needed
        assert (n, D.last_kernel_kinds()) == (1, kind), name
        src = D.last_source()
        assert 'extern "C" __global__' in src and "KArgs" in src, name


def test_softmax_kernel_reads_the_row_once_and_keeps_exp_in_registers(D, rng):
    roots, _ = _cfg_roots(D, rng)["c1_softmax"]
    D.generate_only(roots)
    src = D.last_source()
    body = src[src.index("void dali_row_"):]
    assert body.count("dali_load<float, 4>(q1") == 1  # one global read of the input
    assert body.count("functor::exp<float>::Map") == 1  # exp computed once, reused from registers
    # the row is reduced by wave64 butterflies: inside one wave, or two waves joined through LDS
    assert ("dali_group_reduce<reducers::maximum, float, 64>" in body
            or "dali_block_reduce<reducers::maximum, float, 2>" in body)


def test_rows_off_the_vector_alignment_keep_vector_accesses(D, rng):
    op = D.op
    x = D.Array.from_numpy(rng.randn(8, 1001).astype(np.float32))
    D.generate_only([op.softmax(x)], compile=True)
    body = D.last_source()
    body = body[body.index("void dali_row_"):]
    # source and destination rows start at the same distance from a 16-byte boundary: aligned vectors from the row's first
    # boundary, the elements in front of it and behind the last vector one to a thread
    assert "const int head" in body and "dali_loadu" not in body and "dali_storeu" not in body and "tail_on" in body
    assert "(v1 + (long)ch * 4)" in body and "tail_col = tr < head ? tr : CH * VEC + tr" in body
    y = D.Array.from_numpy(rng.randn(8, 1001).astype(np.float32))
    D.generate_only([op.softmax(x[:, 2:]) * y[:, :999]], compile=True)  # operands that start their rows at different distances
    body = D.last_source()
    body = body[body.index("void dali_row_"):]
    assert "dali_loadu" in body and "dali_storeu" in body and "tail_on" in body  # whole unaligned vectors + one element per thread
    D.generate_only([op.softmax(x[:, 1:])], compile=True)  # 1000 columns starting one element in: no rest, still unaligned
    body = D.last_source()
    body = body[body.index("void dali_row_"):]
    assert "dali_loadu" in body and "tail_on" not in body
    D.generate_only([op.softmax(x[:, :1000])], compile=True)  # row stride 1001: rows start at every alignment
    assert "dali_loadu" in D.last_source()[D.last_source().index("void dali_row_"):]
    small = D.Array.from_numpy(rng.randn(8, 13).astype(np.float32))
    D.generate_only([op.softmax(small)], compile=True)  # short rows: one element per access
    assert "dali_loadu" not in D.last_source()[D.last_source().index("void dali_row_"):]


def test_few_long_ragged_rows_are_cut_into_pieces_inside_the_row_kernel(D, rng):
    op = D.op
    x = D.Array.from_numpy(np.zeros((3, 1000001), np.float32))
    n = D.generate_only([op.argmax(x, 1)], compile=True)
    assert n == 3                                     # pieces, the first best piece of every row, its column
    first = D.generated_source(0)
    first = first[first.index("void dali_row_"):]
    # S * R workgroups, piece `seg` of a row writes element `seg` behind the row's first; the elements past the last whole
    # vector belong to the last piece; columns count from the start of the row
    assert "const int seg" in first and "q0[seg] =" in first and "q1[seg] =" in first and "seg == S - 1" in first
    assert "const int col = ch * VEC + j" in first and "for (int ch = ch_begin + tr; ch < ch_end; ch += TPR)" in first
    assert D.generate_only([op.sum(x, [1])], compile=True) == 2
    # softmax: each piece's maximum and its sum of exponentials relative to it from one walk, the merge of the pieces, the quotient
    assert D.generate_only([op.softmax(x)], compile=True) == 3
    pieces = D.generated_source(0)
    pieces = pieces[pieces.index("void dali_row_"):]
    assert "q0[seg] = (float)(red" in pieces and "q1[seg] = (float)(red" in pieces and pieces.count("for (int ch = ch_begin + tr; ch < ch_end; ch += TPR)") == 1
    assert "void dali_map2d_" in D.generated_source(2)
    # rows that divide into equal aligned pieces keep the reshaped view (cached pieces, (maximum, sum) in one pass)
    y = D.Array.from_numpy(np.zeros((3, 1 << 20), np.float32))
    assert D.generate_only([op.softmax(y)], compile=True) == 3


def test_long_cached_rows_put_part_of_the_row_into_lds(D, rng):
    op = D.op
    x = D.Array.from_numpy(np.zeros((4, 50257), np.float32))
    D.generate_only([op.softmax(x)], compile=True)
    body = D.last_source()
    body = body[body.index("constexpr int EPT_L"):]
    assert "EPT_L = 4" in body and "amdgpu_waves_per_eu(8, 8)" in D.last_source() and "__shared__ __attribute__((aligned(16))) float xl1[EPT_L][1024 * VEC]" in body
    short = D.Array.from_numpy(np.zeros((4, 32000), np.float32))
    D.generate_only([op.softmax(short)], compile=True)
    assert "EPT_L" not in D.last_source()  # 32 cached values per thread: registers alone


def test_planner_splits_what_cannot_fuse(D, rng):
    op = D.op
    m = D.Array.from_numpy(rng.randn(6, 8).astype(np.float32))
    n = D.generate_only([2 + (op.sum(m) - op.max(m))])
    assert D.last_kernel_kinds().split(",").count("all") == 2 and n == 3
    x3 = D.Array.from_numpy(rng.randn(3, 4, 5).astype(np.float32))
    D.generate_only([op.sum(x3, [1])], compile=True)
    assert D.last_kernel_kinds() == "col"  # middle axis: the column kernel over [batch, unit-stride run] kept axes
    assert "k_batch * (long)A.iv[" in D.last_source()
    x4 = D.Array.from_numpy(rng.randn(2, 3, 4, 5).astype(np.float32))
    D.generate_only([op.sum(x4, [0, 2])], compile=True)
    assert D.last_kernel_kinds() == "generic,row,row"  # kept axes on both sides of a reduced one: strided copy first
    D.generate_only([op.mean(m)], compile=True)
    assert D.last_kernel_kinds() == "all"  # the division by the count is folded into the last block


def test_gather_plans_as_an_indirect_row_leaf_and_checks_its_arguments(D, rng):
    table = D.Array.from_numpy(rng.randn(100, 64).astype(np.float32))
    idx = D.Array.from_numpy(np.arange(10, dtype=np.int32))
    g = D.op.gather(table, idx)
    assert g.shape == (10, 64) and not g.is_buffer()
    assert D.generate_only([D.op.tanh(g) * 2.0], compile=True) == 1  # one kernel: the map reads through the gather
    src = D.last_source()
    assert "dali_clamp_index(rl" in src  # the source row pointer goes through the per-row index value, held inside the source
    assert D.op.gather(table, D.Array.from_numpy(np.zeros((2, 3), np.int32))).shape == (2, 3, 64)
    with pytest.raises(RuntimeError, match="indices must be integers"):
        D.op.gather(table, D.Array.from_numpy(np.zeros(3, np.float32)))
    with pytest.raises(RuntimeError, match="same dimensionality"):
        t = D.Array.zeros((3,))
        t <<= D.Array.from_numpy(np.ones((3, 4), np.float32))


def test_scope_observers_see_the_planned_kernels(D, rng):
    """dali/utils/scope.h: an observer is told when a named scope opens and closes; the front-end names every generated
    kernel it plans "JIT[<shape>:<entry point>]" (generation only: no device needed). Observers stack and detach."""
    op = D.op
    x = D.Array.from_numpy(rng.randn(8, 64).astype(np.float32))
    seen = []
    with D.ScopeObserver(lambda name, trace: seen.append(("in", name, tuple(trace))),
                         lambda name, trace: seen.append(("out", name, tuple(trace)))) as outer:
        D.generate_only([op.softmax(x)])
        with D.ScopeObserver() as inner:
            D.generate_only([op.sum(x * 2.0)])
        D.generate_only([op.exp(x)])
    D.generate_only([op.tanh(x)])  # nobody observes any more
    names = [e[1] for e in outer.events if e[0] == "enter"]
    assert len(names) == 3 and names[0].startswith("JIT[row:dali_row_") and names[1].startswith("JIT[all:dali_all_") and names[2].startswith("JIT[flat:dali_flat_")
    assert [e[1] for e in inner.events] == [names[1], names[1]] and [e[0] for e in inner.events] == ["enter", "exit"]
    # every scope that opened closed again, at the depth it opened at, and the callbacks saw the stack of open scopes
    assert [e[0] for e in outer.events] == ["enter", "exit"] * 3 and all(e[2] == 1 for e in outer.events)
    assert seen[0] == ("in", names[0], (names[0],)) and seen[1] == ("out", names[0], (names[0],)) and len(seen) == 6
    assert outer.trace == [] and names[0].endswith("]")


def test_kept_leading_axes_with_a_reversed_axis_are_not_one_batch_axis(D, rng):
    """A reduction along a middle axis reads its kept leading axes as one batch axis only when their strides nest. With a
    reversed axis among them (strides 36, -18 for extents 2, 2) they do not: the plan must not be the batched column kernel
    (generation only; the values are checked on the device)."""
    op = D.op
    x = rng.randn(2, 2, 2, 9).astype(np.float32)
    D.generate_only([op.max(op.tanh(D.Array.from_numpy(x)), [2], True)])
    assert D.last_kernel_kinds() == "col" and "k_batch" in D.last_source()  # contiguous: one launch, batched
    D.generate_only([op.max(op.tanh(D.Array.from_numpy(x)[:, ::-1]), [2], True)])
    assert "k_batch" not in D.last_source()
    # reversed along the reduced axis itself, or along the innermost kept axis: the batch axes still nest
    D.generate_only([op.max(op.tanh(D.Array.from_numpy(x)[:, :, ::-1]), [2], True)])
    assert D.last_kernel_kinds().count("col") <= 1
