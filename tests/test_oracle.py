"""Pins the CPU checker (oracle/) before anything is compared against it.

Every function of the oracle is checked against (i) the expected values the
reference's own tests hold (tests/golden/reference_known_answers.json, with
file:line), (ii) the pieces of the reference compiled from its own headers
(oracle/_ref, when built), and (iii) independent mathematics: fp64 libm closed
forms, invariants and brute force with planted ties. None of these retype the
oracle's own formula.
"""
import math

import numpy as np
import pytest

from conftest import golden

FLT_MAX = np.finfo(np.float32).max


def f64(x):
    return np.asarray(x, dtype=np.float64)


# ------------------------------------------------------------------ functors
UNARY_TRUTH = {
    "sigmoid": lambda x: 1.0 / (1.0 + np.exp(-x)),
    "tanh": np.tanh,
    "exp": np.exp,
    "log": np.log,
    "negative_log": lambda x: -np.log(x),
    "square": lambda x: x * x,
    "cube": lambda x: x * x * x,
    "sqrt_f": np.sqrt,
    "rsqrt": lambda x: 1.0 / np.sqrt(x),
    "inv": lambda x: 1.0 / x,
    "identity": lambda x: x,
    "abs": np.abs,
    "sign": lambda x: np.where(x > 0, 1.0, -1.0),
    "relu": lambda x: np.where(x > 0, x, 0.0),
    "relu_backward": lambda x: np.where(x > 0, 1.0, 0.0),
    "dsigmoid": lambda x: x * (1.0 - x),
    "dtanh": lambda x: 1.0 - x * x,
    "softplus": lambda x: np.where(x > 20.0, x, np.log1p(np.exp(np.minimum(x, 30.0)))),
    "softplus_backward": lambda x: np.where(x > 20.0, 1.0, 1.0 / (1.0 + np.exp(-x))),
    "log_or_zero": lambda x: np.where(x > 0, np.log(np.where(x > 0, x, 1.0)), 0.0),
    "inverse_tanh": lambda x: np.arctanh(x),
    "safe_entropy_log": lambda x: np.log(np.clip(x, 1e-6, 1.0 - 1e-6)),
}


@pytest.mark.parametrize("name", sorted(UNARY_TRUTH))
def test_unary_against_fp64_closed_form(O, name):
    # the reference's own unary tests use x = arange(50)+1 (tests.cpp:1015-1073); a
    # signed range and a (0,1) range cover the functors defined only there
    xs = [np.arange(1, 51, dtype=np.float32), np.linspace(-6, 6, 97).astype(np.float32), np.linspace(0.02, 0.98, 49).astype(np.float32)]
    if name in ("log", "negative_log", "sqrt_f", "rsqrt", "inv"):
        xs = [xs[0], xs[2]]
    if name in ("inverse_tanh", "safe_entropy_log", "dsigmoid"):
        xs = [xs[2]]
    if name in ("exp", "cube"):
        xs = [xs[1], xs[2]]
    for x in xs:
        got = O.unary(name, x)
        want = UNARY_TRUTH[name](f64(x))
        np.testing.assert_allclose(got, want, rtol=3e-6, atol=1e-6, err_msg=name)


def test_sigmoid_is_the_double_precision_formula(O):
    # functor.h:157-162: 1.0 / (1.0 + expf(-a)) in double, rounded once; the float-only
    # formula differs in the last place on part of the range, so this catches dropping the double
    x = np.linspace(-10, 10, 20001).astype(np.float32)
    got = O.unary("sigmoid", x)
    e = np.exp(-x.astype(np.float32)).astype(np.float32)  # float expf
    want = (1.0 / (1.0 + e.astype(np.float64))).astype(np.float32)
    # numpy's float32 exp may differ from glibc expf by an ulp: compare through that slack
    assert np.max(np.abs(got.astype(np.float64) - want.astype(np.float64))) <= 1.2e-7
    assert got[10000] == np.float32(0.5)


def test_round_matches_reference_astype(O):
    g = golden("reference_known_answers.json")["astype_round"]
    got = O.round_to_int(np.array(g["input"], dtype=np.float32))
    assert got.tolist() == g["expected"]


def test_binary_closed_forms(O, rng):
    a = rng.uniform(-3, 3, 200).astype(np.float32)
    b = rng.uniform(0.5, 3, 200).astype(np.float32)
    A, B = f64(a), f64(b)
    checks = {
        "add": A + B, "subtract": A - B, "eltmul": A * B, "eltdiv": A / B,
        "equals": (A == B).astype(np.float64), "max_scalar": np.maximum(A, B), "min_scalar": np.minimum(A, B),
        "threshold": (A < B).astype(np.float64), "lessthanequal": (A <= B).astype(np.float64),
        "greaterthanequal": (A >= B).astype(np.float64), "prelu": np.where(A > 0, A, B * A),
        "clip": np.clip(A, -B, B), "div_grad": A / (B * B), "fill": B,
        "prelu_backward_inputs": np.where(A > 0, 1.0, B), "prelu_backward_weights": np.where(A > 0, 0.0, A * B),
        "steep_sigmoid": 1.0 / (1.0 + np.exp(-B * A)), "steep_sigmoid_backward": B * (A - A * A),
        "clipped_relu": np.where(A > 0, np.minimum(A, B), 0.0),
        "clipped_relu_backward": np.where(A > 0, np.where(A > B, 0.0, 1.0), 0.0),
    }
    for name, want in checks.items():
        np.testing.assert_allclose(O.binary(name, a, b), want, rtol=3e-6, atol=1e-6, err_msg=name)
    np.testing.assert_allclose(O.binary("power", np.abs(a) + 0.1, b), (np.abs(A) + np.float64(np.float32(0.1))) ** B, rtol=1e-5)
    p = rng.uniform(0.05, 0.95, 100).astype(np.float32)
    t = rng.randint(0, 2, 100).astype(np.float32)
    P, T = f64(p), f64(t)
    np.testing.assert_allclose(O.binary("binary_cross_entropy", p, t), -(T * np.log(P) + (1 - T) * np.log(1 - P)), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(O.binary("binary_cross_entropy_grad", p, t), (T - P) / (P * (P - 1)), rtol=1e-5)
    # scalar broadcast on either side (tests.cpp:1075-1117)
    np.testing.assert_allclose(O.binary("subtract", a, 2.0), A - 2.0, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(O.binary("subtract", 2.0, a), 2.0 - A, rtol=1e-6, atol=1e-6)


def test_chain_matches_fp64_truth_and_its_parts(O, rng):
    a, b, c, d = [rng.uniform(-4, 4, 5000).astype(np.float32) for _ in range(4)]
    got = O.chain(a, b, c, d)
    A, B, Cc, Dd = map(f64, (a, b, c, d))
    want = 1.0 / (1.0 + np.exp(-A)) * np.tanh(B) + Cc * Dd - 0.5 * A * A
    scale = np.abs(np.tanh(B)) + np.abs(Cc * Dd) + 0.5 * A * A
    assert np.all(np.abs(got - want) <= 3e-7 * scale + 1e-7)
    # dropping or flipping a term is far outside that bound
    assert np.max(np.abs((want + A * A) - got)) > 1.0
    # and it is exactly the composition of the single-functor entry points, each rounded to fp32
    comp = O.binary("subtract", O.binary("add", O.binary("eltmul", O.unary("sigmoid", a), O.unary("tanh", b)), O.binary("eltmul", c, d)),
                    O.binary("eltmul", np.float32(0.5), O.unary("square", a)))
    assert np.array_equal(comp, got)


# ------------------------------------------------------------------ reducers
def test_all_reduce_closed_forms(O):
    g = golden("reference_known_answers.json")
    for n in (1, 2, 5, 100, 1000):
        assert float(O.all_reduce(O.SUM, np.arange(n, dtype=np.float32))) == n * (n - 1) / 2
    assert float(O.all_reduce(O.PROD, np.array(g["all_reduce_prod"]["input"], np.float32))) == g["all_reduce_prod"]["expected"]
    mm = np.array(g["all_reduce_max_min"]["input"], np.float32)
    assert float(O.all_reduce(O.MAX, mm)) == g["all_reduce_max_min"]["max"]
    assert float(O.all_reduce(O.MIN, mm)) == g["all_reduce_max_min"]["min"]
    # init values: empty reductions return the reducer's neutral element (reducer_kernels.h)
    e = np.zeros(0, np.float32)
    assert float(O.all_reduce(O.SUM, e)) == 0.0 and float(O.all_reduce(O.PROD, e)) == 1.0
    assert O.all_reduce(O.MAX, e) == -FLT_MAX and O.all_reduce(O.MIN, e) == FLT_MAX


def test_sum_is_strictly_sequential_fp32(O):
    # 1 followed by many 2^-24: a left-to-right fp32 sum never leaves 1.0, pairwise or fp64 sums do
    x = np.full(1 + 4096, 2.0 ** -24, dtype=np.float32)
    x[0] = 1.0
    assert float(O.all_reduce(O.SUM, x)) == 1.0
    assert float(O.axis_reduce(O.SUM, x.reshape(1, -1), 1)[0]) == 1.0
    # reversed order accumulates the small terms first
    assert float(O.all_reduce(O.SUM, x[::-1].copy())) > 1.0


def test_axis_reduce_ones_and_strided_view(O, rng):
    # tests.cpp:1215-1239: reductions of ones give the reduced extent
    ones = np.ones((7, 13), np.float32)
    assert np.array_equal(O.axis_reduce(O.SUM, ones, 1), np.full(7, 13, np.float32))
    assert np.array_equal(O.axis_reduce(O.SUM, ones, 0), np.full(13, 7, np.float32))
    x = rng.randn(37, 53).astype(np.float32)
    np.testing.assert_allclose(O.axis_reduce(O.SUM, x, 0), f64(x).sum(0), atol=1e-5 * np.abs(x).sum(0).max())
    np.testing.assert_allclose(O.axis_reduce(O.SUM, x, 1), f64(x).sum(1), atol=1e-5 * np.abs(x).sum(1).max())
    assert np.array_equal(O.axis_reduce(O.MAX, x, 0), x.max(0)) and np.array_equal(O.axis_reduce(O.MAX, x, 1), x.max(1))
    assert np.array_equal(O.axis_reduce(O.MIN, x, 0), x.min(0)) and np.array_equal(O.axis_reduce(O.MIN, x, 1), x.min(1))
    # axis 0 must equal axis 1 of the materialised transpose bit for bit (same sequential order)
    assert np.array_equal(O.axis_reduce(O.SUM, x, 0), O.axis_reduce(O.SUM, np.ascontiguousarray(x.T), 1))
    np.testing.assert_allclose(O.axis_reduce(O.PROD, x[:5, :6], 1), np.prod(f64(x[:5, :6]), 1), rtol=1e-5)


def test_argmax_reference_vectors_and_ties(O):
    g = golden("reference_known_answers.json")["axis_argmax_argmin"]
    x = np.arange(20, dtype=np.float32).reshape(4, 5)
    assert O.arg_axis_reduce(O.MAX, x, 0).tolist() == g["argmax_axis0"]
    assert O.arg_axis_reduce(O.MAX, x, 1).tolist() == g["argmax_axis1"]
    assert O.arg_axis_reduce(O.MIN, x, 0).tolist() == g["argmin_axis0"]
    assert O.arg_axis_reduce(O.MIN, x, 1).tolist() == g["argmin_axis1"]
    # flat argmax / argmin (tests.cpp:1141-1148): ramp -100..99 -> max at the end, min at 0
    ramp = np.arange(-100, 42, dtype=np.float32)
    assert O.arg_all_reduce(O.MAX, ramp) == 141 and O.arg_all_reduce(O.MIN, ramp) == 0
    # planted ties: the FIRST of equal extrema wins (all_reduce_kernel_utils.cpp:217-219)
    t = np.array([[1, 7, 3, 7, 7], [5, 5, 5, 5, 5], [-2, -9, -9, 0, -9]], np.float32)
    assert O.arg_axis_reduce(O.MAX, t, 1).tolist() == [1, 0, 3]
    assert O.arg_axis_reduce(O.MIN, t, 1).tolist() == [0, 0, 1]
    # brute force over every length-4 row of {0,1,2}
    import itertools
    rows = np.array(list(itertools.product([0, 1, 2], repeat=4)), np.float32)
    assert O.arg_axis_reduce(O.MAX, rows, 1).tolist() == [int(np.argmax(r)) for r in rows]
    assert O.arg_axis_reduce(O.MIN, rows, 1).tolist() == [int(np.argmin(r)) for r in rows]
    # sentinel: a row of -FLT_MAX (or -inf) never replaces the initial value, index stays 0
    s = np.array([[-FLT_MAX, -FLT_MAX], [-np.inf, -np.inf]], np.float32)
    assert O.arg_axis_reduce(O.MAX, s, 1).tolist() == [0, 0]


def test_reducers_against_reference_headers(O, rng):
    if O.ref is None:
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    import ctypes as C
    x = rng.randn(19, 23).astype(np.float32)
    x[3, 5] = x[3, 11] = 9.0  # tie
    for red in (O.SUM, O.MAX, O.MIN, O.PROD):
        for (rows, cols, rs, cs, axis) in ((19, 23, 23, 1, 1), (23, 19, 1, 23, 0)):
            want = np.empty(rows, np.float32)
            O.ref.ref_axis_reduce(red, O.fp(x), rows, cols, rs, cs, O.fp(want))
            assert np.array_equal(O.axis_reduce(red, x, axis), want)
        assert O.all_reduce(red, x) == np.float32(O.ref.ref_all_reduce(red, O.fp(x), x.size))
    for red in (O.MAX, O.MIN):
        for (rows, cols, rs, cs, axis) in ((19, 23, 23, 1, 1), (23, 19, 1, 23, 0)):
            want = np.empty(rows, np.int32)
            O.ref.ref_arg_axis_reduce(red, O.fp(x), rows, cols, rs, cs, O.ip(want))
            assert np.array_equal(O.arg_axis_reduce(red, x, axis), want)


def test_reference_index_arithmetic(O):
    if O.ref is None:
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    shape = np.array([3, 4, 5], np.int32)
    out = np.empty(3, np.int32)
    for idx in (0, 7, 23, 59):
        O.ref.ref_index_to_dim3(idx, O.ip(shape), O.ip(out))
        assert tuple(out) == np.unravel_index(idx, (3, 4, 5))
        assert O.ref.ref_indices_to_offset3(O.ip(shape), O.ip(out)) == idx


def test_mean(O):
    x = np.arange(10, dtype=np.float32)
    assert float(O.mean_all(x)) == 4.5


# -------------------------------------------------------- softmax and friends
def test_softmax_invariants(O, rng):
    x = (rng.randn(7, 33) * 3).astype(np.float32)
    s = O.softmax(x)
    e = np.exp(f64(x) - f64(x).max(1, keepdims=True))
    np.testing.assert_allclose(s, e / e.sum(1, keepdims=True), rtol=2e-6)
    np.testing.assert_allclose(s.sum(1), 1.0, atol=1e-6)
    # shift invariance holds up to the rounding of x + c; an exact power-of-two-friendly case is bit-identical
    xi = rng.randint(-8, 8, size=(5, 16)).astype(np.float32)
    assert np.array_equal(O.softmax(xi), O.softmax(xi + 4.0))
    # one dominant logit
    big = np.array([[0.0, 100.0, 0.0]], np.float32)
    assert O.softmax(big)[0, 1] == 1.0
    # the staged computation of tests.cpp:1622-1664 on U(-20,20) [2,5]
    u = rng.uniform(-20, 20, (2, 5)).astype(np.float32)
    staged = O.binary("eltdiv", O.unary("exp", u - u.max(1, keepdims=True)),
                      np.repeat(O.axis_reduce(O.SUM, O.unary("exp", u - u.max(1, keepdims=True)), 1)[:, None], 5, 1))
    np.testing.assert_allclose(O.softmax(u), staged, atol=1e-6)


def test_gather_from_rows_reference_table(O):
    g = golden("reference_known_answers.json")["gather_from_rows_3d"]
    src = np.arange(5 * 6 * 7, dtype=np.float32).reshape(5, 6, 7)
    idx = np.arange(5, dtype=np.int32)
    # the 3-D case gathers whole trailing rows; column j of the table is a 2-D gather on source[:, :, j]
    got = np.stack([O.gather_from_rows(np.ascontiguousarray(src[:, :, j]), idx) for j in range(7)], axis=1)
    assert got.astype(np.int64).tolist() == g["expected"]
    src2 = np.arange(30, dtype=np.float32).reshape(5, 6)
    assert O.gather_from_rows(src2, idx).tolist() == [src2[i, i] for i in range(5)]


def test_one_hot_reference_semantics(O, rng):
    # tests.cpp:984-1012: depth 7, on 112.2, off 42.0 compared with an explicit scatter
    idx = rng.randint(0, 6, size=6).astype(np.int32)
    got = O.one_hot(idx, 7, 112.2, 42.0)
    want = np.full((6, 7), np.float32(42.0), np.float32)
    want[np.arange(6), idx] = np.float32(112.2)
    assert np.array_equal(got, want)


def test_cross_entropy_identities(O, rng):
    x = (rng.randn(5, 97) * 2).astype(np.float32)
    t = rng.randint(0, 97, size=5).astype(np.int32)
    mean, rows, grad = O.softmax_cross_entropy(x, t)
    X = f64(x)
    lse = np.log(np.exp(X - X.max(1, keepdims=True)).sum(1)) + X.max(1)
    want_rows = lse - X[np.arange(5), t]
    np.testing.assert_allclose(rows, want_rows, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(mean, want_rows.mean(), rtol=1e-5)
    sm = np.exp(X - lse[:, None])
    oh = np.zeros_like(X)
    oh[np.arange(5), t] = 1
    np.testing.assert_allclose(grad, sm - oh, atol=2e-6)
    np.testing.assert_allclose(grad.sum(1), 0.0, atol=1e-5)  # rows of softmax - onehot sum to zero
    # agrees with the reference's own forward -log(softmax[i, t]) (cost.cpp:121-122)
    np.testing.assert_allclose(O.softmax_cross_entropy_via_probs(x, t), rows, rtol=1e-5, atol=2e-6)
    # a wrong sign in the gather term or a missing max would break this: loss of a one-hot-dominant row is ~0
    z = np.zeros((1, 4), np.float32)
    z[0, 2] = 50
    assert abs(float(O.softmax_cross_entropy(z, np.array([2], np.int32))[1][0])) < 1e-6


# --------------------------------------------------------------------- gemm
def test_gemm_known_answers(O):
    g = golden("reference_known_answers.json")["dot_known"]
    a = np.ones((2, 3), np.float32)
    b = np.arange(12, dtype=np.float32).reshape(3, 4)
    for mode in ("f64", "f32"):
        assert O.gemm(a, b, mode).tolist() == g["ones_2x3_times_arange_3x4"]
    m = np.arange(12, dtype=np.float32).reshape(4, 3)
    v = np.arange(3, dtype=np.float32).reshape(3, 1)
    assert O.gemm(m, v)[:, 0].tolist() == g["arange_4x3_times_arange_3"]
    ai = np.arange(6, dtype=np.int32).reshape(2, 3)
    bi = np.arange(12, dtype=np.int32).reshape(3, 4)
    assert np.array_equal(O.gemm_i32(ai, bi), ai @ bi)


def test_gemm_layouts_against_numpy_fp64(O, rng):
    A = rng.randn(5, 7).astype(np.float32)
    B = rng.randn(7, 11).astype(np.float32)
    want = f64(A) @ f64(B)
    At = np.ascontiguousarray(A.T).T  # transposed storage
    Bt = np.ascontiguousarray(B.T).T
    wide = rng.randn(5, 20).astype(np.float32)
    As = wide[:, 3:10]  # row-strided view
    for (a, b, w) in ((A, B, want), (At, B, want), (A, Bt, want), (At, Bt, want), (As, B, f64(As) @ f64(B))):
        np.testing.assert_allclose(O.gemm(a, b, "f64"), w, rtol=1e-6, atol=1e-6)
        np.testing.assert_allclose(O.gemm(a, b, "f32"), w, rtol=1e-4, atol=1e-5)


def test_gemm_against_reference_template(O, rng):
    if O.ref is None:
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    # igemm call of cpu_gemm.cpp:14-20,52-58 for row-major lhs[n,k] . rhs[k,m]: (!rhs_T, !lhs_T, m, n, k, rhs, ldr, lhs, ldl, dst, ldd)
    lhs = rng.randint(-5, 5, size=(4, 6)).astype(np.int32)
    rhs = rng.randint(-5, 5, size=(6, 3)).astype(np.int32)
    dst = np.zeros((4, 3), np.int32)
    O.ref.ref_gemm_i32(1, 1, 3, 4, 6, O.ip(rhs), 3, O.ip(lhs), 6, O.ip(dst), 3)
    assert np.array_equal(dst, lhs @ rhs)
    assert np.array_equal(O.gemm_i32(lhs, rhs), dst)
    fl, fr = lhs.astype(np.float32) * 0.37, rhs.astype(np.float32) * 1.3
    fd = np.zeros((4, 3), np.float32)
    O.ref.ref_gemm_f32(1, 1, 3, 4, 6, O.fp(fr), 3, O.fp(fl), 6, O.fp(fd), 3)
    assert np.array_equal(O.gemm(fl, fr, "f32"), fd)  # same sequential fp32 accumulation order


# --------------------------------------------------------------------- lstm
def test_lstm_step_composition(O, rng):
    B, I, H = 3, 8, 8
    X, Hp, Cp = rng.randn(B, I).astype(np.float32), rng.randn(B, H).astype(np.float32), rng.randn(B, H).astype(np.float32)
    W, U = (rng.randn(I, 4 * H) * 0.3).astype(np.float32), (rng.randn(H, 4 * H) * 0.3).astype(np.float32)
    b = (rng.randn(4 * H) * 0.1).astype(np.float32)
    gates, c_new, h_new = O.lstm_step(X, Hp, Cp, W, U, b)
    G = f64(b) + f64(X) @ f64(W) + f64(Hp) @ f64(U)
    np.testing.assert_allclose(gates, G, rtol=1e-5, atol=1e-6)
    sig = lambda z: 1.0 / (1.0 + np.exp(-z))
    i, f, o, g = sig(G[:, :H]), sig(G[:, H:2 * H]), sig(G[:, 2 * H:3 * H]), np.tanh(G[:, 3 * H:])
    c = f * f64(Cp) + i * g
    np.testing.assert_allclose(c_new, c, rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(h_new, o * np.tanh(c), rtol=1e-5, atol=2e-6)
    # gate order matters: swapping o and g changes the answer
    assert np.max(np.abs(h_new - sig(G[:, 3 * H:]) * np.tanh(c))) > 1e-2


# ---------------------------------------------------------------- gather / scatter
def test_gather_rows_is_fancy_indexing(O, rng):
    src = rng.randn(11, 7).astype(np.float32)
    idx = rng.randint(0, 11, 23).astype(np.int32)
    assert np.array_equal(O.gather_rows(src, idx), src[idx])
    # reference_gather of tests.cpp:1251-1272: arange source, arange indices reproduce the source
    a = np.arange(30, dtype=np.float32).reshape(5, 6)
    assert np.array_equal(O.gather_rows(a, np.arange(5)), a)


def test_scatter_rows_reference_known_answers_and_duplicates(O, rng):
    # GatherTests.scatter_simple (tests.cpp:1316-1331): dest[{0,0,1,1,1,2}] += 1 on zeros(3) -> 2, 3, 1
    out = O.scatter_rows(np.zeros((3, 1), np.float32), [0, 0, 1, 1, 1, 2], 1.0, op=1)
    assert out.ravel().tolist() == [2.0, 3.0, 1.0]
    # integer-valued data: any order gives the same sums, numpy's unbuffered add is the library answer
    dest = rng.randint(-5, 5, (9, 4)).astype(np.float32)
    idx = rng.randint(0, 9, 40).astype(np.int32)
    vals = rng.randint(-3, 3, (40, 4)).astype(np.float32)
    want = dest.copy()
    np.add.at(want, idx, vals)
    assert np.array_equal(O.scatter_rows(dest, idx, vals, op=1), want)
    want = dest.copy()
    np.subtract.at(want, idx, vals)
    assert np.array_equal(O.scatter_rows(dest, idx, vals, op=2), want)
    # plain assignment: the last writer in input order wins
    got = O.scatter_rows(dest, idx, vals, op=0)
    for r in range(9):
        hits = np.nonzero(idx == r)[0]
        assert np.array_equal(got[r], vals[hits[-1]] if hits.size else dest[r])
    # fp32 with duplicates: input-order accumulation, restated as an explicit python loop on one column
    d1 = rng.randn(5, 1).astype(np.float32)
    i1 = rng.randint(0, 5, 200).astype(np.int32)
    v1 = (rng.randn(200, 1) * 1e3).astype(np.float32)
    acc = d1.copy()
    for i in range(200):
        acc[i1[i], 0] = np.float32(acc[i1[i], 0] + v1[i, 0])
    assert np.array_equal(O.scatter_rows(d1, i1, v1, op=1), acc)


def test_scatter_to_rows_reference_known_answer(O):
    # GatherTests.scatter_to_rows_simple (tests.cpp:1333-1361): 42 everywhere, +1 at (i, vals[i])
    vals = [0, 0, 1, 1, 1, 2]
    out = O.scatter_to_rows(np.full((7, 3), 42, np.float32)[:6], vals, 1.0, op=1)
    for i, v in enumerate(vals):
        assert out[i].tolist() == [43.0 if j == v else 42.0 for j in range(3)]


def test_axis_scan_known_answers(O, rng):
    # ScanTests.cumsum / cumprod (tests.cpp:1737-1786): arange inputs, 1-D and [2, 10], inclusive and exclusive
    a = np.arange(20, dtype=np.float32)
    assert np.array_equal(O.axis_scan("sum", a), np.cumsum(a))
    assert np.array_equal(O.axis_scan("sum", a, False), np.concatenate([[0], np.cumsum(a)]))
    assert np.array_equal(O.axis_scan("sum", a.reshape(2, 10)), np.cumsum(a.reshape(2, 10), axis=1))
    p = np.arange(1, 11, dtype=np.float32)  # 10! is exact in fp32
    assert np.array_equal(O.axis_scan("product", p), np.cumprod(p.astype(np.float64)).astype(np.float32))
    assert np.array_equal(O.axis_scan("product", p, False)[0:2], [1.0, 1.0])
    x = rng.randn(3, 50).astype(np.float32)
    assert np.array_equal(O.axis_scan("maximum", x), np.maximum.accumulate(x, axis=1))
    assert np.array_equal(O.axis_scan("minimum", x), np.minimum.accumulate(x, axis=1))
    # fp32 sums: numpy's cumsum is the same left-to-right fp32 accumulation
    assert np.array_equal(O.axis_scan("sum", x), np.cumsum(x, axis=1, dtype=np.float32))


def test_circular_convolution_is_a_circular_correlation(O, rng):
    # integer-valued data: exact against the definition written with numpy's roll
    c = rng.randint(-4, 5, (3, 11)).astype(np.float32)
    w = rng.randint(-4, 5, (3, 11)).astype(np.float32)
    want = np.stack([sum(np.roll(c[r], -s) * w[r, s] for s in range(11)) for r in range(3)])
    assert np.array_equal(O.circular_convolution(c, w), want)
    # a one-hot weight at position s shifts the content left by s (circular_convolution.cpp:31-36)
    e = np.zeros(7, np.float32)
    e[2] = 1.0
    x = np.arange(7, dtype=np.float32)
    assert np.array_equal(O.circular_convolution(x, e), np.roll(x, -2))
    # the circular-correlation theorem pins the general case: FFT(out) = FFT(c) * conj(FFT(w)) for real w
    cf, wf = rng.randn(2, 64), rng.randn(2, 64)
    got = O.circular_convolution(cf, wf).astype(np.float64)
    ref = np.fft.ifft(np.fft.fft(cf.astype(np.float32)) * np.conj(np.fft.fft(wf.astype(np.float32)))).real
    assert np.abs(got - ref).max() < 1e-4


# ------------------------------------------------------------------ sliding windows
def _patches_by_slicing(image_nhwc, fh, fw, sh, sw):
    """The definition the reference's test uses (im2col_tests.cpp:7-39): every window of the NHWC image, raveled."""
    n, h, w, _ = image_nhwc.shape
    cols = []
    for b in range(n):
        for i in range(0, h - fh + 1, sh):
            for j in range(0, w - fw + 1, sw):
                cols.append(image_nhwc[b, i:i + fh, j:j + fw].ravel())
    return np.stack(cols, axis=1)


def test_im2col_matches_the_slicing_definition(O, rng):
    # JITTests.im2col_without_channels (im2col_tests.cpp:41-72): arange image [2,1,3,4], 3x3 windows, three layouts
    nchw = np.arange(24, dtype=np.float32).reshape(2, 1, 3, 4)
    nhwc = nchw.transpose(0, 2, 3, 1)
    want = _patches_by_slicing(nhwc, 3, 3, 1, 1)
    assert np.array_equal(O.im2col(nhwc, 3, 3, 1, 1, data_format="NHWC"), want)
    assert np.array_equal(O.im2col(nchw, 3, 3, 1, 1, data_format="NCHW"), want)
    wnch = O.im2col(nchw.transpose(3, 0, 1, 2), 3, 3, 1, 1, data_format="WNCH")
    assert np.array_equal(wnch.reshape(3, 1, 3, -1).transpose(1, 2, 0, 3).reshape(9, -1), want)
    # with channels and strides: NHWC rows run (kh, kw, c), NCHW rows run (c, kh, kw)
    for sh, sw in ((1, 1), (2, 1), (2, 3)):
        x = rng.randint(-9, 10, (3, 7, 9, 4)).astype(np.float32)
        want = _patches_by_slicing(x, 3, 2, sh, sw)
        assert np.array_equal(O.im2col(x, 3, 2, sh, sw, data_format="NHWC"), want)
        got = O.im2col(x.transpose(0, 3, 1, 2), 3, 2, sh, sw, data_format="NCHW")
        assert np.array_equal(got.reshape(4, 3, 2, -1).transpose(1, 2, 0, 3).reshape(24, -1), want)
    # padding = im2col of the zero-padded image
    x = rng.randint(-9, 10, (2, 5, 6, 3)).astype(np.float32)
    padded = np.pad(x, ((0, 0), (1, 2), (2, 1), (0, 0)))
    assert np.array_equal(O.im2col(x, 3, 3, 1, 2, 1, 2, 2, 1, "NHWC"), _patches_by_slicing(padded, 3, 3, 1, 2))


def _direct_conv2d(x_nchw, w_oihw, sh, sw, padding):
    """Direct convolution (the loop of conv_tests.cpp:57-126), fp64."""
    n, c, h, w = x_nchw.shape
    o, _, fh, fw = w_oihw.shape
    if padding == "same":
        oh, ow = -(-h // sh), -(-w // sw)
        ph, pw = max(0, (oh - 1) * sh + fh - h), max(0, (ow - 1) * sw + fw - w)
        x_nchw = np.pad(x_nchw, ((0, 0), (0, 0), (ph // 2, ph - ph // 2), (pw // 2, pw - pw // 2)))
    else:
        oh, ow = -(-(h - fh + 1) // sh), -(-(w - fw + 1) // sw)
    out = np.zeros((n, o, oh, ow))
    for i in range(oh):
        for j in range(ow):
            win = x_nchw[:, :, i * sh:i * sh + fh, j * sw:j * sw + fw].astype(np.float64)
            out[:, :, i, j] = np.einsum("nchw,ochw->no", win, w_oihw.astype(np.float64))
    return out


def test_conv2d_tensorflow_tables_and_direct_loop(O, rng):
    g = golden("reference_known_answers.json")["conv2d_tensorflow"]
    image = np.arange(2 * 3 * 7 * 5, dtype=np.float32).reshape(2, 3, 7, 5)
    filters = np.arange(4 * 3 * 6 * 5, dtype=np.float32).reshape(3, 6, 5, 4).transpose(3, 0, 1, 2)
    for mode in ("f64", "f32"):  # every partial sum is an integer below 2^24: exact either way
        assert np.array_equal(O.conv2d(image, filters, 1, 1, "valid", "NHWC", mode).ravel(), np.array(g["valid"], np.float32))
        assert np.array_equal(O.conv2d(image, filters, 1, 1, "same", "NHWC", mode).ravel(), np.array(g["same"], np.float32))
    # ConvTests.conv2d_forward (conv_tests.cpp:348-410): strides 1..3, both layouts, both paddings
    for sh in (1, 2, 3):
        for sw in (1, 2, 3):
            for padding in ("valid", "same"):
                x = rng.uniform(-1, 1, (5, 3, 6, 8)).astype(np.float32)
                w = rng.uniform(-1, 1, (2, 3, 2, 4)).astype(np.float32)
                want = _direct_conv2d(x, w, sh, sw, padding)
                got = O.conv2d(x, w, sh, sw, padding, "NCHW")
                assert got.shape == want.shape and np.abs(got - want).max() < 1e-5
                got = O.conv2d(x.transpose(0, 2, 3, 1), w.transpose(0, 2, 3, 1), sh, sw, padding, "NHWC")
                assert np.abs(got.transpose(0, 3, 1, 2) - want).max() < 1e-5


def test_col2im_is_the_adjoint_of_im2col(O, rng):
    for fmt, perm in (("NCHW", (0, 1, 2, 3)), ("NHWC", (0, 2, 3, 1))):
        for fh, fw, sh, sw in ((3, 3, 1, 1), (2, 3, 2, 1), (2, 2, 2, 2), (3, 2, 2, 3)):
            shape_nchw = (2, 3, 7, 8)
            # sizes for which the windows tile exactly, as op::col2im requires (col2im.cpp:204-215)
            x = rng.randint(-5, 6, shape_nchw).astype(np.float32).transpose(perm)
            px = O.im2col(x, fh, fw, sh, sw, data_format=fmt)
            y = rng.randint(-5, 6, px.shape).astype(np.float32)
            back = O.col2im(y, x.shape, fh, fw, sh, sw, fmt)
            # <im2col(x), y> == <x, col2im(y)> exactly on small integers
            assert float((px.astype(np.float64) * y).sum()) == float((x.astype(np.float64) * back).sum())
            # col2im(im2col(x)) = x times the number of windows that hold each pixel
            count = O.col2im(np.ones_like(px), x.shape, fh, fw, sh, sw, fmt)
            assert np.array_equal(O.col2im(px, x.shape, fh, fw, sh, sw, fmt), x * count)
            oh, ow = (7 - fh) // sh + 1, (8 - fw) // sw + 1
            assert count.sum() == 2 * 3 * oh * ow * fh * fw
    # JITTests.col2im_without_channels (col2im_tests.cpp:9-35): the two layouts agree
    nchw = np.arange(24, dtype=np.float32).reshape(2, 1, 3, 4)
    nchw[1] *= -1.0
    nhwc = np.ascontiguousarray(nchw.transpose(0, 2, 3, 1))
    a = O.col2im(O.im2col(nchw, 3, 3, 1, 1, data_format="NCHW"), nchw.shape, 3, 3, 1, 1, "NCHW")
    b = O.col2im(O.im2col(nhwc, 3, 3, 1, 1, data_format="NHWC"), nhwc.shape, 3, 3, 1, 1, "NHWC")
    assert np.array_equal(a.transpose(0, 2, 3, 1), b)


def _pool_windows(h, w, wh, ww, sh, sw, padding):
    ceil = lambda a, b: -(-a // b)
    if padding == "same":
        oh, ow = ceil(h, sh), ceil(w, sw)
        ph, pw = max(0, (oh - 1) * sh + wh - h) // 2, max(0, (ow - 1) * sw + ww - w) // 2
    else:
        oh, ow, ph, pw = ceil(h - wh + 1, sh), ceil(w - ww + 1, sw), 0, 0
    for i in range(oh):
        for j in range(ow):
            yield i, j, max(i * sh - ph, 0), min(i * sh + wh - ph, h), max(j * sw - pw, 0), min(j * sw + ww - pw, w)


def test_pool2d_pair_against_window_loops(O, rng):
    # the loops of reference_pool2d / reference_pool2d_backward (conv_tests.cpp:422-545), in fp64, NCHW and NHWC
    for wh in (1, 2, 3):
        for ww in (1, 2, 3):
            for sh, sw in ((1, 1), (2, 1), (2, 2)):
                for padding in ("valid", "same"):
                    for mode in ("max", "avg"):
                        x = rng.uniform(-1, 1, (2, 3, 6, 8)).astype(np.float32)
                        wins = list(_pool_windows(6, 8, wh, ww, sh, sw, padding))
                        oh, ow = wins[-1][0] + 1, wins[-1][1] + 1
                        want = np.zeros((2, 3, oh, ow))
                        for i, j, h0, h1, w0, w1 in wins:
                            win = x[:, :, h0:h1, w0:w1].astype(np.float64).reshape(2, 3, -1)
                            want[:, :, i, j] = win.max(-1) if mode == "max" else win.mean(-1)
                        y = O.pool2d(x, wh, ww, sh, sw, mode, padding, "NCHW")
                        assert y.shape == want.shape and np.abs(y - want).max() < 1e-6
                        xh = np.ascontiguousarray(x.transpose(0, 2, 3, 1))
                        yh = O.pool2d(xh, wh, ww, sh, sw, mode, padding, "NHWC")
                        assert np.array_equal(yh.transpose(0, 3, 1, 2), y)
                        dy = rng.uniform(-1, 1, y.shape).astype(np.float32)
                        dx_want = np.zeros(x.shape)
                        for i, j, h0, h1, w0, w1 in wins:
                            if mode == "avg":
                                dx_want[:, :, h0:h1, w0:w1] += dy[:, :, i, j, None, None].astype(np.float64) / ((h1 - h0) * (w1 - w0))
                            else:
                                hit = x[:, :, h0:h1, w0:w1] == y[:, :, i, j, None, None]
                                dx_want[:, :, h0:h1, w0:w1] += hit * dy[:, :, i, j, None, None].astype(np.float64)
                        dx = O.pool2d_backward(y, dy, x, wh, ww, sh, sw, mode, padding, "NCHW")
                        assert np.abs(dx - dx_want).max() < 1e-6
                        dxh = O.pool2d_backward(yh, np.ascontiguousarray(dy.transpose(0, 2, 3, 1)), xh, wh, ww, sh, sw, mode, padding, "NHWC")
                        assert np.array_equal(dxh.transpose(0, 3, 1, 2), dx)


def test_gru_step_against_fp64_definition(O, rng):
    # dali/layers/gru.cpp:27-44 written out in fp64 with numpy; the checker rounds every operation to fp32
    B, I, H = 6, 10, 8
    X, Hp = rng.randn(B, I).astype(np.float32), rng.randn(B, H).astype(np.float32)
    W, U = rng.uniform(-0.4, 0.4, (I, 3 * H)).astype(np.float32), rng.uniform(-0.4, 0.4, (H, 3 * H)).astype(np.float32)
    b = (rng.randn(3 * H) * 0.1).astype(np.float32)
    x, h, w, u, bb = (f64(v) for v in (X, Hp, W, U, b))
    sig = lambda v: 1.0 / (1.0 + np.exp(-v))
    r = sig(x @ w[:, :H] + h @ u[:, :H] + bb[:H])
    z = sig(x @ w[:, H:2 * H] + h @ u[:, H:2 * H] + bb[H:2 * H])
    m = np.tanh(x @ w[:, 2 * H:] + (r * h) @ u[:, 2 * H:] + bb[2 * H:])
    want = h * (1.0 - z) + m * z
    assert np.abs(O.gru_step(X, Hp, W, U, b) - want).max() < 2e-6
    # GRU::activate_sequence (gru.cpp:59-64) carries the state through the steps: against the fp64 recurrence
    Xg = rng.randn(4, B, I).astype(np.float32)
    state = h
    for t in range(4):
        xt = f64(Xg[t])
        r = sig(xt @ w[:, :H] + state @ u[:, :H] + bb[:H])
        z = sig(xt @ w[:, H:2 * H] + state @ u[:, H:2 * H] + bb[H:2 * H])
        m = np.tanh(xt @ w[:, 2 * H:] + (r * state) @ u[:, 2 * H:] + bb[2 * H:])
        state = state * (1.0 - z) + m * z
        assert np.abs(O.gru_sequence(Xg, Hp, W, U, b)[t] - state).max() < 1e-5
    # the sequence wrapper is the step in turn
    Xs = rng.randn(3, B, H).astype(np.float32)
    W4, U4 = rng.uniform(-0.3, 0.3, (H, 4 * H)).astype(np.float32), rng.uniform(-0.3, 0.3, (H, 4 * H)).astype(np.float32)
    b4 = np.zeros(4 * H, np.float32)
    hs, c = O.lstm_sequence(Xs, Hp, Hp, W4, U4, b4)
    _, c1, h1 = O.lstm_step(Xs[0], Hp, Hp, W4, U4, b4)
    _, c2, h2 = O.lstm_step(Xs[1], h1, c1, W4, U4, b4)
    assert np.array_equal(hs[1], h2) and hs.shape == (3, B, H)


def test_stacked_lstm_step_against_fp64_definition(O, rng):
    # dali/layers/stacked_lstm.cpp:219-283 written out in fp64: layer l reads h'(l-1); a shortcut layer reads [h'(l-1), x]
    B, I, sizes = 5, 7, [6, 4, 9]
    sig = lambda v: 1.0 / (1.0 + np.exp(-v))
    for shortcut in (False, True):
        X = rng.randn(B, I).astype(np.float32)
        Hs = [rng.randn(B, h).astype(np.float32) for h in sizes]
        Cs = [rng.randn(B, h).astype(np.float32) for h in sizes]
        ins = [I] + [sizes[l - 1] + (I if shortcut else 0) for l in range(1, len(sizes))]
        Ws = [rng.uniform(-0.4, 0.4, (n, 4 * h)).astype(np.float32) for n, h in zip(ins, sizes)]
        Us = [rng.uniform(-0.4, 0.4, (h, 4 * h)).astype(np.float32) for h in sizes]
        bs = [(rng.randn(4 * h) * 0.1).astype(np.float32) for h in sizes]
        cs, hs = O.stacked_lstm_step(X, Hs, Cs, Ws, Us, bs, shortcut)
        below = f64(X)
        for l, h in enumerate(sizes):
            inp = np.concatenate([below, f64(X)], 1) if (shortcut and l > 0) else below
            g = inp @ f64(Ws[l]) + f64(Hs[l]) @ f64(Us[l]) + f64(bs[l])
            i_, f_, o_, g_ = sig(g[:, :h]), sig(g[:, h:2 * h]), sig(g[:, 2 * h:3 * h]), np.tanh(g[:, 3 * h:])
            c = f_ * f64(Cs[l]) + i_ * g_
            hid = o_ * np.tanh(c)
            assert np.abs(cs[l] - c).max() < 5e-6 and np.abs(hs[l] - hid).max() < 5e-6, (shortcut, l)
            below = hid
    # one layer is the plain step; a different number of states is refused (stacked_lstm.cpp:225-227)
    _, c1, h1 = O.lstm_step(X, Hs[0], Cs[0], Ws[0], Us[0], bs[0])
    cs, hs = O.stacked_lstm_step(X, Hs[:1], Cs[:1], Ws[:1], Us[:1], bs[:1])
    assert np.array_equal(cs[0], c1) and np.array_equal(hs[0], h1)
    with pytest.raises(ValueError, match="Activating LSTM stack of size 3 with different number of states 2"):
        O.stacked_lstm_step(X, Hs[:2], Cs[:2], Ws, Us, bs)


def test_k_best_against_the_reference_comparators(O, rng):
    """The heap comparators of top_k.cpp:103-135 and the full-sort rule of :139-158, applied by brute force (selection by
    repeated scans, no sort routine) to rows full of ties; argsort is increasing (other_tests.cpp:6-31)."""
    def better_top(row, a, b):  # stable_comp(a, b), reversed = false
        return row[b] < row[a] or (row[b] == row[a] and a < b)

    def better_bottom(row, a, b):  # stable_comp(a, b), reversed = true
        return row[b] > row[a] or (row[b] == row[a] and a > b)

    def select(row, k, better):
        left, out = list(range(len(row))), []
        for _ in range(k):
            best = left[0]
            for c in left[1:]:
                if better(row, c, best):
                    best = c
            out.append(best)
            left.remove(best)
        return out

    for dtype in (np.float32, np.int32, np.float64):
        x = rng.randint(-3, 4, (5, 9)).astype(dtype)
        for k in (2, 3, 8):
            assert O.k_best(x, k, True).tolist() == [select(r, k, better_top) for r in x]
            assert O.k_best(x, k, False).tolist() == [select(r, k, better_bottom) for r in x]
        # the whole row: values in order, equal values in ascending position
        full_top = O.k_best(x, 9, True)
        full_bottom = O.k_best(x, 9, False)
        for r in range(5):
            assert full_top[r].tolist() == sorted(range(9), key=lambda c: (-float(x[r, c]), c))
            assert full_bottom[r].tolist() == sorted(range(9), key=lambda c: (float(x[r, c]), c))
        assert np.array_equal(O.k_best(x, 1, True)[:, 0], x.argmax(1)) and np.array_equal(O.k_best(x, 1, False)[:, 0], x.argmin(1))
    a = rng.uniform(-20, 20, (2, 3, 4)).astype(np.float32)
    flat = O.argsort(a)
    assert flat.dtype == np.int32 and np.all(np.diff(a.reshape(-1)[flat]) >= 0)
    for axis in range(3):
        idx = O.argsort(a, axis)
        assert idx.shape == a.shape and np.all(np.diff(np.take_along_axis(a, idx, axis), axis=axis) >= 0)
    assert O.k_best(np.array([[7.0]]), 3, True).tolist() == [[0]]  # one element: zeros of the input's shape (top_k.cpp:202-204)
