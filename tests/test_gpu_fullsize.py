"""The five benchmark configurations at their full sizes (BASELINE.json), checked
through size-independent properties plus oracle comparisons on slices the CPU
finishes in seconds."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def arr(D, x):
    return D.Array.from_numpy(x)


def test_c1_softmax_4096x1024(gpu, D, O):
    rng = np.random.RandomState(1)
    x = rng.randn(4096, 1024).astype(np.float32)
    s = D.op.softmax(arr(D, x)).numpy()
    np.testing.assert_allclose(s, O.softmax(x), rtol=1e-5, atol=1e-10)
    np.testing.assert_allclose(s.astype(np.float64).sum(1), 1.0, atol=2e-6)
    assert np.array_equal(s.argmax(1), x.argmax(1))


def test_c2_chain_67m(gpu, D, O):
    n = 67108864
    rs = [np.random.RandomState(seed) for seed in (2, 3, 4, 5)]
    a, b, c, d = (r.uniform(-4, 4, n).astype(np.float32) for r in rs)
    op = D.op
    A = arr(D, a)
    y = (op.sigmoid(A) * op.tanh(arr(D, b)) + arr(D, c) * arr(D, d) - 0.5 * op.square(A)).numpy()
    assert D.last_kernel_kinds() == "flat"
    # oracle on the head, the tail and a strided sample
    for sl in (slice(0, 1 << 20), slice(n - (1 << 20), n), slice(12345, n, 997)):
        want = O.chain(a[sl], b[sl], c[sl], d[sl])
        scale = np.abs(np.tanh(b[sl])) + np.abs(c[sl] * d[sl]) + 0.5 * a[sl] * a[sl]
        assert np.all(np.abs(y[sl] - want) <= 1e-5 * scale + 1e-6)
    # linearity in (c, d): y(c, d) - y(0, d) == c*d wherever the sum is exact enough
    assert np.isfinite(y).all()


def test_c3_reductions_8192x8192(gpu, D, O):
    rng = np.random.RandomState(6)
    x = rng.randn(8192, 8192).astype(np.float32)
    X = arr(D, x)
    op = D.op
    x64 = x.astype(np.float64)
    tol1, tol0 = 1e-5 * np.abs(x64).sum(1), 1e-5 * np.abs(x64).sum(0)
    s1, s0 = op.sum(X, [1]).numpy(), op.sum(X, [0]).numpy()
    assert np.all(np.abs(s1 - O.axis_reduce(O.SUM, x, 1)) <= tol1) and np.all(np.abs(s1 - x64.sum(1)) <= tol1)
    assert np.all(np.abs(s0 - O.axis_reduce(O.SUM, x, 0)) <= tol0) and np.all(np.abs(s0 - x64.sum(0)) <= tol0)
    assert np.array_equal(op.max(X, [1]).numpy(), x.max(1)) and np.array_equal(op.max(X, [0]).numpy(), x.max(0))
    total = float(op.sum(X).numpy())
    assert abs(total - x64.sum()) <= 1e-5 * np.abs(x64).sum() and abs(total - float(O.all_reduce(O.SUM, x))) <= 1e-5 * np.abs(x64).sum()
    assert float(op.max(X).numpy()) == x.max()
    am = op.argmax(X, 1).numpy()
    assert am.dtype == np.int32 and np.array_equal(am, O.arg_axis_reduce(O.MAX, x, 1))
    # argmax with planted ties, both axes: the first index must win (all_reduce_kernel_utils.cpp:217-219)
    xt = x.copy()
    peak = np.float32(np.abs(x).max() + 1.0)
    for c in range(0, 8192, 97):
        xt[[5000 + c % 100, 17 + c % 50, 8191], c] = peak  # three equal maxima in column c
    for r in range(0, 8192, 89):
        xt[r, [8000, 3 + r % 64, 4096]] = peak + 1.0
    XT = arr(D, xt)
    a0, a1 = op.argmax(XT, 0).numpy(), op.argmax(XT, 1).numpy()
    assert a0.dtype == np.int32 and np.array_equal(a0, xt.argmax(0)) and np.array_equal(a1, xt.argmax(1))
    assert np.array_equal(a0, O.arg_axis_reduce(O.MAX, xt, 0))
    assert np.array_equal(op.argmin(XT, 0).numpy(), xt.argmin(0))
    # checksum of checksums: the row sums and the column sums add up to the same total
    assert abs(s1.astype(np.float64).sum() - s0.astype(np.float64).sum()) <= 1e-5 * np.abs(x64).sum()


def test_c4_cross_entropy_8192x32000(gpu, D, O):
    rows, vocab = 8192, 32000
    x = (np.random.RandomState(7).randn(rows, vocab) * 2).astype(np.float32)
    t = np.random.RandomState(8).randint(0, vocab, rows).astype(np.int32)
    k0 = D.jit_stats()["kernels"]
    mean, rl, grad = D.op.softmax_cross_entropy(arr(D, x), arr(D, t))
    assert D.jit_stats()["kernels"] - k0 == 1  # logits are read once: gradient, row losses and the mean loss leave one launch
    g, r = grad.numpy(), rl.numpy()
    sel = np.r_[0:64, rows // 2:rows // 2 + 64, rows - 64:rows]
    _, orows, ograd = O.softmax_cross_entropy(x[sel], t[sel])
    # The checker sums 32000 terms left to right in fp32 and loses small terms to the running sum. Measured on an MI355X
    # over 768 rows of this input: row losses differ by at most 8.3e-7 relative (9.5e-6 absolute), gradient entries by at
    # most 1.0e-5 relative. The bounds are four times that (the checker's a-priori bound n * 2^-24 = 1.9e-3 is 190 times it).
    np.testing.assert_allclose(r[sel], orows, rtol=3.5e-6, atol=0)
    np.testing.assert_allclose(g[sel], ograd, rtol=4e-5, atol=1e-8)
    x64 = x[sel].astype(np.float64)
    lse = np.log(np.exp(x64 - x64.max(1, keepdims=True)).sum(1)) + x64.max(1)
    np.testing.assert_allclose(r[sel], lse - x64[np.arange(len(sel)), t[sel]], rtol=1e-5, atol=2e-6)  # fp64 truth, plain 1e-5
    sm = np.exp(x64 - lse[:, None])
    sm[np.arange(len(sel)), t[sel]] -= 1.0
    np.testing.assert_allclose(g[sel], sm, rtol=1e-5, atol=1e-8)
    assert abs(float(mean.numpy()) - r.astype(np.float64).mean()) <= 1e-5 * r.astype(np.float64).mean()
    assert np.all(r > 0)
    assert np.abs(g.astype(np.float64).sum(1)).max() <= 1e-4  # softmax - onehot sums to zero in every row
    picked = g[np.arange(rows), t]
    assert np.all(picked < 0) and np.all(picked >= -1)
    # softmax[i, t_i] = 1 + grad[i, t_i] = exp(-loss_i), to the spacing of floats next to -1
    assert np.abs((1.0 + picked.astype(np.float64)) - np.exp(-r.astype(np.float64))).max() <= 1.3e-7


def test_c5_lstm_step_256x1024x1024(gpu, D, O):
    B, I, H = 256, 1024, 1024
    X, Hp, Cp = (np.random.RandomState(s).randn(B, n).astype(np.float32) for s, n in ((9, I), (10, H), (11, H)))
    lim = np.sqrt(6.0 / (1024 + 4096))
    W, U = (np.random.RandomState(s).uniform(-lim, lim, (1024, 4096)).astype(np.float32) for s in (12, 13))
    b = np.zeros(4096, np.float32)
    cn, hn = D.op.lstm_step(*(arr(D, v) for v in (X, Hp, Cp, W, U, b)))
    G = X.astype(np.float64) @ W + Hp.astype(np.float64) @ U  # fp64 truth for the two products
    pre = (D.op.dot(arr(D, X), arr(D, W)) + D.op.dot(arr(D, Hp), arr(D, U))).numpy()
    assert np.abs(pre - G).max() <= 1e-4 * np.abs(G).max()
    sig = lambda z: 1.0 / (1.0 + np.exp(-z))
    c = sig(G[:, H:2 * H]) * Cp + sig(G[:, :H]) * np.tanh(G[:, 3 * H:])
    h = sig(G[:, 2 * H:3 * H]) * np.tanh(c)
    np.testing.assert_allclose(cn.numpy(), c, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(hn.numpy(), h, rtol=1e-4, atol=1e-5)
    # and the gate arithmetic alone against the oracle, fed the GPU's own pre-activations
    gf = pre.astype(np.float32)
    oc = O.binary("add", O.binary("eltmul", O.unary("sigmoid", gf[:, H:2 * H]), Cp), O.binary("eltmul", O.unary("sigmoid", gf[:, :H]), O.unary("tanh", gf[:, 3 * H:])))
    np.testing.assert_allclose(cn.numpy(), oc.reshape(B, H), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("shape,axis", [((64, 1 << 20), 1), ((3, 1 << 22), 1), ((2, 5, 1 << 18), 2), ((1 << 20, 64), 0), ((1 << 22, 8), 0),
                                        ((65536, 100), 0), ((100, 100000), 1)])
def test_reductions_of_starved_shapes_take_two_passes(gpu, D, rng, shape, axis):
    """Few long rows and the leading axis of a narrow matrix: reshaped two-stage reductions, same results."""
    x = rng.uniform(-1.0, 1.0, shape).astype(np.float32)
    a = D.Array.from_numpy(x)
    n_red = shape[axis]
    for name, f in (("sum", np.sum), ("max", np.max), ("min", np.min)):
        before = D.jit_stats()["kernels"]
        got = getattr(D.op, name)(a, [axis]).numpy()
        launched = D.jit_stats()["kernels"] - before
        want = f(x.astype(np.float64), axis=axis)
        assert got.shape == want.shape
        if name == "sum":
            bound = 1e-5 * np.abs(x.astype(np.float64)).sum(axis=axis) + 1e-6
            assert (np.abs(got - want) <= bound).all()
        else:
            assert np.array_equal(got, want.astype(np.float32))
        if shape not in ((100, 100000),):
            assert launched == 2, (name, launched)
    # accumulate into an existing destination: only the second pass applies the operator
    acc = D.Array.from_numpy(np.ones(got.shape, np.float32))
    acc += D.op.max(a, [axis])
    assert np.array_equal(acc.numpy(), 1.0 + x.max(axis=axis))
    assert n_red > 0


def test_leading_axis_reduction_of_a_very_wide_matrix(gpu, D, rng):
    """More 256-column strips than the workspace has tickets: the reduced rows are then not split across workgroups."""
    x = rng.uniform(-1.0, 1.0, (3, (1 << 23) + 12)).astype(np.float32)
    a = D.Array.from_numpy(x)
    np.testing.assert_allclose(D.op.sum(a, [0]).numpy(), x.astype(np.float64).sum(axis=0), rtol=1e-6, atol=1e-6)
    assert np.array_equal(D.op.max(a, [0]).numpy(), x.max(axis=0))
    assert np.array_equal(D.op.argmax(a, 0).numpy(), x.argmax(axis=0).astype(np.int32))


def test_top_k_over_the_cross_entropy_logits_shape(gpu, D, O):
    """The 8 largest and the 8 smallest of 32000 scores in each of 8192 rows (the selection kernel at full width): the
    values at the returned positions are the row's extremes in order, the positions are distinct, and the first rows
    agree with the checker position for position."""
    rng = np.random.RandomState(21)
    x = (rng.randn(8192, 32000) * 2).astype(np.float32)
    X = arr(D, x)
    top = D.op.top_k(X, 8).numpy()
    bottom = D.op.bottom_k(X, 8).numpy()
    assert top.shape == bottom.shape == (8192, 8) and top.dtype == np.int32
    part = np.partition(x, (8, 31991), axis=1)
    want_top = np.sort(part[:, 31992:], axis=1)[:, ::-1]
    want_bottom = np.sort(part[:, :8], axis=1)
    assert np.array_equal(np.take_along_axis(x, top.astype(np.int64), 1), want_top)
    assert np.array_equal(np.take_along_axis(x, bottom.astype(np.int64), 1), want_bottom)
    assert all(len(set(r)) == 8 for r in top[::64].tolist()) and all(len(set(r)) == 8 for r in bottom[::64].tolist())
    assert np.array_equal(top[:16], O.k_best(x[:16], 8, True)) and np.array_equal(bottom[:16], O.k_best(x[:16], 8, False))
    assert np.array_equal(top[:, 0], D.op.argmax(X, 1).numpy())
