"""Parity of the sliding-window operators (im2col, col2im, conv2d and its gradients, pool2d and its gradient)
against the CPU checker, on a real MI355X, through the front-end and the C ABI underneath it.

im2col, col2im and the pooling pair move or add values in the reference's order: bit-exact. conv2d adds a matrix
product: rel 1e-4 of max|out| against the checker's fp64-accumulated product, exact on the integer-valued tables.
"""
import numpy as np
import pytest

from conftest import golden

import ctypes as C

pytestmark = pytest.mark.gpu


def arr(D, x):
    return D.Array.from_numpy(np.ascontiguousarray(x))


@pytest.mark.parametrize("fmt,shape", [("NHWC", (3, 9, 11, 8)), ("NHWC", (2, 7, 6, 3)), ("NCHW", (3, 5, 9, 11)), ("WNCH", (11, 2, 3, 9)),
                                       ("CNHW", (4, 2, 9, 7))])
def test_im2col_matches_oracle(gpu, D, O, rng, fmt, shape):
    x = rng.uniform(-1, 1, shape).astype(np.float32)
    for fh, fw, sh, sw, pads in ((3, 3, 1, 1, (0, 0, 0, 0)), (2, 3, 2, 1, (1, 0, 1, 2)), (3, 2, 2, 3, (1, 1, 2, 1)), (1, 1, 1, 1, (0, 0, 0, 0))):
        got = D.op.im2col(arr(D, x), fh, fw, sh, sw, *pads, data_format=fmt)
        want = O.im2col(x, fh, fw, sh, sw, *pads, data_format=fmt)
        assert got.shape == want.shape
        assert np.array_equal(got.numpy(), want)


def test_im2col_reference_cases(gpu, D, O):
    # JITTests.im2col_without_channels (im2col_tests.cpp:41-72): int32 arange image, the three layouts agree
    nchw = np.arange(24, dtype=np.int32).reshape(2, 1, 3, 4)
    want = O.im2col(nchw.astype(np.float32), 3, 3, 1, 1, data_format="NCHW").astype(np.int32)
    a = D.op.im2col(arr(D, nchw), 3, 3, 1, 1, data_format="NCHW")
    assert a.numpy().dtype == np.int32 and np.array_equal(a.numpy(), want)
    b = D.op.im2col(arr(D, nchw).transpose([0, 2, 3, 1]), 3, 3, 1, 1, data_format="NHWC")
    assert np.array_equal(b.numpy(), want)
    c = D.op.im2col(arr(D, nchw).transpose([3, 0, 1, 2]), 3, 3, 1, 1, data_format="WNCH")
    assert np.array_equal(c.numpy().reshape(3, 1, 3, -1).transpose(1, 2, 0, 3).reshape(9, -1), want)
    # a 3-D image is a batch of one
    img = np.arange(60, dtype=np.float32).reshape(3, 4, 5)
    got = D.op.im2col(arr(D, img), 2, 2, 1, 1, data_format="NCHW").numpy()
    assert np.array_equal(got, O.im2col(img[None], 2, 2, 1, 1, data_format="NCHW"))
    with pytest.raises(Exception):
        D.op.im2col(arr(D, img), 5, 2, 1, 1, data_format="NCHW")  # filter taller than the image
    with pytest.raises(Exception):
        D.op.im2col(arr(D, img), 2, 2, 1, 1, data_format="NCHX")


@pytest.mark.parametrize("fmt,perm", [("NCHW", (0, 1, 2, 3)), ("NHWC", (0, 2, 3, 1))])
def test_col2im_matches_oracle(gpu, D, O, rng, fmt, perm):
    for fh, fw, sh, sw in ((3, 3, 1, 1), (2, 3, 2, 1), (2, 2, 2, 2), (3, 2, 2, 3), (1, 1, 1, 1)):
        shape = tuple(int(v) for v in np.array((2, 4, 7, 8))[list(perm)])
        x = rng.uniform(-1, 1, shape).astype(np.float32)
        px = O.im2col(x, fh, fw, sh, sw, data_format=fmt)
        y = rng.uniform(-1, 1, px.shape).astype(np.float32)
        want = O.col2im(y, shape, fh, fw, sh, sw, fmt)
        assert np.array_equal(D.op.col2im(arr(D, y), shape, fh, fw, sh, sw, fmt).numpy(), want)
        # the same matrix handed over as a transposed view of its patch-major copy
        yt = arr(D, np.ascontiguousarray(y.T)).transpose()
        assert np.array_equal(D.op.col2im(yt, shape, fh, fw, sh, sw, fmt).numpy(), want)
        # composed on the device: col2im(im2col(x)) = x * (number of windows over each pixel)
        count = O.col2im(np.ones_like(px), shape, fh, fw, sh, sw, fmt)
        round_trip = D.op.col2im(D.op.im2col(arr(D, x), fh, fw, sh, sw, data_format=fmt), shape, fh, fw, sh, sw, fmt).numpy()
        assert np.array_equal(round_trip, O.col2im(px, shape, fh, fw, sh, sw, fmt))
        np.testing.assert_allclose(round_trip, x * count, rtol=1e-6, atol=1e-6)
    with pytest.raises(Exception):
        D.op.col2im(arr(D, np.zeros((5, 5), np.float32)), (2, 4, 7, 8), 3, 3, 1, 1, fmt)


def test_conv2d_tensorflow_tables(gpu, D):
    # ConvTests.reference_valid_padding_conv2d / reference_same_padding_conv2d (conv_tests.cpp:132-216)
    g = golden("reference_known_answers.json")["conv2d_tensorflow"]
    image = np.arange(2 * 3 * 7 * 5, dtype=np.float32).reshape(2, 3, 7, 5)
    filters = np.arange(4 * 3 * 6 * 5, dtype=np.float32).reshape(3, 6, 5, 4).transpose(3, 0, 1, 2)
    valid = D.op.conv2d(arr(D, image), arr(D, filters), 1, 1, "valid", "NHWC")
    assert valid.shape == (2, 1, 2, 4) and np.array_equal(valid.numpy().ravel(), np.array(g["valid"], np.float32))
    same = D.op.conv2d(arr(D, image), arr(D, filters), 1, 1, "same", "NHWC")
    assert same.shape == (2, 3, 7, 4) and np.array_equal(same.numpy().ravel(), np.array(g["same"], np.float32))
    # the same convolution in NCHW
    same_c = D.op.conv2d(arr(D, image.transpose(0, 3, 1, 2)), arr(D, filters.transpose(0, 3, 1, 2)), 1, 1, "same", "NCHW")
    assert same_c.shape == (2, 4, 3, 7) and np.array_equal(same_c.numpy().transpose(0, 2, 3, 1).ravel(), np.array(g["same"], np.float32))


@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_conv2d_forward_matches_oracle(gpu, D, O, rng, fmt):
    # ConvTests.conv2d_forward (conv_tests.cpp:348-410): strides 1..3, both paddings
    for sh in (1, 2, 3):
        for sw in (1, 2, 3):
            for padding in ("valid", "same"):
                x = rng.uniform(-1, 1, (5, 3, 6, 8)).astype(np.float32)
                w = rng.uniform(-1, 1, (2, 3, 2, 4)).astype(np.float32)
                if fmt == "NHWC":
                    x, w = np.ascontiguousarray(x.transpose(0, 2, 3, 1)), np.ascontiguousarray(w.transpose(0, 2, 3, 1))
                want = O.conv2d(x, w, sh, sw, padding, fmt)
                got = D.op.conv2d(arr(D, x), arr(D, w), sh, sw, padding, fmt)
                assert got.shape == want.shape
                assert np.abs(got.numpy() - want).max() <= 1e-4 * np.abs(want).max()
    # a layer-sized case: 64 -> 128 channels, 3x3, 28x28 images
    x = rng.uniform(-1, 1, (8, 64, 28, 28)).astype(np.float32)
    w = rng.uniform(-1, 1, (128, 64, 3, 3)).astype(np.float32)
    if fmt == "NHWC":
        x, w = np.ascontiguousarray(x.transpose(0, 2, 3, 1)), np.ascontiguousarray(w.transpose(0, 2, 3, 1))
    want = O.conv2d(x, w, 1, 1, "same", fmt)
    got = D.op.conv2d(arr(D, x), arr(D, w), 1, 1, "same", fmt).numpy()
    assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()


@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_conv2d_gradients_are_adjoints(gpu, D, O, rng, fmt):
    # integer-valued operands: every product and partial sum is exact, so the three bilinear forms agree exactly
    for sh, sw, fh, fw in ((1, 1, 3, 3), (2, 2, 2, 2), (2, 1, 2, 3)):
        x = rng.randint(-3, 4, (2, 3, 8, 9)).astype(np.float32)
        w = rng.randint(-3, 4, (4, 3, fh, fw)).astype(np.float32)
        if (8 - fh) % sh or (9 - fw) % sw:
            x = x[:, :, :8 - (8 - fh) % sh, :9 - (9 - fw) % sw]
        if fmt == "NHWC":
            x, w = np.ascontiguousarray(x.transpose(0, 2, 3, 1)), np.ascontiguousarray(w.transpose(0, 2, 3, 1))
        y = D.op.conv2d(arr(D, x), arr(D, w), sh, sw, "valid", fmt).numpy()
        assert np.array_equal(y, O.conv2d(x, w, sh, sw, "valid", fmt))
        dy = rng.randint(-3, 4, y.shape).astype(np.float32)
        dx = D.op.conv2d_backward_input(arr(D, w), arr(D, dy), sh, sw, x.shape, "valid", fmt)
        dw = D.op.conv2d_backward_filters(arr(D, x), arr(D, dy), sh, sw, w.shape, "valid", fmt)
        assert dx.shape == x.shape and dw.shape == w.shape
        lhs = float((y.astype(np.float64) * dy).sum())
        assert float((dx.numpy().astype(np.float64) * x).sum()) == lhs
        assert float((dw.numpy().astype(np.float64) * w).sum()) == lhs
        # and element by element against the checker's composition of the same steps (conv.cpp:278-393)
        n_dim, c_dim = fmt.index("N"), fmt.index("C")
        w2 = w.reshape(w.shape[0], -1)
        dy2 = np.ascontiguousarray(np.moveaxis(dy, c_dim, 0)).reshape(w.shape[0], -1)
        assert np.array_equal(dx.numpy(), O.col2im(O.gemm(np.ascontiguousarray(w2.T), dy2), x.shape, fh, fw, sh, sw, fmt))
        assert np.array_equal(dw.numpy(), O.gemm(dy2, np.ascontiguousarray(O.im2col(x, fh, fw, sh, sw, data_format=fmt).T)).reshape(w.shape))
    # ConvTests.conv_backward_bias (conv_tests.cpp:641-652)
    bias = D.op.conv2d_backward_bias(arr(D, np.ones((2, 3, 4, 5), np.float32)), "NCHW").numpy()
    assert bias.tolist() == [40.0, 40.0, 40.0]


@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_pool2d_pair_matches_oracle(gpu, D, O, rng, fmt):
    # the loops of ConvTests.pool2d_forward / unpool2d_forward (conv_tests.cpp:584-760)
    # (every window / stride pair is a kernel of its own to compile: a cross-section of the reference's 3 x 3 x 4 grid)
    for wh, ww in ((1, 1), (2, 3), (3, 2), (3, 3)):
        if True:
            for sh, sw in ((1, 1), (1, 2), (2, 2)):
                for padding in ("valid", "same"):
                    for mode in ("max", "avg"):
                        x = rng.uniform(-1, 1, (5, 3, 6, 8) if fmt == "NCHW" else (5, 6, 8, 3)).astype(np.float32)
                        want = O.pool2d(x, wh, ww, sh, sw, mode, padding, fmt)
                        xa = arr(D, x)
                        y = D.op.pool2d(xa, wh, ww, sh, sw, mode, padding, fmt)
                        assert y.shape == want.shape and np.array_equal(y.numpy(), want)
                        dy = rng.uniform(-1, 1, want.shape).astype(np.float32)
                        dx = D.op.pool2d_backward(y, arr(D, dy), xa, wh, ww, sh, sw, mode, padding, fmt)
                        assert np.array_equal(dx.numpy(), O.pool2d_backward(want, dy, x, wh, ww, sh, sw, mode, padding, fmt))
    # ties: every element of a window equal to its maximum receives the gradient (reducer_kernels.h:107-109)
    x = np.ones((1, 1, 4, 4) if fmt == "NCHW" else (1, 4, 4, 1), np.float32)
    y = D.op.pool2d(arr(D, x), 2, 2, 2, 2, "max", "valid", fmt)
    dx = D.op.pool2d_backward(y, arr(D, np.full(y.shape, 3.0, np.float32)), arr(D, x), 2, 2, 2, 2, "max", "valid", fmt).numpy()
    assert np.array_equal(dx, np.full(x.shape, 3.0, np.float32))
    # a layer-sized case
    x = rng.uniform(-1, 1, (16, 64, 56, 56) if fmt == "NCHW" else (16, 56, 56, 64)).astype(np.float32)
    assert np.array_equal(D.op.pool2d(arr(D, x), 3, 3, 2, 2, "max", "same", fmt).numpy(), O.pool2d(x, 3, 3, 2, 2, "max", "same", fmt))
    with pytest.raises(Exception):
        D.op.pool2d(arr(D, x), 2, 2, 2, 2, "max", "valid", "CHWN")


def test_sgemm_terms_is_a_convolution_over_overlapping_rows(gpu, rng):
    """dali_hip_sgemm_terms through the C ABI: filter rows as terms over a padded channels-last image whose pixel rows
    overlap (lda = C < K), every padded position computed, the row map keeping the valid ones."""
    hip = gpu
    N, Hp, Wp, Cc, O, fh, fw = 3, 9, 11, 8, 12, 3, 2
    oh, ow = Hp - fh + 1, Wp - fw + 1
    slack = (fh - 1) * Wp + fw
    xp = np.zeros((N * Hp * Wp + slack, Cc), np.float32)
    xp[:N * Hp * Wp] = rng.randint(-3, 4, (N * Hp * Wp, Cc))
    f = rng.randint(-3, 4, (O, fh, fw, Cc)).astype(np.float32)

    def dev(a):
        p = C.c_void_p()
        assert hip.dali_hip_malloc(C.byref(p), a.nbytes) == 0
        assert hip.dali_hip_memcpy_h2d(p, a.ctypes.data_as(C.c_void_p), a.nbytes) == 0
        return p

    dx, df = dev(xp), dev(f)
    out = np.full((N, oh, ow, O), 7.0, np.float32)
    dout = dev(out)
    K = (C.c_int * fh)(*[fw * Cc] * fh)
    As = (C.c_void_p * fh)(*[dx.value + t * Wp * Cc * 4 for t in range(fh)])
    Bs = (C.c_void_p * fh)(*[df.value + t * fw * Cc * 4 for t in range(fh)])
    row_map = (C.c_int * 4)(Hp, Wp, oh, ow)
    st = hip.dali_hip_sgemm_terms(fh, 0, 1, N * Hp * Wp, O, K, As, Cc, Bs, fh * fw * Cc, 1.0, 0.0, dout, O, row_map)
    assert st == 0, hip.dali_hip_last_error()
    assert hip.dali_hip_memcpy_d2h(out.ctypes.data_as(C.c_void_p), dout, out.nbytes) == 0
    img = xp[:N * Hp * Wp].reshape(N, Hp, Wp, Cc).astype(np.float64)
    want = np.zeros((N, oh, ow, O))
    for i in range(oh):
        for j in range(ow):
            want[:, i, j, :] = np.einsum("nhwc,ohwc->no", img[:, i:i + fh, j:j + fw, :], f.astype(np.float64))
    assert np.array_equal(out, want)  # small integers: exact
    # without the map every padded position is stored, the valid ones in place
    full = np.zeros((N * Hp * Wp, O), np.float32)
    dfull = dev(full)
    assert hip.dali_hip_sgemm_terms(fh, 0, 1, N * Hp * Wp, O, K, As, Cc, Bs, fh * fw * Cc, 1.0, 0.0, dfull, O, None) == 0
    assert hip.dali_hip_memcpy_d2h(full.ctypes.data_as(C.c_void_p), dfull, full.nbytes) == 0
    assert np.array_equal(full.reshape(N, Hp, Wp, O)[:, :oh, :ow, :], want)
    bad = (C.c_int * 4)(Hp, Wp, Hp + 1, ow)
    assert hip.dali_hip_sgemm_terms(fh, 0, 1, N * Hp * Wp, O, K, As, Cc, Bs, fh * fw * Cc, 1.0, 0.0, dout, O, bad) != 0
    for p in (dx, df, dout, dfull):
        hip.dali_hip_free(p)


def test_conv2d_nhwc_direct_path_equals_the_two_step_form(gpu, D, O, rng):
    """Channels-last, stride 1: one padding copy + a multi-term product. Same numbers as im2col + one product on
    integer-valued data, and one kernel plus one product instead of a patch matrix."""
    for padding in ("valid", "same"):
        for fh, fw in ((3, 3), (1, 1), (5, 2), (2, 7)):
            x = rng.randint(-3, 4, (4, 12, 10, 8)).astype(np.float32)
            w = rng.randint(-3, 4, (16, fh, fw, 8)).astype(np.float32)
            before = D.jit_stats()
            y = D.op.conv2d(arr(D, x), arr(D, w), 1, 1, padding, "NHWC")
            got = y.numpy()
            after = D.jit_stats()
            assert "pad" in D.last_kernel_kinds() and after["gemms"] - before["gemms"] == 1
            assert np.array_equal(got, O.conv2d(x, w, 1, 1, padding, "NHWC"))
    # channel counts that are not multiples of 4 keep the patch-matrix form
    x = rng.randint(-3, 4, (2, 6, 7, 3)).astype(np.float32)
    w = rng.randint(-3, 4, (5, 3, 3, 3)).astype(np.float32)
    assert np.array_equal(D.op.conv2d(arr(D, x), arr(D, w), 1, 1, "same", "NHWC").numpy(), O.conv2d(x, w, 1, 1, "same", "NHWC"))
    assert "im2col" in D.last_kernel_kinds() or D.jit_stats()["gemms"] > 0


@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_sliding_windows_in_double_and_int32(gpu, D, O, rng, fmt):
    """The kernels are generated per dtype: fp64 agrees with the fp32 checker on values that are exact in both,
    int32 pooling takes the maximum / the truncating integer average of the reference's `res / area` with T = int."""
    shape = (2, 3, 6, 8) if fmt == "NCHW" else (2, 6, 8, 3)
    xi = rng.randint(-20, 21, shape).astype(np.int32)
    for dtype in (np.float64, np.int32):
        x = xi.astype(dtype)
        y = D.op.pool2d(arr(D, x), 2, 3, 2, 1, "max", "same", fmt)
        want = O.pool2d(xi.astype(np.float32), 2, 3, 2, 1, "max", "same", fmt)
        assert y.numpy().dtype == dtype and np.array_equal(y.numpy(), want.astype(dtype))
        p = D.op.im2col(arr(D, x), 2, 2, 1, 2, 1, 0, 0, 1, data_format=fmt)
        assert np.array_equal(p.numpy(), O.im2col(xi.astype(np.float32), 2, 2, 1, 2, 1, 0, 0, 1, data_format=fmt).astype(dtype))
        back = D.op.col2im(D.op.im2col(arr(D, x), 2, 2, 2, 2, data_format=fmt), shape, 2, 2, 2, 2, fmt)
        assert np.array_equal(back.numpy(), x)  # windows that tile the image exactly: every pixel once
    # sums of integers in fp64 and their division by the window area; the int32 average truncates towards zero
    sums = O.pool2d(xi.astype(np.float32), 2, 2, 2, 2, "avg", "valid", fmt).astype(np.float64) * 4.0
    got = D.op.pool2d(arr(D, xi.astype(np.float64)), 2, 2, 2, 2, "avg", "valid", fmt).numpy()
    assert np.array_equal(got, sums / 4.0)
    goti = D.op.pool2d(arr(D, xi), 2, 2, 2, 2, "avg", "valid", fmt).numpy()
    assert np.array_equal(goti, np.trunc(sums / 4.0).astype(np.int32))
    dy = rng.randint(-5, 6, got.shape).astype(np.float64)
    dx = D.op.pool2d_backward(arr(D, got), arr(D, dy), arr(D, xi.astype(np.float64)), 2, 2, 2, 2, "avg", "valid", fmt).numpy()
    want_dx = O.pool2d_backward(got.astype(np.float32), dy.astype(np.float32), xi.astype(np.float32), 2, 2, 2, 2, "avg", "valid", fmt)
    assert np.array_equal(dx, want_dx.astype(np.float64))
