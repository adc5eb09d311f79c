"""The CPU oracle's convolution and pooling against the reference's golden
vectors, against scipy's and numpy's own routines, and the shape rules against
the reference's tables of valid and invalid arguments."""
import numpy as np
import pytest
from scipy import signal

import oracle
from conv_pool_cases import CASES, case_id, run_case_on, vgg_conv_case, vgg_pool_case
from util import vector_match


@pytest.mark.parametrize("kc", CASES, ids=case_id)
def test_oracle_matches_reference_vectors(kc):
    for want, got in run_case_on(oracle, *kc):
        assert vector_match(want, got), kc[1]["source"]


def test_oracle_vgg16_first_layer():
    c = vgg_conv_case()
    y = oracle.conv2d_fw(c["x"], c["w"], c["x_dims"], 1, c["w_dims"], 1, *c["args"])
    assert np.array_equal(y, c["y"])
    gx, gw = oracle.conv2d_bw(c["x"], c["w"], np.ones_like(y), np.ones_like(c["x"]), np.ones_like(c["w"]),
                              c["x_dims"], 1, c["w_dims"], 1, *c["args"])
    assert np.array_equal(gx, c["gx"]) and np.array_equal(gw, c["gw"])


def test_oracle_vgg16_third_layer_pooling():
    c = vgg_pool_case()
    y = oracle.max_pool2d_fw(c["x"], c["x_dims"], 1, *c["args"])
    assert np.array_equal(y, c["y"])
    gx = oracle.max_pool2d_bw(c["x"], y, np.ones_like(y), np.ones_like(c["x"]), c["x_dims"], 1, *c["args"])
    assert np.array_equal(gx, c["gx"])


def planes(v, dims):
    """Flat primitiv array -> [..., d1, d0] numpy array (dimension 0 fastest)."""
    return np.asarray(v, np.float64).reshape(list(dims)[::-1])


@pytest.mark.parametrize("h,w,c,kh,kw,oc", [(7, 6, 1, 3, 2, 1), (9, 8, 3, 3, 3, 4), (5, 11, 2, 5, 1, 3)])
def test_forward_is_scipys_convolution(h, w, c, kh, kw, oc):
    # stride 1, no padding, no dilation: y[oc] = sum_c convolve2d(x[c], w[oc][c], 'valid')
    rng = np.random.default_rng(h * w + c)
    x = rng.standard_normal(h * w * c).astype(np.float32)
    k = rng.standard_normal(kh * kw * c * oc).astype(np.float32)
    got = planes(oracle.conv2d_fw(x, k, [h, w, c], 1, [kh, kw, c, oc], 1, 0, 0, 1, 1, 1, 1), [h - kh + 1, w - kw + 1, oc])
    X, K = planes(x, [h, w, c]), planes(k, [kh, kw, c, oc])
    for o in range(oc):
        want = sum(signal.convolve2d(X[ch], K[o, ch], mode="valid") for ch in range(c))
        assert np.allclose(got[o], want, rtol=1e-5, atol=1e-5)
    # 'full' convolution is padding kernel - 1
    got = planes(oracle.conv2d_fw(x, k, [h, w, c], 1, [kh, kw, c, oc], 1, kh - 1, kw - 1, 1, 1, 1, 1),
                 [h + kh - 1, w + kw - 1, oc])
    for o in range(oc):
        want = sum(signal.convolve2d(X[ch], K[o, ch], mode="full") for ch in range(c))
        assert np.allclose(got[o], want, rtol=1e-5, atol=1e-5)


def test_stride_and_dilation_subsample_the_dense_result():
    rng = np.random.default_rng(4)
    h, w, kh, kw = 13, 12, 3, 2
    x = rng.standard_normal(h * w).astype(np.float32)
    k = rng.standard_normal(kh * kw).astype(np.float32)
    dense = planes(oracle.conv2d_fw(x, k, [h, w], 1, [kh, kw], 1, 1, 2, 1, 1, 1, 1), [h + 2 - kh + 1, w + 4 - kw + 1])
    strided = planes(oracle.conv2d_fw(x, k, [h, w], 1, [kh, kw], 1, 1, 2, 3, 2, 1, 1),
                     [(h + 2 - kh) // 3 + 1, (w + 4 - kw) // 2 + 1])
    assert np.array_equal(strided, dense[::2, ::3])
    # a dilated kernel is the kernel with zeros between its elements
    dil = np.zeros((3, 5), np.float32)                  # [(kw-1)*2+1][(kh-1)*2+1], dimension 0 fastest
    dil[::2, ::2] = k.reshape(kw, kh)
    a = oracle.conv2d_fw(x, k, [h, w], 1, [kh, kw], 1, 0, 0, 1, 1, 2, 2)
    b = oracle.conv2d_fw(x, dil.reshape(-1), [h, w], 1, [5, 3], 1, 0, 0, 1, 1, 1, 1)
    assert np.allclose(a, b, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("bx,bw", [(1, 1), (3, 1), (1, 3), (3, 3)])
def test_backward_is_the_gradient_of_forward(bx, bw):
    # <gy, conv(x + dx, w + dw) - conv(x, w)> = <gx, dx> + <gw, dw> + second order, and conv is bilinear:
    # check the two linear parts exactly (up to rounding) with dw = 0 and dx = 0
    rng = np.random.default_rng(10 * bx + bw)
    xd, wd, a = [6, 5, 2], [3, 2, 2, 3], (1, 0, 2, 1, 1, 2)
    x = rng.standard_normal(60 * bx).astype(np.float32)
    w = rng.standard_normal(36 * bw).astype(np.float32)
    y = oracle.conv2d_fw(x, w, xd, bx, wd, bw, *a)
    gy = rng.standard_normal(y.size).astype(np.float32)
    gx, gw = oracle.conv2d_bw(x, w, gy, np.zeros_like(x), np.zeros_like(w), xd, bx, wd, bw, *a)
    dx = rng.standard_normal(x.size).astype(np.float32)
    dw = rng.standard_normal(w.size).astype(np.float32)
    lin_x = np.dot(gy.astype(np.float64), oracle.conv2d_fw(dx, w, xd, bx, wd, bw, *a))
    lin_w = np.dot(gy.astype(np.float64), oracle.conv2d_fw(x, dw, xd, bx, wd, bw, *a))
    assert np.isclose(lin_x, np.dot(gx.astype(np.float64), dx), rtol=1e-4, atol=1e-4)
    assert np.isclose(lin_w, np.dot(gw.astype(np.float64), dw), rtol=1e-4, atol=1e-4)


def test_pooling_is_numpys_window_maximum():
    rng = np.random.default_rng(8)
    h, w, c, bs = 9, 7, 2, 3
    x = rng.standard_normal(h * w * c * bs).astype(np.float32)
    win0, win1, pad0, pad1, s0, s1 = 3, 2, 1, 1, 2, 1
    got = oracle.max_pool2d_fw(x, [h, w, c], bs, win0, win1, pad0, pad1, s0, s1)
    X = np.full((bs * c, w + 2 * pad1, h + 2 * pad0), -np.inf)
    X[:, pad1:pad1 + w, pad0:pad0 + h] = x.reshape(bs * c, w, h)
    oh, ow = (h + 2 * pad0 - win0) // s0 + 1, (w + 2 * pad1 - win1) // s1 + 1
    want = np.empty((bs * c, ow, oh))
    for i in range(ow):
        for j in range(oh):
            want[:, i, j] = X[:, i * s1:i * s1 + win1, j * s0:j * s0 + win0].max(axis=(1, 2))
    assert np.array_equal(got, want.reshape(-1).astype(np.float32))
    # backward: every window's gradient lands on exactly one element, the first maximum in window order
    gy = rng.standard_normal(got.size).astype(np.float32)
    gx = oracle.max_pool2d_bw(x, got, gy, np.zeros_like(x), [h, w, c], bs, win0, win1, pad0, pad1, s0, s1)
    assert np.isclose(gx.sum(dtype=np.float64), gy.sum(dtype=np.float64), atol=1e-4)
    ties = np.float32([2, 2, 2, 2, 2, 2])                         # 3 x 2 plane of equal values
    g = oracle.max_pool2d_bw(ties, np.float32([2]), np.float32([5]), np.zeros(6, np.float32), [3, 2], 1, 3, 2, 0, 0, 1, 1)
    assert np.array_equal(g, np.float32([5, 0, 0, 0, 0, 0]))


# shape rules: test/shape_ops_test.cc CheckConv2D / CheckInvalidConv2D / CheckPool2D / CheckInvalidPool2D
def test_shape_rules():
    assert oracle.shape_conv2d([], 1, [], 1, 0, 0, 1, 1, 1, 1) == ([1, 1, 1], 1)
    assert oracle.shape_conv2d([5, 5, 3], 4, [2, 2, 3, 7], 1, 1, 1, 2, 2, 1, 1) == ([3, 3, 7], 4)
    assert oracle.shape_conv2d([5, 5], 1, [2, 2], 3, 0, 0, 1, 1, 2, 2) == ([3, 3, 1], 3)
    for bad in (([2], 1, [3], 1, 0, 0, 1, 1, 1, 1),            # kernel larger than the image
                ([5, 5, 2], 1, [2, 2, 3], 1, 0, 0, 1, 1, 1, 1),  # channels differ
                ([5, 5], 2, [2, 2], 3, 0, 0, 1, 1, 1, 1),        # minibatches differ
                ([5, 5], 1, [2, 2], 1, 0, 0, 0, 1, 1, 1),        # zero stride
                ([5, 5], 1, [2, 2], 1, 0, 0, 1, 1, 1, 0),        # zero dilation
                ([5, 5, 1, 2], 1, [2, 2], 1, 0, 0, 1, 1, 1, 1)):  # x deeper than 3
        with pytest.raises(ValueError):
            oracle.shape_conv2d(*bad)
    assert oracle.shape_pool2d([5, 5, 3], 2, 2, 0, 0, 2, 2) == [2, 2, 3]
    assert oracle.shape_pool2d([5, 4], 3, 2, 1, 1, 1, 2) == [5, 3, 1]
    for bad in (([2, 2], 3, 1, 0, 0, 1, 1), ([5, 5], 0, 1, 0, 0, 1, 1), ([5, 5], 1, 1, 0, 0, 1, 0),
                ([5, 5, 1, 2], 1, 1, 0, 0, 1, 1)):
        with pytest.raises(ValueError):
            oracle.shape_pool2d(*bad)


def test_host_shape_rules_agree_with_the_oracle():
    # the Python mirror's shape_ops.conv2d / pool2d (host logic, no GPU) against the oracle's restatement,
    # valid and invalid arguments alike
    import itertools
    import primitiv_amd as pa
    S = pa.Shape
    xs = [([5, 5], 1), ([5, 4, 3], 2), ([7], 1), ([], 1), ([6, 6, 2], 3)]
    ws = [([2, 2], 1), ([3, 2, 3, 4], 1), ([1], 2), ([], 1), ([2, 3, 2, 5], 3), ([9, 1], 1)]
    args = [(0, 0, 1, 1, 1, 1), (1, 2, 2, 1, 1, 2), (0, 1, 1, 0, 1, 1), (2, 0, 3, 2, 0, 1), (3, 3, 1, 1, 3, 3)]
    agree = 0
    for (xd, bx), (wd, bw), a in itertools.product(xs, ws, args):
        try:
            want = oracle.shape_conv2d(xd, bx, wd, bw, *a)
        except ValueError:
            want = None
        try:
            got = pa.shape_ops.conv2d(S(xd, bx), S(wd, bw), *a)
            got = ([got[0], got[1], got[2]], got.batch())
        except pa.Error:
            got = None
        assert got == want, (xd, bx, wd, bw, a)
        agree += want is not None
    assert agree > 20
    for (xd, bx), a in itertools.product(xs, [(2, 2, 0, 0, 2, 2), (3, 1, 1, 0, 1, 1), (0, 1, 0, 0, 1, 1), (2, 2, 1, 1, 0, 1),
                                           (9, 9, 1, 1, 1, 1), (1, 1, 0, 0, 3, 2)]):
        try:
            want = oracle.shape_pool2d(xd, *a)
        except ValueError:
            want = None
        try:
            got = pa.shape_ops.pool2d(S(xd, bx), *a)
            got = [got[0], got[1], got[2]]
        except pa.Error:
            got = None
        assert got == want, (xd, a)
