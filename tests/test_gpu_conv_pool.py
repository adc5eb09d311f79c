"""conv2d and max_pool2d of the HIP devices (through the C ABI) against the
reference's golden vectors and the CPU oracle.

Tolerances: golden vectors to the reference's 4 ULPs (fp32 device; they are
small integers, exact in any summation order); random inputs
max|x - ref| / max|ref| <= 1e-4 (fp32), <= 2e-2 (16-bit storage, against the
fp32 oracle fed the un-rounded inputs); pooling is exact.
"""
import numpy as np
import pytest

import oracle
import primitiv_amd as pa
from conv_pool_cases import CASES, case_id, run_case_on, vgg_conv_case, vgg_pool_case
from util import norm_rel_err, vector_match

pytestmark = pytest.mark.gpu

S = pa.Shape
F32_TOL = 1e-4
H16_TOL = 2e-2


class DeviceBackend:
    """Golden-case backend over a device: flat arrays in, flat arrays out."""

    def __init__(self, dev):
        self.dev = dev

    def t(self, x, dims, batch):
        return self.dev.new_tensor_by_vector(S(dims, batch), np.asarray(x, dtype=np.float32))

    def conv2d_fw(self, x, w, x_dims, bx, w_dims, bw, *a):
        return self.dev.conv2d_fw(self.t(x, x_dims, bx), self.t(w, w_dims, bw), *a).to_vector()

    def conv2d_bw(self, x, w, gy, gx, gw, x_dims, bx, w_dims, bw, *a):
        tx, tw = self.t(x, x_dims, bx), self.t(w, w_dims, bw)
        ty = self.dev.conv2d_fw(tx, tw, *a)
        tgy = self.dev.new_tensor_by_vector(ty.shape(), np.asarray(gy, np.float32))
        tgx, tgw = self.t(gx, x_dims, bx), self.t(gw, w_dims, bw)
        self.dev.conv2d_bw(tx, tw, ty, tgy, *a, tgx, tgw)
        return tgx.to_vector(), tgw.to_vector()

    def max_pool2d_fw(self, x, x_dims, bs, *a):
        return self.dev.max_pool2d_fw(self.t(x, x_dims, bs), *a).to_vector()

    def max_pool2d_bw(self, x, y, gy, gx, x_dims, bs, *a):
        tx = self.t(x, x_dims, bs)
        sy = pa.shape_ops.pool2d(tx.shape(), *a)
        tgx = self.t(gx, x_dims, bs)
        self.dev.max_pool2d_bw(tx, self.dev.new_tensor_by_vector(sy, np.asarray(y, np.float32)),
                               self.dev.new_tensor_by_vector(sy, np.asarray(gy, np.float32)), *a, tgx)
        return tgx.to_vector()


@pytest.fixture(scope="module")
def dev():
    d = pa.HIP(0)
    yield d
    d.close()


@pytest.fixture(scope="module", params=["f16", "bf16"])
def dev16(request):
    d = pa.HIP16(0, storage=request.param)
    yield d
    d.close()


@pytest.mark.parametrize("kc", CASES, ids=case_id)
def test_reference_vectors(dev, kc):
    for want, got in run_case_on(DeviceBackend(dev), *kc):
        assert vector_match(want, got), kc[1]["source"]


@pytest.mark.parametrize("kc", [kc for kc in CASES if kc[0].startswith("max_pool2d")], ids=case_id)
def test_reference_pooling_vectors_half_storage(dev16, kc):
    # small integers are exact in 16-bit storage too
    for want, got in run_case_on(DeviceBackend(dev16), *kc):
        assert np.array_equal(np.float32(want), got), kc[1]["source"]


def test_vgg16_first_layer(dev):
    c = vgg_conv_case()
    b = DeviceBackend(dev)
    assert np.array_equal(b.conv2d_fw(c["x"], c["w"], c["x_dims"], 1, c["w_dims"], 1, *c["args"]), c["y"])
    gx, gw = b.conv2d_bw(c["x"], c["w"], np.ones_like(c["y"]), np.ones_like(c["x"]), np.ones_like(c["w"]),
                         c["x_dims"], 1, c["w_dims"], 1, *c["args"])
    assert np.array_equal(gx, c["gx"])
    assert vector_match(c["gw"], gw)


def test_vgg16_first_layer_minibatch_in_groups(dev):
    # 100 samples: the unfolded image of one sample is 27 x 50176 elements, so the samples pass
    # through scratch memory in two groups; all-ones inputs keep every sum an exact integer
    c = vgg_conv_case()
    bs = 100
    b = DeviceBackend(dev)
    x = np.ones(c["x"].size * bs, np.float32)
    y = b.conv2d_fw(x, c["w"], c["x_dims"], bs, c["w_dims"], 1, *c["args"])
    assert np.array_equal(y, np.tile(c["y"], bs))
    gx, gw = b.conv2d_bw(x, c["w"], np.ones_like(y), np.ones_like(x), np.ones_like(c["w"]), c["x_dims"], bs,
                         c["w_dims"], 1, *c["args"])
    assert np.array_equal(gx, np.tile(c["gx"], bs))
    assert vector_match(1 + (c["gw"] - 1) * bs, gw)


def test_vgg16_third_layer_pooling(dev):
    c = vgg_pool_case()
    b = DeviceBackend(dev)
    y = b.max_pool2d_fw(c["x"], c["x_dims"], 1, *c["args"])
    assert np.array_equal(y, c["y"])
    gx = b.max_pool2d_bw(c["x"], y, np.ones_like(y), np.ones_like(c["x"]), c["x_dims"], 1, *c["args"])
    assert np.array_equal(gx, c["gx"])


CONV_RANDOM = [  # x dims, w dims, (pad0, pad1, str0, str1, dil0, dil1)
    ([28, 28, 1], [5, 5, 1, 8], (2, 2, 1, 1, 1, 1)),
    ([14, 14, 8], [5, 5, 8, 16], (2, 2, 1, 1, 1, 1)),
    ([17, 13, 3], [3, 2, 3, 5], (1, 0, 2, 1, 1, 2)),
    ([9, 31, 4], [1, 1, 4, 6], (0, 0, 1, 1, 1, 1)),       # no unfolding: the image is the operand
    ([9, 31, 4], [1, 1, 4, 6], (1, 0, 2, 3, 1, 1)),       # 1 x 1 kernel that does need it
    ([32, 32, 16], [3, 3, 16, 32], (1, 1, 1, 1, 1, 1)),
    ([12, 10, 2], [4, 3, 2, 3], (3, 2, 3, 2, 2, 3)),
]


@pytest.mark.parametrize("bx,bw", [(1, 1), (5, 1), (1, 5), (5, 5)])
@pytest.mark.parametrize("xd,wd,a", CONV_RANDOM)
def test_convolution_matches_oracle(dev, xd, wd, a, bx, bw):
    rng = np.random.default_rng(sum(xd) + sum(wd) + 10 * bx + bw)
    x = rng.standard_normal(int(np.prod(xd)) * bx).astype(np.float32)
    w = rng.standard_normal(int(np.prod(wd)) * bw).astype(np.float32)
    b = DeviceBackend(dev)
    y = b.conv2d_fw(x, w, xd, bx, wd, bw, *a)
    ry = oracle.conv2d_fw(x, w, xd, bx, wd, bw, *a)
    assert norm_rel_err(y, ry) <= F32_TOL
    gy = rng.standard_normal(y.size).astype(np.float32)
    gx0 = rng.standard_normal(x.size).astype(np.float32)
    gw0 = rng.standard_normal(w.size).astype(np.float32)
    gx, gw = b.conv2d_bw(x, w, gy, gx0, gw0, xd, bx, wd, bw, *a)
    rgx, rgw = oracle.conv2d_bw(x, w, gy, gx0, gw0, xd, bx, wd, bw, *a)
    assert norm_rel_err(gx, rgx) <= F32_TOL
    assert norm_rel_err(gw, rgw) <= F32_TOL


@pytest.mark.parametrize("bx,bw", [(1, 1), (4, 1), (1, 4), (4, 4)])
@pytest.mark.parametrize("xd,wd,a", CONV_RANDOM[1:5])
def test_convolution_half_storage(dev16, xd, wd, a, bx, bw):
    rng = np.random.default_rng(sum(xd) + sum(wd) + 10 * bx + bw)
    x = rng.standard_normal(int(np.prod(xd)) * bx).astype(np.float32)
    w = (0.2 * rng.standard_normal(int(np.prod(wd)) * bw)).astype(np.float32)
    b = DeviceBackend(dev16)
    y = b.conv2d_fw(x, w, xd, bx, wd, bw, *a)
    assert norm_rel_err(y, oracle.conv2d_fw(x, w, xd, bx, wd, bw, *a)) <= H16_TOL
    gy = rng.standard_normal(y.size).astype(np.float32)
    gx0 = rng.standard_normal(x.size).astype(np.float32)
    gw0 = rng.standard_normal(w.size).astype(np.float32)
    gx, gw = b.conv2d_bw(x, w, gy, gx0, gw0, xd, bx, wd, bw, *a)
    rgx, rgw = oracle.conv2d_bw(x, w, gy, gx0, gw0, xd, bx, wd, bw, *a)
    assert norm_rel_err(gx, rgx) <= H16_TOL
    assert norm_rel_err(gw, rgw) <= H16_TOL


POOL_RANDOM = [  # x dims, batch, (win0, win1, pad0, pad1, str0, str1)
    ([28, 28, 8], 3, (2, 2, 0, 0, 2, 2)),
    ([17, 13, 3], 2, (3, 3, 1, 1, 2, 2)),       # overlapping windows
    ([9, 31, 4], 1, (9, 31, 0, 0, 1, 1)),       # one window per plane
    ([12, 10, 2], 4, (3, 2, 2, 1, 1, 3)),
    ([64, 64], 2, (5, 5, 2, 2, 1, 1)),
    ([17, 13, 3], 2, (2, 3, 1, 2, 2, 3)),       # disjoint windows with padding
    ([20, 21, 2], 3, (2, 2, 1, 1, 3, 4)),       # gaps between the windows
]


@pytest.mark.parametrize("xd,bs,a", POOL_RANDOM)
def test_pooling_matches_oracle(dev, xd, bs, a):
    rng = np.random.default_rng(sum(xd) + bs)
    # few distinct values: plenty of ties, so that WHICH maximum receives the gradient matters
    x = rng.integers(-3, 4, int(np.prod(xd)) * bs).astype(np.float32)
    b = DeviceBackend(dev)
    y = b.max_pool2d_fw(x, xd, bs, *a)
    assert np.array_equal(y, oracle.max_pool2d_fw(x, xd, bs, *a))
    gy = rng.integers(-8, 9, y.size).astype(np.float32)
    gx0 = rng.integers(-8, 9, x.size).astype(np.float32)
    gx = b.max_pool2d_bw(x, y, gy, gx0, xd, bs, *a)
    assert np.array_equal(gx, oracle.max_pool2d_bw(x, y, gy, gx0, xd, bs, *a))


def test_invalid_arguments(dev):
    x = dev.new_tensor_by_constant(S([5, 5, 2]), 1)
    for w_shape, a in ((S([6, 1, 2]), (0, 0, 1, 1, 1, 1)), (S([2, 2, 3]), (0, 0, 1, 1, 1, 1)),
                       (S([2, 2, 2]), (0, 0, 0, 1, 1, 1)), (S([2, 2, 2]), (0, 0, 1, 1, 0, 1)),
                       (S([2, 2, 2], 3), (0, 0, 1, 1, 1, 1))):
        xb = dev.new_tensor_by_constant(S([5, 5, 2], 2), 1) if w_shape.batch() == 3 else x
        with pytest.raises(pa.Error, match="Invalid arguments to calculate a convolution"):
            dev.conv2d_fw(xb, dev.new_tensor_by_constant(w_shape, 1), *a)
    for a in ((6, 1, 0, 0, 1, 1), (0, 1, 0, 0, 1, 1), (1, 1, 0, 0, 1, 0)):
        with pytest.raises(pa.Error, match="Invalid arguments to calculate a pooling"):
            dev.max_pool2d_fw(x, *a)
    y = dev.conv2d_fw(x, dev.new_tensor_by_constant(S([2, 2, 2, 3]), 1), 0, 0, 1, 1, 1, 1)
    with pytest.raises(pa.Error, match="Shape mismatched at conv2d_bw"):
        dev.conv2d_bw(x, dev.new_tensor_by_constant(S([2, 2, 2, 3]), 1), y, y, 0, 0, 1, 1, 1, 1,
                      dev.new_tensor_by_constant(S([5, 5]), 0), dev.new_tensor_by_constant(S([2, 2, 2, 3]), 0))
