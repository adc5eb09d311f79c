"""Elementwise operations of the HIP devices (through the C ABI) against the
reference's golden vectors and, at larger sizes, against the CPU oracle."""
import numpy as np
import pytest

import oracle
import primitiv_amd as pa
from pointwise_cases import CASES, run_case_on, case_id
from util import round_to_storage, ulp_diff

pytestmark = pytest.mark.gpu

S = pa.Shape


class DeviceBackend:
    """Runs a golden case on a device; arrays go in and come out as float32."""

    def __init__(self, dev):
        self.dev = dev

    def t(self, values, volume=None, batch=1):
        values = np.asarray(values, dtype=np.float32).reshape(-1)
        volume = values.size // batch if volume is None else volume
        return self.dev.new_tensor_by_vector(S([volume], batch), values)

    def unary_fw(self, op, x):
        return self.dev.unary_fw(op, self.t(x)).to_vector()

    def unary_bw(self, op, x, y, gy, gx):
        g = self.t(gx)
        self.dev.unary_bw(op, self.t(x), self.t(y), self.t(gy), g)
        return g.to_vector()

    def const_fw(self, op, x, k):
        return self.dev.const_fw(op, self.t(x), k).to_vector()

    def const_bw(self, op, x, y, gy, k, gx):
        g = self.t(gx)
        self.dev.const_bw(op, self.t(x), self.t(y), self.t(gy), k, g)
        return g.to_vector()

    def pown_fw(self, x, k):
        return self.dev.pown_fw(self.t(x), k).to_vector()

    def pown_bw(self, x, y, gy, k, gx):
        g = self.t(gx)
        self.dev.pown_bw(self.t(x), self.t(y), self.t(gy), k, g)
        return g.to_vector()

    def scalar_fw(self, op, k_on_left, x, k, volume, bx, bk):
        name = {("add", False): "add_scalar", ("add", True): "add_scalar",
                ("multiply", False): "multiply_scalar", ("multiply", True): "multiply_scalar"}.get(
                    (op, bool(k_on_left)), "%s_scalar_%s" % (op, "l" if k_on_left else "r"))
        kt = self.dev.new_tensor_by_vector(S([], bk), k)
        return self.dev.scalar_fw(name, self.t(x, volume, bx), kt).to_vector()

    def binary_fw(self, op, a, b, volume, ba, bb):
        return self.dev.binary_fw(op, self.t(a, volume, ba), self.t(b, volume, bb)).to_vector()

    def binary_bw(self, op, a, b, y, gy, ga, gb, volume, ba, bb):
        tga, tgb = self.t(ga, volume, ba), self.t(gb, volume, bb)
        self.dev.binary_bw(op, self.t(a, volume, ba), self.t(b, volume, bb), self.t(y, volume, max(ba, bb)),
                           self.t(gy, volume, max(ba, bb)), tga, tgb)
        return tga.to_vector(), tgb.to_vector()

    def inplace_subtract(self, x, y, volume, bx, by):
        ty = self.t(y, volume, by)
        self.dev.inplace_subtract(self.t(x, volume, bx), ty)
        return ty.to_vector()

    def inplace_multiply_const(self, k, x):
        tx = self.t(x)
        self.dev.inplace_multiply_const(k, tx)
        return tx.to_vector()

    def identity(self, rows):
        return self.dev.identity(rows).to_vector()


@pytest.fixture(scope="module")
def dev():
    return pa.HIP(0)


@pytest.fixture(scope="module", params=["f16", "bf16"])
def dev16(request):
    return pa.HIP16(0, storage=request.param)


@pytest.mark.parametrize("case", CASES, ids=case_id)
def test_f32_matches_reference_vectors(dev, case):
    # the ULP bound is the one the reference's own test grants a 32-bit device
    for got, want in run_case_on(DeviceBackend(dev), case):
        want = np.asarray(want, dtype=np.float32)
        assert got.shape == want.shape
        assert int(ulp_diff(got, want).max()) <= case["ulps"], (got, want)


@pytest.mark.parametrize("case", CASES, ids=case_id)
def test_half_storage_matches_reference_vectors(dev16, case):
    # bound of the reference's half-precision device (fp32 ULPs).  The reference
    # has no bf16 device: bf16 keeps 8 significant bits against half's 11 (one
    # rounding = 8x half's 4096 ULPs) and operands and result are each rounded,
    # hence 32x.  Values the 16-bit type cannot hold (overflow, or results
    # below its smallest normal number) are skipped.
    f16 = dev16._SUFFIX == "f16"
    bound = max(case["ulps16"], 1 << 12) * (1 if f16 else 32)
    tiny, huge = (6.2e-5, 6.0e4) if f16 else (1e-37, 3e38)
    if not f16 and "Convergence" in case["source"]:
        # 0.999 and 1.001 both round to 1 in bf16, so the power does not decay there: what the device must
        # give is the power of the operand it holds, +-1 to an odd or even exponent
        xr = round_to_storage(case["x"], "bf16")
        assert np.all(np.abs(xr) == 1.0)
        want = xr if case["k"] % 2 else np.ones_like(xr)
        (got, _), = run_case_on(DeviceBackend(dev16), case)
        assert np.array_equal(np.asarray(got, dtype=np.float32).reshape(-1), want)
        return
    for k in ("x", "a", "b", "gy", "y", "k"):
        v = case.get(k)
        if isinstance(v, list) and v and (np.max(np.abs(v)) > huge):
            pytest.skip("operand outside the 16-bit range")
    for got, want in run_case_on(DeviceBackend(dev16), case):
        want = np.asarray(want, dtype=np.float32)
        ok = (np.abs(want) < huge) & ((np.abs(want) > tiny * 64) | (want == 0))
        if not ok.any():
            continue
        d = ulp_diff(got[ok], want[ok])
        exact0 = (want[ok] == 0) & (np.abs(got[ok]) < 1e-3)
        assert int(np.where(exact0, 0, d).max()) <= bound, (got, want)


SIZES = [1, 7, 64, 1000, 4099, 1 << 20]


@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("op", pa.HIP.UNARY_OPS)
def test_unary_matches_oracle(dev, op, n):
    rng = np.random.default_rng(n)
    x = rng.uniform(0.1, 3.0, n).astype(np.float32)
    if op not in ("sqrt", "log"):
        x *= rng.choice([-1, 1], n).astype(np.float32)
    be = DeviceBackend(dev)
    y = be.unary_fw(op, x)
    ry = oracle.unary_fw(op, x)
    assert np.allclose(y, ry, rtol=2e-6, atol=1e-7)
    if op == "negate":
        return
    gy = rng.standard_normal(n).astype(np.float32)
    g0 = rng.standard_normal(n).astype(np.float32)
    assert np.allclose(be.unary_bw(op, x, ry, gy, g0), oracle.unary_bw(op, x, ry, gy, g0), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("n", [5, 4099, 1 << 18])
@pytest.mark.parametrize("op", pa.HIP.CONST_OPS)
def test_const_matches_oracle(dev, op, n):
    rng = np.random.default_rng(n + 1)
    x = rng.uniform(0.2, 2.0, n).astype(np.float32)
    if op in ("prelu", "elu", "add_const", "multiply_const"):
        x *= rng.choice([-1, 1], n).astype(np.float32)
    k = 1.5
    be = DeviceBackend(dev)
    ry = oracle.const_fw(op, x, k)
    assert np.allclose(be.const_fw(op, x, k), ry, rtol=2e-6, atol=1e-7)
    gy = rng.standard_normal(n).astype(np.float32)
    g0 = rng.standard_normal(n).astype(np.float32)
    assert np.allclose(be.const_bw(op, x, ry, gy, k, g0), oracle.const_bw(op, x, ry, gy, k, g0), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("k", [0, 1, 3, -2, 7])
def test_pown_matches_oracle(dev, k):
    rng = np.random.default_rng(k + 10)
    x = rng.uniform(0.5, 1.5, 3001).astype(np.float32) * rng.choice([-1, 1], 3001).astype(np.float32)
    be = DeviceBackend(dev)
    ry = oracle.pown_fw(x, k)
    assert np.allclose(be.pown_fw(x, k), ry, rtol=1e-6)
    gy = rng.standard_normal(x.size).astype(np.float32)
    g0 = rng.standard_normal(x.size).astype(np.float32)
    assert np.allclose(be.pown_bw(x, ry, gy, k, g0), oracle.pown_bw(x, ry, gy, k, g0), rtol=1e-5, atol=1e-6)


BATCHES = [(1, 1), (5, 5), (1, 5), (5, 1), (1, 64), (64, 1)]
VOLUMES = [1, 6, 256, 1001, 10000]


@pytest.mark.parametrize("volume", VOLUMES)
@pytest.mark.parametrize("ba,bb", BATCHES)
@pytest.mark.parametrize("op", pa.HIP.BINARY_OPS)
def test_binary_matches_oracle(dev, op, ba, bb, volume):
    rng = np.random.default_rng(volume + 7 * ba + bb)
    bs = max(ba, bb)
    a = rng.uniform(0.5, 2.0, volume * ba).astype(np.float32)
    b = rng.uniform(0.5, 2.0, volume * bb).astype(np.float32)
    be = DeviceBackend(dev)
    ry = oracle.binary_fw(op, a, b, volume, ba, bb)
    assert np.allclose(be.binary_fw(op, a, b, volume, ba, bb), ry, rtol=2e-6)
    gy = rng.standard_normal(volume * bs).astype(np.float32)
    ga0 = rng.standard_normal(a.size).astype(np.float32)
    gb0 = rng.standard_normal(b.size).astype(np.float32)
    ga, gb = be.binary_bw(op, a, b, ry, gy, ga0, gb0, volume, ba, bb)
    rga, rgb = oracle.binary_bw(op, a, b, ry, gy, ga0, gb0, volume, ba, bb)
    # the sum over the minibatch runs in a different order than the oracle's
    assert np.allclose(ga, rga, rtol=1e-4, atol=1e-4 * np.sqrt(bs))
    assert np.allclose(gb, rgb, rtol=1e-4, atol=1e-4 * np.sqrt(bs))


@pytest.mark.parametrize("op", sorted(pa.HIP.SCALAR_OPS))
@pytest.mark.parametrize("bx,bk", [(1, 1), (4, 4), (1, 4), (4, 1)])
def test_scalar_matches_oracle(dev, op, bx, bk):
    rng = np.random.default_rng(bx * 5 + bk)
    volume = 1003
    x = rng.uniform(0.5, 2.0, volume * bx).astype(np.float32)
    k = rng.uniform(0.5, 2.0, bk).astype(np.float32)
    binary, left = pa.HIP.SCALAR_OPS[op]
    y = dev.scalar_fw(op, dev.new_tensor_by_vector(S([volume], bx), x), dev.new_tensor_by_vector(S([], bk), k))
    assert y.shape() == S([volume], max(bx, bk))
    assert np.allclose(y.to_vector(), oracle.scalar_fw(binary, left, x, k, volume, bx, bk), rtol=2e-6)


def test_gradients_of_one_tensor_used_twice(dev):
    # x + x and x * x hand the same gradient tensor to both operands
    # (primitiv/core/graph.cc:205-216): it must receive both contributions.
    x = np.arange(1, 1001, dtype=np.float32)
    gy = np.full(1000, 2, dtype=np.float32)
    tx = dev.new_tensor_by_vector(S([1000]), x)
    tgy = dev.new_tensor_by_vector(S([1000]), gy)
    for op, want in (("add", 2 * gy), ("multiply", 2 * x * gy)):
        y = dev.binary_fw(op, tx, tx)
        g = dev.new_tensor_by_constant(S([1000]), 1)
        dev.binary_bw(op, tx, tx, y, tgy, g, g)
        assert np.array_equal(g.to_vector(), 1 + want)


def test_shape_errors(dev):
    a = dev.new_tensor_by_constant(S([2, 2]), 0)
    b = dev.new_tensor_by_constant(S([3]), 0)
    with pytest.raises(pa.Error):
        dev.binary_fw("add", a, b)
    with pytest.raises(pa.Error):
        dev.scalar_fw("add_scalar", a, b)
    with pytest.raises(pa.Error):
        dev.binary_fw("add", dev.new_tensor_by_constant(S([2, 2], 2), 0), dev.new_tensor_by_constant(S([2, 2], 3), 0))
    with pytest.raises(pa.Error):
        dev.inplace_subtract(b, a)
    with pytest.raises(pa.Error):
        dev.identity(0)


@pytest.mark.parametrize("n", [33, 1 << 16])
def test_half_storage_matches_oracle(dev16, n):
    rng = np.random.default_rng(n)
    tol = 2e-2
    be = DeviceBackend(dev16)
    x = (rng.uniform(0.25, 2.0, n) * rng.choice([-1, 1], n)).astype(np.float32)
    for op in ("tanh", "sigmoid", "exp", "softplus"):
        ry = oracle.unary_fw(op, x)
        assert np.max(np.abs(be.unary_fw(op, x) - ry)) <= tol * np.max(np.abs(ry))
    a = rng.uniform(0.5, 2.0, n).astype(np.float32)
    b = rng.uniform(0.5, 2.0, 4 * n).astype(np.float32)
    gy = rng.standard_normal(4 * n).astype(np.float32)
    for op in ("add", "multiply", "divide"):
        ry = oracle.binary_fw(op, a, b, n, 1, 4)
        y = be.binary_fw(op, a, b, n, 1, 4)
        assert np.max(np.abs(y - ry)) <= tol * np.max(np.abs(ry))
        ga, gb = be.binary_bw(op, a, b, ry, gy, np.zeros_like(a), np.zeros_like(b), n, 1, 4)
        rga, rgb = oracle.binary_bw(op, a, b, ry, gy, np.zeros_like(a), np.zeros_like(b), n, 1, 4)
        assert np.max(np.abs(ga - rga)) <= tol * np.max(np.abs(rga))
        assert np.max(np.abs(gb - rgb)) <= tol * np.max(np.abs(rgb))
