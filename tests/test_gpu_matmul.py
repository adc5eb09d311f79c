"""Parity of the HIP matmul path with the CPU oracle, through the C ABI.

Tolerance gate (stated with every check): max|x - ref| / max|ref| per output
tensor; fp32 device <= 1e-4, 16-bit storage <= 2e-2 against the fp32 oracle
fed the un-rounded inputs.  Integer-valued golden vectors of the reference's
own tests must match to 4 ULPs as they do there.
"""
import numpy as np
import pytest

import oracle
import primitiv_amd as pa
from primitiv_amd import _lib
from primitiv_amd.configs import WORKLOADS
from util import norm_rel_err, np_matmul_bw, np_matmul_fw, vector_match

pytestmark = pytest.mark.gpu

F32_TOL = 1e-4
H16_TOL = 2e-2


@pytest.fixture(scope="module")
def dev():
    d = pa.HIP(0)
    yield d
    d.close()


@pytest.fixture(scope="module")
def dev16():
    d = pa.HIP16(0, storage="f16")
    yield d
    d.close()


@pytest.fixture(scope="module")
def devbf16():
    d = pa.HIP16(0, storage="bf16")
    yield d
    d.close()


def _fw_bw(dev, a, b, gy, ga0, gb0, di, dj, dk, ba, bb):
    bs = max(ba, bb)
    ta = dev.new_tensor_by_vector(pa.Shape([di, dj], ba), a)
    tb = dev.new_tensor_by_vector(pa.Shape([dj, dk], bb), b)
    ty = dev.matmul_fw(ta, tb)
    assert ty.shape() == pa.Shape([di, dk], bs)
    tgy = dev.new_tensor_by_vector(ty.shape(), gy)
    tga = dev.new_tensor_by_vector(ta.shape(), ga0)
    tgb = dev.new_tensor_by_vector(tb.shape(), gb0)
    dev.matmul_bw(ta, tb, ty, tgy, tga, tgb)
    return ty.to_vector(), tga.to_vector(), tgb.to_vector()


# ---- the reference's golden vectors -----------------------------------------

def test_golden_forward(dev, golden):
    for c in golden["matmul_fw"]:
        a = dev.new_tensor_by_vector(pa.Shape([c["di"], c["dj"]], c["ba"]), c["a"])
        b = dev.new_tensor_by_vector(pa.Shape([c["dj"], c["dk"]], c["bb"]), c["b"])
        y = dev.matmul_fw(a, b)
        assert y.shape() == pa.Shape([c["di"], c["dk"]], max(c["ba"], c["bb"]))
        assert vector_match(c["y"], y.to_vector()), c["source"]


def test_golden_forward_large(dev, golden):
    n = golden["matmul_fw_large"]["n"]
    i = np.arange(n, dtype=np.float64)
    a_data = np.tile(i / 16.0, n)
    b_data = np.repeat(i / 16.0, n)
    y1 = np.outer(i, i).T.reshape(-1) * n / 256.0
    y2 = np.full(n * n, np.sum(i * i) / 256.0)
    a = dev.new_tensor_by_vector([n, n], a_data)
    b = dev.new_tensor_by_vector([n, n], b_data)
    assert vector_match(y1, dev.matmul_fw(a, b).to_vector())
    assert vector_match(y2, dev.matmul_fw(b, a).to_vector())


def test_golden_backward(dev, golden):
    for c in golden["matmul_bw"] + [golden["matmul_operator"]]:
        a = dev.new_tensor_by_vector(pa.Shape([c["di"], c["dj"]], c["ba"]), c["a"])
        b = dev.new_tensor_by_vector(pa.Shape([c["dj"], c["dk"]], c["bb"]), c["b"])
        y = dev.matmul_fw(a, b)
        gy = dev.new_tensor_by_vector(y.shape(), c["gy"])
        ga = dev.new_tensor_by_constant(a.shape(), 0)
        gb = dev.new_tensor_by_constant(b.shape(), 0)
        dev.matmul_bw(a, b, y, gy, ga, gb)
        assert vector_match(c["ga"], ga.to_vector()), c["source"]
        assert vector_match(c["gb"], gb.to_vector()), c["source"]


def test_invalid_matmul(dev, golden):
    # test/tensor_forward_test.cc:1907-1927
    for c in golden["shape_matmul_invalid"]["cases"]:
        a = dev.new_tensor_by_constant(pa.Shape(c["a"], c["ba"]), 0)
        b = dev.new_tensor_by_constant(pa.Shape(c["b"], c["bb"]), 0)
        with pytest.raises(pa.Error):
            dev.matmul_fw(a, b)


def test_golden_half_storage(dev16, devbf16, golden):
    # small integers are exact in either 16-bit format; the reference's own
    # half device needs 16384 ULPs on CheckMatMulAB (tensor_forward_test.cc:1838-1842)
    for d in (dev16, devbf16):
        for c in golden["matmul_fw"]:
            a = d.new_tensor_by_vector(pa.Shape([c["di"], c["dj"]], c["ba"]), c["a"])
            b = d.new_tensor_by_vector(pa.Shape([c["dj"], c["dk"]], c["bb"]), c["b"])
            y = d.matmul_fw(a, b).to_vector()
            assert norm_rel_err(y, c["y"]) <= (2.0 ** -9 if d is dev16 else 2.0 ** -8), c["source"]
        for c in golden["matmul_bw"] + [golden["matmul_operator"]]:
            a = d.new_tensor_by_vector(pa.Shape([c["di"], c["dj"]], c["ba"]), c["a"])
            b = d.new_tensor_by_vector(pa.Shape([c["dj"], c["dk"]], c["bb"]), c["b"])
            y = d.matmul_fw(a, b)
            gy = d.new_tensor_by_vector(y.shape(), c["gy"])
            ga = d.new_tensor_by_constant(a.shape(), 0)
            gb = d.new_tensor_by_constant(b.shape(), 0)
            d.matmul_bw(a, b, y, gy, ga, gb)
            assert vector_match(c["ga"], ga.to_vector()), c["source"]
            assert vector_match(c["gb"], gb.to_vector()), c["source"]


# ---- random shapes against the oracle ------------------------------------------

SHAPES = [  # di, dj, dk : aligned, ragged, degenerate, larger than one tile in every direction
    (1, 1, 1), (1, 5, 1), (7, 1, 3), (2, 3, 4), (33, 17, 65), (64, 64, 64),
    (123, 123, 123), (128, 128, 128), (130, 70, 258), (257, 129, 31), (300, 20, 5),
    (8, 1000, 8), (5, 4097, 3), (650, 64, 1), (512, 96, 260),
]
BATCHES = [(1, 1), (3, 3), (1, 3), (3, 1), (1, 37), (37, 1)]


@pytest.mark.parametrize("ba,bb", BATCHES)
def test_random_shapes_f32(dev, ba, bb):
    rng = np.random.default_rng(100 * ba + bb)
    for di, dj, dk in SHAPES:
        bs = max(ba, bb)
        if di * dj * dk * bs > 40_000_000:
            continue
        a = rng.standard_normal(di * dj * ba).astype(np.float32)
        b = rng.standard_normal(dj * dk * bb).astype(np.float32)
        gy = rng.standard_normal(di * dk * bs).astype(np.float32)
        ga0 = rng.standard_normal(a.size).astype(np.float32)
        gb0 = rng.standard_normal(b.size).astype(np.float32)
        y, ga, gb = _fw_bw(dev, a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
        ry = oracle.matmul_fw(a, b, di, dj, dk, ba, bb, 4)
        rga, rgb = oracle.matmul_bw(a, b, gy, ga0, gb0, di, dj, dk, ba, bb, 4)
        tag = "shape (%d,%d,%d) batch (%d,%d)" % (di, dj, dk, ba, bb)
        assert norm_rel_err(y, ry) <= F32_TOL, "y " + tag
        assert norm_rel_err(ga, rga) <= F32_TOL, "ga " + tag
        assert norm_rel_err(gb, rgb) <= F32_TOL, "gb " + tag


@pytest.mark.parametrize("which", ["f16", "bf16"])
@pytest.mark.parametrize("ba,bb", [(1, 1), (3, 3), (1, 5), (5, 1)])
def test_random_shapes_h16(dev16, devbf16, which, ba, bb):
    # Tiny outputs (a handful of terms that may cancel) make max|ref| an unfair
    # yardstick for 8..11-bit inputs, so the error is measured against the
    # magnitude the terms had before cancelling: max over the tensor of
    # sum|a||b| (+|g0|), which the oracle computes from the absolute values.
    # Where nothing cancels this is the plain gate max|x-ref|/max|ref|.
    d = dev16 if which == "f16" else devbf16
    tol = H16_TOL
    rng = np.random.default_rng(7 * ba + bb)
    for di, dj, dk in SHAPES:
        bs = max(ba, bb)
        a = rng.standard_normal(di * dj * ba).astype(np.float32)
        b = rng.standard_normal(dj * dk * bb).astype(np.float32)
        gy = rng.standard_normal(di * dk * bs).astype(np.float32)
        ga0 = rng.standard_normal(a.size).astype(np.float32)
        gb0 = rng.standard_normal(b.size).astype(np.float32)
        y, ga, gb = _fw_bw(d, a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
        ry = oracle.matmul_fw(a, b, di, dj, dk, ba, bb, 4)
        rga, rgb = oracle.matmul_bw(a, b, gy, ga0, gb0, di, dj, dk, ba, bb, 4)
        sy = oracle.matmul_fw(np.abs(a), np.abs(b), di, dj, dk, ba, bb, 4)
        sga, sgb = oracle.matmul_bw(np.abs(a), np.abs(b), np.abs(gy), np.abs(ga0), np.abs(gb0),
                                    di, dj, dk, ba, bb, 4)
        tag = "%s shape (%d,%d,%d) batch (%d,%d)" % (which, di, dj, dk, ba, bb)
        for name, got, ref, scale in (("y", y, ry, sy), ("ga", ga, rga, sga), ("gb", gb, rgb, sgb)):
            err = float(np.max(np.abs(got.astype(np.float64) - ref)) / np.max(scale))
            assert err <= tol, "%s %s err %.3g" % (name, tag, err)
            if min(di, dj, dk) >= 64:
                assert norm_rel_err(got, ref) <= tol, name + " " + tag


def _drawn_dim(rng):
    kind = int(rng.integers(0, 6))
    if kind == 0:
        return int(rng.integers(1, 20))
    if kind == 1:
        return int(rng.integers(1, 200))
    if kind == 2:
        return int(rng.integers(1, 90)) * 8
    if kind == 3:
        return int(rng.integers(100, 1400))
    if kind == 4:
        return int(rng.choice([64, 128, 256, 512, 1024, 650, 2600, 2048, 4096]))
    return int(rng.integers(1000, 5000))


@pytest.mark.parametrize("seed", range(4))
def test_drawn_dimensions_all_devices(dev, dev16, devbf16, seed):
    # Dimensions drawn from tiny / odd / multiple-of-8 / layer-sized / long
    # classes, independently per axis, so that a seed crosses most kernel
    # choices and their edge handling.  Reference: float64 numpy on the values
    # each device actually stores (gate: F32_TOL, H16_TOL of max|ref|).
    rng = np.random.default_rng(9000 + seed)
    for it in range(25):
        di, dj, dk = (_drawn_dim(rng) for _ in range(3))
        ba, bb = [(1, 1), (1, 1), (1, int(rng.integers(2, 6))), (int(rng.integers(2, 6)), 1), (3, 3)][
            int(rng.integers(0, 5))]
        bs = max(ba, bb)
        while di * dj * dk * bs > 2e9 or max(di * dj * ba, dj * dk * bb, di * dk * bs) > 2e7:
            if di >= dj and di >= dk:
                di = di // 2 + 1
            elif dj >= dk:
                dj = dj // 2 + 1
            else:
                dk = dk // 2 + 1
        a = rng.standard_normal(di * dj * ba).astype(np.float32)
        b = rng.standard_normal(dj * dk * bb).astype(np.float32)
        gy = rng.standard_normal(di * dk * bs).astype(np.float32)
        ga0 = rng.standard_normal(a.size).astype(np.float32)
        gb0 = rng.standard_normal(b.size).astype(np.float32)
        for d, tol in ((dev, F32_TOL), (dev16, H16_TOL), (devbf16, H16_TOL)):
            stored = [d.new_tensor_by_vector(pa.Shape(dims, n), v).to_vector().astype(np.float64)
                      for dims, n, v in (([di, dj], ba, a), ([dj, dk], bb, b), ([di, dk], bs, gy),
                                         ([di, dj], ba, ga0), ([dj, dk], bb, gb0))]
            y, ga, gb = _fw_bw(d, a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
            ry = np_matmul_fw(stored[0], stored[1], di, dj, dk, ba, bb)
            dga, dgb = np_matmul_bw(stored[0], stored[1], stored[2], di, dj, dk, ba, bb)
            tag = "%s draw %d shape (%d,%d,%d) batch (%d,%d)" % (type(d).__name__, it, di, dj, dk, ba, bb)
            assert norm_rel_err(y, ry) <= tol, "y " + tag
            assert norm_rel_err(ga, stored[3] + dga) <= tol, "ga " + tag
            assert norm_rel_err(gb, stored[4] + dgb) <= tol, "gb " + tag


def _drawn_shape(rng, kind):
    if kind == 0:   # small, any alignment
        return [int(rng.integers(1, 300)) for _ in range(3)]
    if kind == 1:   # few columns against a long or tall operand: the per-timestep shapes
        return [int(rng.integers(1, 4000)), int(rng.integers(1, 3000)), int(rng.integers(1, 130))]
    if kind == 2:   # short K: rank-K updates
        return [int(rng.integers(64, 3000)), int(rng.integers(1, 100)), int(rng.integers(64, 2000))]
    if kind == 3:   # mid-size, multiples of 4: the tile kernels and their split / mixed launches
        return [int(rng.integers(16, 500)) * 4 for _ in range(3)]
    if kind == 4:   # few outputs over a very long K
        return [int(rng.integers(1, 200)), int(rng.integers(2000, 40000)), int(rng.integers(1, 200))]
    return [int(rng.integers(100, 1800)) for _ in range(3)]   # mid-size, any alignment


@pytest.mark.parametrize("seed", range(2))
def test_drawn_shape_classes_all_devices(dev, dev16, devbf16, seed):
    # Whole shapes drawn class by class (where the draw above draws each axis on its own), each in a drawn
    # batch case, on the fp32 device in both accumulation modes and on both 16-bit devices, against
    # float64 numpy on the values each device stores.
    rng = np.random.default_rng(7000 + seed)
    det = pa.HIP(0)
    det.set_deterministic(True)
    for it in range(30):
        di, dj, dk = _drawn_shape(rng, it % 6)
        ba, bb = [(1, 1), (1, int(rng.integers(2, 6))), (int(rng.integers(2, 6)), 1), (3, 3)][int(rng.integers(0, 4))]
        bs = max(ba, bb)
        while di * dj * dk * bs > 2e9:
            di, dk = max(1, di // 2), max(1, dk // 2)
        a = rng.standard_normal(di * dj * ba).astype(np.float32)
        b = rng.standard_normal(dj * dk * bb).astype(np.float32)
        gy = rng.standard_normal(di * dk * bs).astype(np.float32)
        ga0 = rng.standard_normal(a.size).astype(np.float32)
        gb0 = rng.standard_normal(b.size).astype(np.float32)
        for d, tol in ((dev, F32_TOL), (det, F32_TOL), (dev16, H16_TOL), (devbf16, H16_TOL)):
            stored = [d.new_tensor_by_vector(pa.Shape(dims, n), v).to_vector().astype(np.float64)
                      for dims, n, v in (([di, dj], ba, a), ([dj, dk], bb, b), ([di, dk], bs, gy),
                                         ([di, dj], ba, ga0), ([dj, dk], bb, gb0))]
            y, ga, gb = _fw_bw(d, a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
            ry = np_matmul_fw(stored[0], stored[1], di, dj, dk, ba, bb)
            dga, dgb = np_matmul_bw(stored[0], stored[1], stored[2], di, dj, dk, ba, bb)
            tag = "%s%s draw %d shape (%d,%d,%d) batch (%d,%d)" % (type(d).__name__, " deterministic" if d is det else "",
                                                                   it, di, dj, dk, ba, bb)
            assert norm_rel_err(y, ry) <= tol, "y " + tag
            assert norm_rel_err(ga, stored[3] + dga) <= tol, "ga " + tag
            assert norm_rel_err(gb, stored[4] + dgb) <= tol, "gb " + tag
    det.close()


# shapes that reach the fp32 128x128x32 global-to-LDS kernel (>= one tile per CU)
# with ragged edges in every dimension (multiples of 4, not of 128 / 32)
BIG_F32 = [  # di, dj, dk, ba, bb
    (2056, 2064, 2072, 1, 1),
    (776, 520, 1032, 16, 16),
    (136, 2056, 2064, 16, 1),
    (2056, 264, 520, 1, 4),
]


@pytest.mark.parametrize("di,dj,dk,ba,bb", BIG_F32)
def test_large_tile_f32(dev, di, dj, dk, ba, bb):
    rng = np.random.default_rng(di + dj + dk + ba)
    bs = max(ba, bb)
    a = rng.standard_normal(di * dj * ba).astype(np.float32)
    b = rng.standard_normal(dj * dk * bb).astype(np.float32)
    gy = rng.standard_normal(di * dk * bs).astype(np.float32)
    ga0 = rng.standard_normal(a.size).astype(np.float32)
    gb0 = rng.standard_normal(b.size).astype(np.float32)
    y, ga, gb = _fw_bw(dev, a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
    ry = oracle.matmul_fw(a, b, di, dj, dk, ba, bb, 8)
    rga, rgb = oracle.matmul_bw(a, b, gy, ga0, gb0, di, dj, dk, ba, bb, 8)
    assert norm_rel_err(y, ry) <= F32_TOL
    assert norm_rel_err(ga, rga) <= F32_TOL
    assert norm_rel_err(gb, rgb) <= F32_TOL


# a large operand streamed against at most 64 output columns (the output-projection
# products): 32 x 64 tiles with the K range cut between workgroups.  Aligned and
# 4-byte-aligned narrow operands, ragged M / N / K, N = 1, a contraction over
# the minibatch, a minibatch of large operands.
STREAMED_F32 = [  # di, dj, dk, ba, bb
    (4100, 520, 1, 1, 64),
    (4100, 518, 1, 1, 40),
    (1028, 512, 48, 5, 1),
    (8192, 260, 1, 1, 1),
    (4100, 520, 2, 1, 30),
    # weight gradients that are rank-K updates (K = minibatch <= 64) of a large matrix:
    # 128 x 128 tiles in one round; aligned and 4-byte-aligned x, K = 64 / 40 / 20, a minibatch of updates
    (4100, 1300, 1, 1, 64),
    (4100, 1302, 1, 1, 40),
    (4100, 1300, 1, 1, 20),
    (1028, 1300, 30, 4, 4),
]


@pytest.mark.parametrize("di,dj,dk,ba,bb", STREAMED_F32)
def test_streamed_operand_f32(dev, di, dj, dk, ba, bb):
    rng = np.random.default_rng(di + dj + dk + ba)
    bs = max(ba, bb)
    a = rng.standard_normal(di * dj * ba).astype(np.float32)
    b = rng.standard_normal(dj * dk * bb).astype(np.float32)
    gy = rng.standard_normal(di * dk * bs).astype(np.float32)
    ga0 = rng.standard_normal(a.size).astype(np.float32)
    gb0 = rng.standard_normal(b.size).astype(np.float32)
    y, ga, gb = _fw_bw(dev, a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
    ry = oracle.matmul_fw(a, b, di, dj, dk, ba, bb, 8)
    rga, rgb = oracle.matmul_bw(a, b, gy, ga0, gb0, di, dj, dk, ba, bb, 8)
    assert norm_rel_err(y, ry) <= F32_TOL
    assert norm_rel_err(ga, rga) <= F32_TOL
    assert norm_rel_err(gb, rgb) <= F32_TOL
    # the second call's y lands in pool memory that still holds the first call's
    # results: an overwriting product must not add to them (a split product zero-fills first)
    y2, _, _ = _fw_bw(dev, a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
    assert norm_rel_err(y2, ry) <= F32_TOL


# both gradient products of a small matmul leave in one launch when their outputs do not
# overlap: the dense layer, the recurrent gate (a rank-K update by staged 64 x 64 tiles
# beside a long-K product split between workgroups), ragged edges, a contraction over
# the minibatch, per-sample products
PAIRED_F32 = [  # di, dj, dk, ba, bb
    (256, 784, 1, 1, 128),
    (2048, 512, 1, 1, 64),
    (2052, 516, 1, 1, 60),
    (512, 96, 260, 1, 1),
    (64, 64, 8, 9, 1),
    (132, 260, 24, 6, 6),
    (1024, 1024, 1, 1, 8),
    (2600, 650, 1, 1, 64),      # an LSTM's gates with 650 hidden units: rows of b^T are not 16-byte aligned
]


@pytest.mark.parametrize("di,dj,dk,ba,bb", PAIRED_F32)
def test_paired_gradient_products_f32(dev, di, dj, dk, ba, bb):
    rng = np.random.default_rng(di * 3 + dj + dk + ba)
    bs = max(ba, bb)
    a = rng.standard_normal(di * dj * ba).astype(np.float32)
    b = rng.standard_normal(dj * dk * bb).astype(np.float32)
    gy = rng.standard_normal(di * dk * bs).astype(np.float32)
    ga0 = rng.standard_normal(a.size).astype(np.float32)
    gb0 = rng.standard_normal(b.size).astype(np.float32)
    _, ga, gb = _fw_bw(dev, a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
    rga, rgb = oracle.matmul_bw(a, b, gy, ga0, gb0, di, dj, dk, ba, bb, 8)
    assert norm_rel_err(ga, rga) <= F32_TOL
    assert norm_rel_err(gb, rgb) <= F32_TOL


def test_gradients_into_one_buffer(dev):
    # ga and gb may be the same memory (the gradient of x.x for a square x): the two
    # products must then add one after the other, not race
    from primitiv_amd import _lib
    n = 96
    rng = np.random.default_rng(5)
    a = rng.standard_normal(n * n).astype(np.float32)
    b = rng.standard_normal(n * n).astype(np.float32)
    gy = rng.standard_normal(n * n).astype(np.float32)
    g0 = rng.standard_normal(n * n).astype(np.float32)
    sh = pa.Shape([n, n])
    ta, tb, tgy, tg = (dev.new_tensor_by_vector(sh, v) for v in (a, b, gy, g0))
    rc = _lib.lib().phip_matmul_bw_f32(dev.ctx(), ta.handle(), tb.handle(), tgy.handle(), tg.handle(), tg.handle(),
                                       n, n, n, 1, 1)
    assert rc == 0
    zero = np.zeros(n * n, np.float32)
    rga, rgb = oracle.matmul_bw(a, b, gy, g0, zero, n, n, n, 1, 1, 4)
    assert norm_rel_err(tg.to_vector(), rga + rgb) <= F32_TOL


# mid-size products: with a long K (from 2048) and fewer 128 x 128 tiles than CUs the large-tile
# kernel with its K range cut between workgroups - forward (partial tiles and tickets), both
# gradients (atomics), ragged edges, per-sample products, a contraction over the minibatch
MIDSIZE_F32 = [  # di, dj, dk, ba, bb
    (1536, 2048, 512, 1, 1),
    (1024, 1024, 2048, 1, 1),
    (2048, 1024, 1024, 1, 1),
    (1028, 1100, 2052, 1, 1),
    (520, 2080, 300, 3, 3),
    (700, 1040, 520, 3, 1),
    # shorter K: 64 x 64 tiles moved global -> LDS directly (forward unsplit, gradients split with atomics)
    (1028, 520, 1100, 1, 1),
    (400, 264, 400, 4, 4),
    (400, 264, 400, 4, 1),
]


@pytest.mark.parametrize("di,dj,dk,ba,bb", MIDSIZE_F32)
def test_midsize_long_k_f32(dev, di, dj, dk, ba, bb):
    rng = np.random.default_rng(di + 2 * dj + 3 * dk + ba)
    bs = max(ba, bb)
    a = rng.standard_normal(di * dj * ba).astype(np.float32)
    b = rng.standard_normal(dj * dk * bb).astype(np.float32)
    gy = rng.standard_normal(di * dk * bs).astype(np.float32)
    ga0 = rng.standard_normal(a.size).astype(np.float32)
    gb0 = rng.standard_normal(b.size).astype(np.float32)
    y, ga, gb = _fw_bw(dev, a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
    ry = oracle.matmul_fw(a, b, di, dj, dk, ba, bb, 8)
    rga, rgb = oracle.matmul_bw(a, b, gy, ga0, gb0, di, dj, dk, ba, bb, 8)
    assert norm_rel_err(y, ry) <= F32_TOL
    assert norm_rel_err(ga, rga) <= F32_TOL
    assert norm_rel_err(gb, rgb) <= F32_TOL


# an overwriting product with at most one 64 x 64 tile per compute unit: eight wavefronts per tile, each with
# its own operand blocks in LDS and no barrier in the K loop, pairs of wavefronts taking alternate K tiles -
# a K of five K tiles, an odd number of them, not a multiple of 32; ragged M and N; a minibatch on the grid
# and one folded into the columns
ALONE_F32 = [  # di, dj, dk, ba, bb
    (1024, 1024, 1024, 1, 1),
    (768, 800, 776, 1, 1),
    (1000, 132, 520, 1, 1),
    (1000, 160, 1020, 1, 1),
    (520, 1036, 264, 3, 3),
    (776, 2000, 200, 1, 4),
]


@pytest.mark.parametrize("di,dj,dk,ba,bb", ALONE_F32)
def test_one_tile_per_compute_unit_f32(dev, di, dj, dk, ba, bb):
    rng = np.random.default_rng(3 * di + dj + 11 * dk + ba)
    a = rng.standard_normal(di * dj * ba).astype(np.float32)
    b = rng.standard_normal(dj * dk * bb).astype(np.float32)
    ta = dev.new_tensor_by_vector(pa.Shape([di, dj], ba), a)
    tb = dev.new_tensor_by_vector(pa.Shape([dj, dk], bb), b)
    dev.gemm_trace(True)
    y = dev.matmul_fw(ta, tb).to_vector()
    assert dev.gemm_trace(False) == ["f32_lds64w"]
    assert norm_rel_err(y, oracle.matmul_fw(a, b, di, dj, dk, ba, bb, 8)) <= F32_TOL
    for _ in range(5):
        assert np.array_equal(dev.matmul_fw(ta, tb).to_vector(), y)


# tiles that do not fill a whole number of rounds on the chip: the first rounds' tiles whole, the rest cut
# into K ranges that spread over all compute units (partial tiles and tickets forward, atomics backward):
# 64 x 64 tiles (576 = 2 x 256 + 64), ragged edges, a minibatch of products, and 128 x 128 tiles
MIXED_F32 = [  # di, dj, dk, ba, bb
    (1536, 1536, 1536, 1, 1),
    (1540, 1000, 1530, 1, 1),
    (520, 520, 640, 9, 9),
    (2056, 2064, 2072, 1, 1),
]


@pytest.mark.parametrize("di,dj,dk,ba,bb", MIXED_F32)
def test_partly_filled_last_round_f32(dev, di, dj, dk, ba, bb):
    rng = np.random.default_rng(di + 5 * dj + 7 * dk + ba)
    bs = max(ba, bb)
    a = rng.standard_normal(di * dj * ba).astype(np.float32)
    b = rng.standard_normal(dj * dk * bb).astype(np.float32)
    gy = rng.standard_normal(di * dk * bs).astype(np.float32)
    ga0 = rng.standard_normal(a.size).astype(np.float32)
    gb0 = rng.standard_normal(b.size).astype(np.float32)
    dev.gemm_trace(True)
    y, ga, gb = _fw_bw(dev, a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
    kernels = dev.gemm_trace(False)
    assert any(k.endswith("_mixed") for k in kernels), kernels   # (listed per stream, not in call order)
    ry = oracle.matmul_fw(a, b, di, dj, dk, ba, bb, 8)
    rga, rgb = oracle.matmul_bw(a, b, gy, ga0, gb0, di, dj, dk, ba, bb, 8)
    assert norm_rel_err(y, ry) <= F32_TOL
    assert norm_rel_err(ga, rga) <= F32_TOL
    assert norm_rel_err(gb, rgb) <= F32_TOL


# an overwriting product with few output tiles and a long K is cut between workgroups
# that meet through partial tiles, summed in a fixed order by whichever finishes last:
# right, and the same bits on every run
@pytest.mark.parametrize("di,dj,dk,ba,bb", [(256, 784, 1, 1, 128), (64, 3000, 1, 1, 40), (100, 5000, 33, 1, 1),
                                            (48, 2048, 8, 3, 3), (1028, 2052, 1100, 1, 1),
                                            (1024, 4096, 1, 1, 128), (1536, 1536, 1536, 1, 1),
                                            (520, 520, 640, 9, 9)])
def test_split_forward_is_right_and_reproducible(dev, di, dj, dk, ba, bb):
    rng = np.random.default_rng(di + dj)
    a = rng.standard_normal(di * dj * ba).astype(np.float32)
    b = rng.standard_normal(dj * dk * bb).astype(np.float32)
    ta = dev.new_tensor_by_vector(pa.Shape([di, dj], ba), a)
    tb = dev.new_tensor_by_vector(pa.Shape([dj, dk], bb), b)
    first = dev.matmul_fw(ta, tb).to_vector()
    assert norm_rel_err(first, oracle.matmul_fw(a, b, di, dj, dk, ba, bb, 8)) <= F32_TOL
    for _ in range(25):
        assert np.array_equal(dev.matmul_fw(ta, tb).to_vector(), first)


# an overwriting product with very few outputs and a K of 256..1024 runs on 16 x 16 tiles whose
# eight wavefronts split K (no exchange between workgroups): the dense layer, ragged rows and
# columns, K not a multiple of the 16 k of a load round or of four (4-byte loads of b), the shortest
# and longest K it takes, a minibatch folded into the columns
TILE16_F32 = [(256, 784, 1, 1, 128), (250, 700, 1, 1, 100), (33, 1024, 17, 1, 1), (16, 256, 16, 1, 1),
              (100, 701, 1, 1, 50), (129, 999, 3, 1, 7), (7, 513, 5, 1, 1), (300, 1000, 1, 1, 40)]


@pytest.mark.parametrize("di,dj,dk,ba,bb", TILE16_F32)
def test_few_outputs_long_k_forward_f32(dev, di, dj, dk, ba, bb):
    rng = np.random.default_rng(di * 7 + dj)
    a = rng.standard_normal(di * dj * ba).astype(np.float32)
    b = rng.standard_normal(dj * dk * bb).astype(np.float32)
    ta = dev.new_tensor_by_vector(pa.Shape([di, dj], ba), a)
    tb = dev.new_tensor_by_vector(pa.Shape([dj, dk], bb), b)
    want = oracle.matmul_fw(a, b, di, dj, dk, ba, bb, 8)
    first = dev.matmul_fw(ta, tb).to_vector()
    assert norm_rel_err(first, want) <= F32_TOL
    # every element, not only the largest: a row or column dropped at a ragged edge shows here
    assert np.max(np.abs(np.asarray(first) - want)) <= 1e-4 * max(1.0, np.max(np.abs(want)))
    for _ in range(5):                      # overwrites whatever the pool block held, same bits every time
        assert np.array_equal(dev.matmul_fw(ta, tb).to_vector(), first)
    # b at an address that is not 16-byte aligned: the same product through 4-byte loads of b
    whole = dev.new_tensor_by_vector(pa.Shape([dj * dk * bb + 1]), np.concatenate([[0.0], b]).astype(np.float32))
    y = dev.new_raw_tensor(pa.Shape([di, dk], bb))
    _lib.call("phip_matmul_fw_f32", dev.ctx(), ta.handle(), whole.handle() + 4, y.mutable_handle(), di, dj, dk, ba, bb)
    assert norm_rel_err(y.to_vector(), want) <= F32_TOL


# accumulating products whose contraction is cut between workgroups: the dense layer's and the
# recurrent gate's gradients (small, both products normally in one launch), an output projection
# (rank-K update + streamed operand, whole and split tiles), mid-size long-K products (large tiles),
# ragged shapes, per-sample products and a contraction over the minibatch
SPLIT_BW = [(256, 784, 1, 1, 128), (2048, 512, 1, 1, 64), (4100, 650, 1, 1, 64), (10000, 650, 1, 1, 64),
            (1028, 2052, 1100, 1, 1), (1536, 512, 4096, 1, 1), (96, 1000, 5, 1, 3), (48, 2048, 8, 3, 3),
            (300, 20, 5, 9, 1), (130, 70, 258, 1, 4), (1536, 1536, 1536, 1, 1), (1540, 1000, 1530, 1, 1)]


@pytest.mark.parametrize("di,dj,dk,ba,bb", SPLIT_BW)
def test_split_backward_is_reproducible(di, dj, dk, ba, bb):
    # with phip_set_deterministic the tiles of a split product are added in a fixed order: the same bits
    # on every run (the default adds them with atomics: right to rounding, bits vary)
    d = pa.HIP(0)
    d.set_deterministic(True)
    rng = np.random.default_rng(di + dj + dk)
    bs = max(ba, bb)
    a = rng.standard_normal(di * dj * ba).astype(np.float32)
    b = rng.standard_normal(dj * dk * bb).astype(np.float32)
    gy = rng.standard_normal(di * dk * bs).astype(np.float32)
    ga0 = rng.standard_normal(a.size).astype(np.float32)
    gb0 = rng.standard_normal(b.size).astype(np.float32)
    ta = d.new_tensor_by_vector(pa.Shape([di, dj], ba), a)
    tb = d.new_tensor_by_vector(pa.Shape([dj, dk], bb), b)
    ty = d.matmul_fw(ta, tb)
    tgy = d.new_tensor_by_vector(ty.shape(), gy)

    def run():
        tga = d.new_tensor_by_vector(ta.shape(), ga0)
        tgb = d.new_tensor_by_vector(tb.shape(), gb0)
        d.matmul_bw(ta, tb, ty, tgy, tga, tgb)
        return tga.to_vector(), tgb.to_vector()

    ga, gb = run()
    rga, rgb = oracle.matmul_bw(a, b, gy, ga0, gb0, di, dj, dk, ba, bb, 8)
    assert norm_rel_err(ga, rga) <= F32_TOL and norm_rel_err(gb, rgb) <= F32_TOL
    for _ in range(12):
        ga2, gb2 = run()
        assert np.array_equal(ga, ga2) and np.array_equal(gb, gb2)
    d.close()



# shapes that reach the 256x256x64 large-tile kernel with ragged edges in every
# dimension (multiples of 8, not of 256 / 64), in each batch case
BIG_H16 = [  # di, dj, dk, ba, bb
    (2824, 2832, 2840, 1, 1),
    (776, 520, 1032, 16, 16),
    (136, 2824, 2832, 16, 1),
    (2824, 264, 712, 1, 4),
    # one partial K tile, and two K tiles of which the second is partial, in the forward product
    (4096, 24, 4096, 1, 1),
    (3080, 72, 3592, 1, 1),
    # too few 256 x 256 tiles for the chip: 128 x 128 tiles, all three products / per-sample / shared a
    (1480, 1608, 1544, 1, 1),
    (520, 392, 264, 12, 12),
    (1288, 1032, 40, 1, 40),
    # at most one such tile per CU: four K tiles resident or in flight; K of exactly 4 tiles, 5 with a tail
    # of 8, 3 (the two-stage form), and a long one
    (1032, 256, 776, 1, 1),
    (1024, 264, 1024, 1, 1),
    (1032, 192, 776, 1, 1),
    (776, 3080, 760, 1, 1),
    # 48 K tiles; 3 samples of 16 tiles summed into a shared operand's gradient
    (776, 3072, 760, 1, 1),
    (1024, 512, 1024, 1, 3),
    # one large shared a against at least 16 Ki columns: the forward product runs on a transposed copy of a
    # (both operands then contiguous along k); ragged in every dimension, K tail, odd dk
    (1032, 1048, 2049, 1, 8),
    (2824, 1032, 4100, 1, 4),
]


@pytest.mark.parametrize("which", ["f16", "bf16"])
@pytest.mark.parametrize("di,dj,dk,ba,bb", BIG_H16)
def test_large_tile_h16(dev16, devbf16, which, di, dj, dk, ba, bb):
    d = dev16 if which == "f16" else devbf16
    rng = np.random.default_rng(di + dj + dk + ba)
    bs = max(ba, bb)
    a = rng.standard_normal(di * dj * ba).astype(np.float32)
    b = rng.standard_normal(dj * dk * bb).astype(np.float32)
    gy = rng.standard_normal(di * dk * bs).astype(np.float32)
    ga0 = rng.standard_normal(a.size).astype(np.float32)
    gb0 = rng.standard_normal(b.size).astype(np.float32)
    y, ga, gb = _fw_bw(d, a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
    ry = oracle.matmul_fw(a, b, di, dj, dk, ba, bb, 8)
    rga, rgb = oracle.matmul_bw(a, b, gy, ga0, gb0, di, dj, dk, ba, bb, 8)
    assert norm_rel_err(y, ry) <= H16_TOL
    assert norm_rel_err(ga, rga) <= H16_TOL
    assert norm_rel_err(gb, rgb) <= H16_TOL
    # inputs exactly representable in 16 bits: only the output rounding is left
    r16 = (lambda x: x.astype(np.float16).astype(np.float32)) if which == "f16" else \
        (lambda x: (x.view(np.uint32) & 0xFFFF0000).view(np.float32))
    a, b, gy = r16(a), r16(b), r16(gy)
    z = lambda n: np.zeros(n, dtype=np.float32)
    y, ga, gb = _fw_bw(d, a, b, gy, z(a.size), z(b.size), di, dj, dk, ba, bb)
    ry = oracle.matmul_fw(a, b, di, dj, dk, ba, bb, 8)
    rga, rgb = oracle.matmul_bw(a, b, gy, z(a.size), z(b.size), di, dj, dk, ba, bb, 8)
    ulp = 2.0 ** -10 if which == "f16" else 2.0 ** -7
    for got, ref in ((y, ry), (ga, rga), (gb, rgb)):
        assert norm_rel_err(got, ref) <= ulp


def test_mid_tiles_take_four_stages_h16(dev16):
    # at most one 128 x 128 tile per CU: the launch with four LDS stages; more tiles than CUs: two stages
    rng = np.random.default_rng(3)
    for (di, dj, dk), want in (((1536, 1536, 1536), "h16_lds128_deep"), ((1024, 192, 1024), "h16_lds128"),
                               ((2304, 1024, 2048), "h16_lds128")):
        a = dev16.new_tensor_by_vector(pa.Shape([di, dj]), rng.standard_normal(di * dj).astype(np.float32))
        b = dev16.new_tensor_by_vector(pa.Shape([dj, dk]), rng.standard_normal(dj * dk).astype(np.float32))
        dev16.gemm_trace(True)
        y = dev16.matmul_fw(a, b)
        assert dev16.gemm_trace(False) == [want], (di, dj, dk)
        ref = a.to_vector().astype(np.float64).reshape(dj, di).T @ b.to_vector().astype(np.float64).reshape(dk, dj).T
        assert norm_rel_err(y.to_vector(), ref.T.reshape(-1)) <= H16_TOL


# few output tiles over a long K on the 16-bit devices: the K range is cut between
# workgroups that leave fp32 partial tiles, summed in order by a second launch
# (gb of the first two shapes, the forward product of the third)
@pytest.mark.parametrize("which", ["f16", "bf16"])
@pytest.mark.parametrize("di,dj,dk,ba,bb", [(4100, 520, 1, 1, 64), (2050, 130, 3, 1, 9), (70, 3000, 40, 1, 1),
                                            (1030, 48, 24, 6, 1)])
def test_long_k_few_tiles_h16(dev16, devbf16, which, di, dj, dk, ba, bb):
    d = dev16 if which == "f16" else devbf16
    rng = np.random.default_rng(di + dj + dk + ba)
    bs = max(ba, bb)
    r16 = (lambda x: x.astype(np.float16).astype(np.float32)) if which == "f16" else \
        (lambda x: (x.view(np.uint32) & 0xFFFF0000).view(np.float32))
    # inputs exactly representable in 16 bits: only the output rounding is left
    a = r16(rng.standard_normal(di * dj * ba).astype(np.float32))
    b = r16(rng.standard_normal(dj * dk * bb).astype(np.float32))
    gy = r16(rng.standard_normal(di * dk * bs).astype(np.float32))
    ga0 = r16(rng.standard_normal(a.size).astype(np.float32))
    gb0 = r16(rng.standard_normal(b.size).astype(np.float32))
    y, ga, gb = _fw_bw(d, a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
    ry = oracle.matmul_fw(a, b, di, dj, dk, ba, bb, 8)
    rga, rgb = oracle.matmul_bw(a, b, gy, ga0, gb0, di, dj, dk, ba, bb, 8)
    ulp = 2.0 ** -10 if which == "f16" else 2.0 ** -7
    for got, ref in ((y, ry), (ga, rga), (gb, rgb)):
        assert norm_rel_err(got, ref) <= ulp


# The per-timestep shapes on the 16-bit devices: a narrow side (the minibatch) against a weight
# matrix, forward and both gradients - the streamed-operand and paired-gradient lists of the fp32
# device, plus rows that are not 16-byte aligned (650, 1300, 518 columns of 16-bit values), ragged
# M / N / K, a minibatch of 1 and of 100, per-sample operands, a contraction over the minibatch.
# Inputs are exactly representable, so what is left is the one rounding of each output.
SKINNY_H16 = [  # di, dj, dk, ba, bb
    (10000, 650, 1, 1, 64),     # output projection
    (2048, 512, 1, 1, 64),      # recurrent gate
    (2600, 1300, 1, 1, 64),     # an LSTM layer with 650 hidden units
    (2600, 1300, 1, 1, 20),
    (256, 784, 1, 1, 128),      # dense layer
    (4100, 518, 1, 1, 40),
    (4100, 520, 2, 1, 30),
    (2052, 516, 1, 1, 60),
    (1028, 512, 48, 5, 1),      # the shared operand on the right: contraction over the minibatch
    (132, 260, 24, 6, 6),       # per-sample products
    (8192, 260, 1, 1, 1),
    (70, 3000, 40, 1, 1),       # long K, one tile
    (66, 70, 34, 1, 3),         # everything ragged and small
    (64, 64, 64, 1, 1),
    (800, 784, 1, 1, 100),
    (10, 800, 1, 1, 100),       # ten output rows
]


@pytest.mark.parametrize("which", ["f16", "bf16"])
@pytest.mark.parametrize("di,dj,dk,ba,bb", SKINNY_H16)
def test_per_timestep_shapes_h16(dev16, devbf16, which, di, dj, dk, ba, bb):
    d = dev16 if which == "f16" else devbf16
    rng = np.random.default_rng(di + 3 * dj + dk + ba)
    bs = max(ba, bb)
    r16 = (lambda x: x.astype(np.float16).astype(np.float32)) if which == "f16" else \
        (lambda x: (x.view(np.uint32) & 0xFFFF0000).view(np.float32))
    a = r16(rng.standard_normal(di * dj * ba).astype(np.float32))
    b = r16(rng.standard_normal(dj * dk * bb).astype(np.float32))
    gy = r16(rng.standard_normal(di * dk * bs).astype(np.float32))
    ga0 = r16(rng.standard_normal(a.size).astype(np.float32))
    gb0 = r16(rng.standard_normal(b.size).astype(np.float32))
    d.gemm_trace(True)
    y, ga, gb = _fw_bw(d, a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
    kernels = d.gemm_trace(False)
    if dj % 2 == 0 and di % 2 == 0:          # the kernel this list is for
        assert kernels[0].startswith("h16_skinny"), kernels
        # (a contraction over fewer than 16 values, e.g. the weight gradient of a minibatch of one, is left to the staged kernel)
        assert min(di, dj, dk * bb) < 16 or all(k.startswith("h16_skinny") for k in kernels), kernels
    ry = oracle.matmul_fw(a, b, di, dj, dk, ba, bb, 8)
    rga, rgb = oracle.matmul_bw(a, b, gy, ga0, gb0, di, dj, dk, ba, bb, 8)
    ulp = 2.0 ** -10 if which == "f16" else 2.0 ** -7
    for name, got, ref in (("y", y, ry), ("ga", ga, rga), ("gb", gb, rgb)):
        assert norm_rel_err(got, ref) <= ulp, name
    # again, over pool memory that holds the first call's results: an overwriting product must not add
    y2, ga2, gb2 = _fw_bw(d, a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
    assert np.array_equal(y2, y) and np.array_equal(ga2, ga) and np.array_equal(gb2, gb)     # and the same bits


# a long contraction against few output tiles: K ranges of more than 18 K tiles, which the 32 x 32 tiles walk in
# rounds through two halves of LDS - K not a multiple of 64 or of 8, a contraction that runs over the
# minibatch (its K tiles restart with every sample), one to five rounds, with and without a cut between workgroups
LONG_K_H16 = [  # di, dj, dk, ba, bb
    (34, 5000, 20, 1, 1),
    (40, 2890, 30, 1, 1),
    (650, 10000, 1, 1, 20),
    (96, 1234, 64, 1, 1),
    (20, 1300, 2, 1, 64),
    (1300, 130, 48, 9, 1),
    (3000, 64, 64, 1, 1),
    (2600, 34, 36, 3, 1),
]


@pytest.mark.parametrize("which", ["f16", "bf16"])
@pytest.mark.parametrize("di,dj,dk,ba,bb", LONG_K_H16)
def test_long_k_narrow_h16(dev16, devbf16, which, di, dj, dk, ba, bb):
    d = dev16 if which == "f16" else devbf16
    rng = np.random.default_rng(7 * di + dj + 13 * dk + ba)
    bs = max(ba, bb)
    r16 = (lambda x: x.astype(np.float16).astype(np.float32)) if which == "f16" else \
        (lambda x: (x.view(np.uint32) & 0xFFFF0000).view(np.float32))
    a = r16(rng.standard_normal(di * dj * ba).astype(np.float32))
    b = r16(rng.standard_normal(dj * dk * bb).astype(np.float32))
    gy = r16(rng.standard_normal(di * dk * bs).astype(np.float32))
    ga0 = r16(rng.standard_normal(a.size).astype(np.float32))
    gb0 = r16(rng.standard_normal(b.size).astype(np.float32))
    y, ga, gb = _fw_bw(d, a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
    ry = oracle.matmul_fw(a, b, di, dj, dk, ba, bb, 8)
    rga, rgb = oracle.matmul_bw(a, b, gy, ga0, gb0, di, dj, dk, ba, bb, 8)
    ulp = 2.0 ** -10 if which == "f16" else 2.0 ** -7
    for name, got, ref in (("y", y, ry), ("ga", ga, rga), ("gb", gb, rgb)):
        assert norm_rel_err(got, ref) <= ulp, name
    y2, ga2, gb2 = _fw_bw(d, a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
    assert np.array_equal(y2, y) and np.array_equal(ga2, ga) and np.array_equal(gb2, gb)


def test_f16_matches_oracle_on_rounded_inputs(dev16):
    # With inputs already representable in fp16 the only error left is the
    # final rounding of the output (<= 2^-11 relative per element) on top of
    # fp32 accumulation: a far tighter gate than 2e-2.
    rng = np.random.default_rng(5)
    di, dj, dk, ba, bb = 200, 160, 72, 1, 3
    r16 = lambda x: x.astype(np.float16).astype(np.float32)
    a = r16(rng.standard_normal(di * dj * ba).astype(np.float32))
    b = r16(rng.standard_normal(dj * dk * bb).astype(np.float32))
    gy = r16(rng.standard_normal(di * dk * bb).astype(np.float32))
    z = lambda n: np.zeros(n, dtype=np.float32)
    y, ga, gb = _fw_bw(dev16, a, b, gy, z(a.size), z(b.size), di, dj, dk, ba, bb)
    ry = np_matmul_fw(a, b, di, dj, dk, ba, bb)
    rga, rgb = np_matmul_bw(a, b, gy, di, dj, dk, ba, bb)
    for got, ref in ((y, ry), (ga, rga), (gb, rgb)):
        ref16 = ref.astype(np.float16).astype(np.float64)
        # allow one fp16 ULP of the largest magnitude for accumulation-order ties
        assert np.max(np.abs(got - ref16)) <= np.max(np.abs(ref)) * 2.0 ** -10


# ---- properties that hold at any size ------------------------------------------

def test_backward_accumulates_and_forward_overwrites(dev):
    rng = np.random.default_rng(11)
    di, dj, dk, ba, bb = 96, 80, 48, 1, 4
    a = rng.standard_normal(di * dj).astype(np.float32)
    b = rng.standard_normal(dj * dk * bb).astype(np.float32)
    gy = rng.standard_normal(di * dk * bb).astype(np.float32)
    ta = dev.new_tensor_by_vector(pa.Shape([di, dj]), a)
    tb = dev.new_tensor_by_vector(pa.Shape([dj, dk], bb), b)
    ty = dev.matmul_fw(ta, tb)
    tgy = dev.new_tensor_by_vector(ty.shape(), gy)
    ga = dev.new_tensor_by_constant(ta.shape(), 0)
    gb = dev.new_tensor_by_constant(tb.shape(), 0)
    dev.matmul_bw(ta, tb, ty, tgy, ga, gb)
    ga1, gb1 = ga.to_vector(), gb.to_vector()
    dev.matmul_bw(ta, tb, ty, tgy, ga, gb)
    assert norm_rel_err(ga.to_vector(), 2 * ga1) <= 1e-6
    assert norm_rel_err(gb.to_vector(), 2 * gb1) <= 1e-6
    # forward into a block that held other data gives the same result
    y1 = ty.to_vector()
    del ty
    junk = dev.new_tensor_by_constant(pa.Shape([di, dk], bb), 123.0)
    del junk
    assert np.array_equal(dev.matmul_fw(ta, tb).to_vector(), y1)


def test_copy_on_write_gradient(dev):
    # a gradient tensor that shares its block must be cloned before the
    # backward pass adds into it (primitiv/core/tensor.cc:33-41)
    a = dev.new_tensor_by_vector([2, 2], [1, 2, 3, 4])
    b = dev.new_tensor_by_vector([2, 2], [1, 0, 0, 2])
    y = dev.matmul_fw(a, b)
    gy = dev.new_tensor_by_vector([2, 2], [1, -1, 2, -2])
    ga = dev.new_tensor_by_constant([2, 2], 0)
    gb = dev.new_tensor_by_constant([2, 2], 0)
    shared = ga.copy()
    dev.matmul_bw(a, b, y, gy, ga, gb)
    assert vector_match([1, -1, 4, -4], ga.to_vector())
    assert vector_match([0, 0, 0, 0], shared.to_vector())


def test_broadcast_equals_tiled(dev):
    rng = np.random.default_rng(13)
    di, dj, dk, n = 70, 50, 30, 6
    a = rng.standard_normal(di * dj).astype(np.float32)
    b = rng.standard_normal(dj * dk * n).astype(np.float32)
    gy = rng.standard_normal(di * dk * n).astype(np.float32)
    z = lambda m: np.zeros(m, dtype=np.float32)
    y1, ga1, gb1 = _fw_bw(dev, a, b, gy, z(a.size), z(b.size), di, dj, dk, 1, n)
    at = np.tile(a, n)
    yn, gan, gbn = _fw_bw(dev, at, b, gy, z(at.size), z(b.size), di, dj, dk, n, n)
    assert norm_rel_err(y1, yn) <= 1e-6
    assert norm_rel_err(gb1, gbn) <= 1e-6
    assert norm_rel_err(ga1, gan.reshape(n, -1).sum(0)) <= 1e-5


# ---- the benchmark workloads at full size --------------------------------------

def _run_workload(dev, w, steps):
    a, bs, gys = w.inputs(seed=0, steps=steps)
    ta = dev.new_tensor_by_vector(pa.Shape([w.di, w.dj], w.ba), a)
    ga = dev.new_tensor_by_constant(ta.shape(), 0)
    outs = []
    for t in range(steps):
        tb = dev.new_tensor_by_vector(pa.Shape([w.dj, w.dk], w.bb), bs[t])
        ty = dev.matmul_fw(ta, tb)
        tgy = dev.new_tensor_by_vector(ty.shape(), gys[t])
        gb = dev.new_tensor_by_constant(tb.shape(), 0)
        dev.matmul_bw(ta, tb, ty, tgy, ga, gb)   # ga persists across steps
        outs.append((ty.to_vector(), gb.to_vector()))
    return a, bs, gys, outs, ga.to_vector()


@pytest.mark.parametrize("name,steps", [("dense", 1), ("rnn_gate", 30), ("square_batched", 1),
                                        ("output_projection", 35)])
def test_workload_f32(dev, name, steps):
    w = WORKLOADS[name]
    a, bs, gys, outs, ga = _run_workload(dev, w, steps)
    rga = np.zeros(a.size, dtype=np.float32)
    for t in range(steps):
        ry = oracle.matmul_fw(a, bs[t], w.di, w.dj, w.dk, w.ba, w.bb, 8)
        rga, rgb = oracle.matmul_bw(a, bs[t], gys[t], rga, np.zeros(bs[t].size, np.float32),
                                    w.di, w.dj, w.dk, w.ba, w.bb, 8)
        assert norm_rel_err(outs[t][0], ry) <= w.tolerance, "%s step %d y" % (name, t)
        assert norm_rel_err(outs[t][1], rgb) <= w.tolerance, "%s step %d gb" % (name, t)
    assert norm_rel_err(ga, rga) <= w.tolerance, name + " ga"


@pytest.fixture(scope="module")
def half_storage_inputs():
    w = WORKLOADS["half_storage"]
    a, bs, gys = w.inputs(seed=0)
    return w, a, bs[0], gys[0]


def _tile_edge_indices(n, tile=256):
    """Indices on both sides of the first, a middle and the last boundary of `tile`-wide tiles, and the ends."""
    mid = (n // tile // 2) * tile
    last = (n - 1) // tile * tile
    return np.unique(np.clip([0, 1, tile - 1, tile, mid - 1, mid, last - 1, last, n - 2, n - 1], 0, n - 1))


@pytest.mark.parametrize("which", ["f16", "bf16"])
def test_workload_half_storage_strips(dev16, devbf16, half_storage_inputs, which):
    # Full size on the GPU.  The oracle's arithmetic (fp32 products of the un-rounded inputs; any row of an
    # output depends only on the same row of one operand, any column on one column of the other) is redone
    # here by the library's fp32 matrix product for COMPLETE rows and columns of y, ga and gb on both sides
    # of the first, a middle and the last 256-wide tile boundary and at both ends: ten full rows and ten
    # full columns of each output, 1.1 M to 0.33 M elements per strip set.  Gate: max|x - ref| / max|ref|
    # <= 2e-2 per strip set, as for every 16-bit result.
    d = dev16 if which == "f16" else devbf16
    w, a, b, gy = half_storage_inputs
    di, dj, dk, n = w.di, w.dj, w.dk, w.bb
    ta = d.new_tensor_by_vector(pa.Shape([di, dj]), a)
    tb = d.new_tensor_by_vector(pa.Shape([dj, dk], n), b)
    ty = d.matmul_fw(ta, tb)
    tgy = d.new_tensor_by_vector(ty.shape(), gy)
    ga = d.new_tensor_by_constant(ta.shape(), 0)
    gb = d.new_tensor_by_constant(tb.shape(), 0)
    d.matmul_bw(ta, tb, ty, tgy, ga, gb)
    y = ty.to_vector().reshape(n * dk, di)        # [column of Y'][row]
    gav = ga.to_vector().reshape(dj, di)          # [j][i]
    gbv = gb.to_vector().reshape(n * dk, dj)      # [column][j]
    del ta, tb, ty, tgy, ga, gb
    A = a.reshape(dj, di)                         # A[j][i]
    B = b.reshape(n * dk, dj)                     # B'[col][j]
    GY = gy.reshape(n * dk, di)                   # gY'[col][i]
    rows, jcols, cols = _tile_edge_indices(di), _tile_edge_indices(dj), _tile_edge_indices(n * dk)
    tol = w.tolerance
    # y = a . B':  y[col][i] = sum_j B'[col][j] A[j][i]
    assert norm_rel_err(y[:, rows], B @ A[:, rows]) <= tol                 # full rows of y
    assert norm_rel_err(y[cols], B[cols] @ A) <= tol                       # full columns of y
    # ga[j][i] = sum_col B'[col][j] gY'[col][i]
    assert norm_rel_err(gav[:, rows], B.T @ GY[:, rows]) <= tol            # full rows of ga (all j)
    assert norm_rel_err(gav[jcols], B[:, jcols].T @ GY) <= tol             # full columns of ga (all i)
    # gb[col][j] = sum_i gY'[col][i] A[j][i]
    assert norm_rel_err(gbv[:, jcols], GY @ A[jcols].T) <= tol             # full rows of gb (all columns)
    assert norm_rel_err(gbv[cols], GY[cols] @ A.T) <= tol                  # full columns of gb (all j)
