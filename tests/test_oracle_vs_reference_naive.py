"""Pins the CPU oracle against primitiv's own plain CPU device (devices::Naive), compiled from the
primitiv source tree where it lies and driven through its Device front.  Needs that tree and g++
(the build container); skipped elsewhere.  No GPU needed.

The Naive device accumulates a product's terms one by one in float (devices/naive/ops/matmul.cc),
the oracle follows the Eigen device's blocked order, so products of random operands agree to
rounding (1e-5 of the largest element); on small integers every partial sum is exact in float and
the two must agree bit for bit whatever the order.
"""
import numpy as np
import pytest

import host_class_lib as hc
import oracle
import primitiv_amd as pa
from util import norm_rel_err

pytestmark = pytest.mark.skipif(not hc.available(), reason=hc.REASON)

S = pa.Shape

CASES = [  # di, dj, dk, ba, bb
    (1, 1, 1, 1, 1), (1, 7, 1, 1, 1), (5, 1, 3, 1, 4), (3, 4, 6, 1, 1), (17, 9, 5, 3, 3), (17, 9, 5, 1, 3),
    (17, 9, 5, 3, 1), (33, 65, 31, 2, 2), (40, 37, 19, 1, 5), (64, 64, 16, 4, 1), (50, 101, 7, 1, 1),
]


@pytest.fixture(scope="module")
def naive():
    d = hc.HostDevice("naive")
    yield d
    d.close()


def _operands(rng, n, integers):
    if integers:
        return rng.integers(-4, 5, n).astype(np.float32)
    return rng.standard_normal(n).astype(np.float32)


def _run_reference(naive, a, b, gy, ga0, gb0, di, dj, dk, ba, bb):
    bs = max(ba, bb)
    ta, tb = naive.new_tensor_by_vector(S([di, dj], ba), a), naive.new_tensor_by_vector(S([dj, dk], bb), b)
    ty = naive.matmul_fw(ta, tb)
    tga, tgb = naive.new_tensor_by_vector(S([di, dj], ba), ga0), naive.new_tensor_by_vector(S([dj, dk], bb), gb0)
    naive.matmul_bw(ta, tb, ty, naive.new_tensor_by_vector(S([di, dk], bs), gy), tga, tgb)
    return np.asarray(ty.to_vector()), np.asarray(tga.to_vector()), np.asarray(tgb.to_vector())


@pytest.mark.parametrize("integers", [True, False])
def test_matmul_forward_backward_match_the_reference_device(naive, integers):
    rng = np.random.default_rng(11)
    for di, dj, dk, ba, bb in CASES:
        bs = max(ba, bb)
        a, b = _operands(rng, di * dj * ba, integers), _operands(rng, dj * dk * bb, integers)
        gy = _operands(rng, di * dk * bs, integers)
        ga0, gb0 = _operands(rng, di * dj * ba, integers), _operands(rng, dj * dk * bb, integers)   # gradients accumulate
        y_ref, ga_ref, gb_ref = _run_reference(naive, a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
        y = oracle.matmul_fw(a, b, di, dj, dk, ba, bb)
        ga, gb = oracle.matmul_bw(a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
        case = (di, dj, dk, ba, bb)
        if integers:
            assert np.array_equal(y, y_ref), case
            assert np.array_equal(ga, ga_ref), case
            assert np.array_equal(gb, gb_ref), case
        else:
            assert norm_rel_err(y, y_ref) <= 1e-5, case
            assert norm_rel_err(ga, ga_ref) <= 1e-5, case
            assert norm_rel_err(gb, gb_ref) <= 1e-5, case


def test_a_wrong_oracle_would_be_caught(naive):
    # the check above has teeth: the gradients of swapped operands differ from the reference device's
    rng = np.random.default_rng(12)
    di, dj, dk = 5, 4, 3
    a, b, gy = _operands(rng, di * dj, True), _operands(rng, dj * dk, True), _operands(rng, di * dk, True)
    zero_a, zero_b = np.zeros(di * dj, np.float32), np.zeros(dj * dk, np.float32)
    _, ga_ref, gb_ref = _run_reference(naive, a, b, gy, zero_a, zero_b, di, dj, dk, 1, 1)
    ga, gb = oracle.matmul_bw(a, b, -gy, zero_a, zero_b, di, dj, dk, 1, 1)
    assert not np.array_equal(ga, ga_ref) and not np.array_equal(gb, gb_ref)


def test_inplace_add_and_batch_sum_match_the_reference_device(naive):
    rng = np.random.default_rng(13)
    for volume, bx, by in [(7, 1, 1), (12, 3, 3), (12, 1, 4), (12, 5, 1), (1, 6, 1)]:
        x, y = _operands(rng, volume * bx, False), _operands(rng, volume * by, False)
        tx, ty = naive.new_tensor_by_vector(S([volume], bx), x), naive.new_tensor_by_vector(S([volume], by), y)
        naive.inplace_add(tx, ty)
        mine = oracle.inplace_add(x, y, volume, bx, by)
        assert norm_rel_err(mine, ty.to_vector()) <= 1e-6, (volume, bx, by)
    for volume, bs in [(9, 1), (9, 4), (1, 7), (33, 16)]:
        x = _operands(rng, volume * bs, False)
        ref = naive.batch_sum_fw(naive.new_tensor_by_vector(S([volume], bs), x)).to_vector()
        assert norm_rel_err(oracle.batch_sum(x, volume, bs), ref) <= 1e-6, (volume, bs)


# ---- the widened rows: the same call on primitiv's Naive device and on devices::HIP over the host
# stand-in, whose arithmetic is the oracle's (tests/host_class/phip_host_stub.cc) -----------------

@pytest.fixture(scope="module")
def mine():
    d = hc.HostDevice("f32")
    yield d
    d.close()


def _ulps(a, b):
    a, b = np.asarray(a, np.float32), np.asarray(b, np.float32)
    ia, ib = a.view(np.int32).astype(np.int64), b.view(np.int32).astype(np.int64)
    ia = np.where(ia < 0, -(ia & 0x7fffffff), ia)
    ib = np.where(ib < 0, -(ib & 0x7fffffff), ib)
    d = np.abs(ia - ib)
    d[np.isnan(a) & np.isnan(b)] = 0
    return int(d.max()) if d.size else 0


def _both(naive, mine, fn):
    return np.asarray(fn(naive)), np.asarray(fn(mine))


def test_elementwise_families_match_the_reference_device(naive, mine):
    rng = np.random.default_rng(21)
    shape = S([5, 3], 4)
    x = (rng.standard_normal(60) * 1.5).astype(np.float32)
    xp = np.abs(x) + 0.25                                   # sqrt, log, pow want positive arguments
    gy = rng.standard_normal(60).astype(np.float32)
    x2 = rng.standard_normal(60).astype(np.float32)
    for op in pa.HIP.UNARY_OPS:
        arg = xp if op in ("sqrt", "log") else x
        def fw(d):
            return d.unary_fw(op, d.new_tensor_by_vector(shape, arg)).to_vector()
        def bw(d):
            tx = d.new_tensor_by_vector(shape, arg)
            ty = d.unary_fw(op, tx)
            gx = d.new_tensor_by_vector(shape, gy * 0.5)   # gradients accumulate
            d.unary_bw(op, tx, ty, d.new_tensor_by_vector(shape, gy), gx)
            return gx.to_vector()
        assert _ulps(*_both(naive, mine, fw)) <= 4, op      # test/test_utils.h:26-45 grants 4 on a 32-bit device
        if op != "negate":                                  # the Device interface has no negate_bw
            assert _ulps(*_both(naive, mine, bw)) <= 4, op
    for op in pa.HIP.CONST_OPS:
        arg = xp if op in ("pow_const_r", "pow_const_l") else x
        for k in (0.75, 2.5):
            def fw(d):
                return d.const_fw(op, d.new_tensor_by_vector(shape, arg), k).to_vector()
            def bw(d):
                tx = d.new_tensor_by_vector(shape, arg)
                ty = d.const_fw(op, tx, k)
                gx = d.new_tensor_by_vector(shape, gy * 0.5)
                d.const_bw(op, tx, ty, d.new_tensor_by_vector(shape, gy), k, gx)
                return gx.to_vector()
            assert _ulps(*_both(naive, mine, fw)) <= 4, (op, k)
            assert _ulps(*_both(naive, mine, bw)) <= 4, (op, k)
    for op in pa.HIP.BINARY_OPS:
        for ba, bb in ((4, 4), (1, 4), (4, 1)):
            a = xp[:15 * ba] if op == "pow" else x[:15 * ba]
            b = x2[:15 * bb] + (3.0 if op == "divide" else 0.0)
            def fw(d):
                return d.binary_fw(op, d.new_tensor_by_vector(S([5, 3], ba), a), d.new_tensor_by_vector(S([5, 3], bb), b)).to_vector()
            def bw(d):
                ta, tb = d.new_tensor_by_vector(S([5, 3], ba), a), d.new_tensor_by_vector(S([5, 3], bb), b)
                ty = d.binary_fw(op, ta, tb)
                ga, gb = d.new_tensor_by_constant(S([5, 3], ba), 0.5), d.new_tensor_by_constant(S([5, 3], bb), -0.25)
                d.binary_bw(op, ta, tb, ty, d.new_tensor_by_vector(S([5, 3], max(ba, bb)), gy[:15 * max(ba, bb)]), ga, gb)
                return np.concatenate([ga.to_vector(), gb.to_vector()])
            assert _ulps(*_both(naive, mine, fw)) <= 4, (op, ba, bb)
            r, m = _both(naive, mine, bw)
            assert norm_rel_err(m, r) <= 2e-6, (op, ba, bb)   # sums over the minibatch: order of addition


def test_moving_and_reducing_operations_match_the_reference_device(naive, mine):
    rng = np.random.default_rng(22)
    shape = S([4, 3, 5], 2)
    x = rng.standard_normal(120).astype(np.float32)
    def run(fn):
        r, m = _both(naive, mine, fn)
        return r, m
    for dim in (0, 1, 2):
        for op in ("sum", "logsumexp", "max", "min"):
            r, m = run(lambda d: d.reduce_fw(op, d.new_tensor_by_vector(shape, x), dim).to_vector())
            if op == "logsumexp":      # log of a sum near 1 cancels to near 0: ULPs of the result mean nothing
                assert np.max(np.abs(r - m)) <= 2e-7 * max(1.0, np.max(np.abs(r))), (op, dim)
            else:
                assert _ulps(r, m) <= 4, (op, dim)
        r, m = run(lambda d: d.flip_fw(d.new_tensor_by_vector(shape, x), dim).to_vector())
        assert np.array_equal(r, m)
        r, m = run(lambda d: d.slice_fw(d.new_tensor_by_vector(shape, x), dim, 1, 3).to_vector())
        assert np.array_equal(r, m)
        r, m = run(lambda d: d.pick_fw(d.new_tensor_by_vector(shape, x), [2, 0], dim).to_vector())
        assert np.array_equal(r, m)
        r, m = run(lambda d: d.concat_fw([d.new_tensor_by_vector(shape, x), d.new_tensor_by_vector(shape, -x)], dim).to_vector())
        assert np.array_equal(r, m)
        r, m = run(lambda d: np.asarray(d.arg_extremum("max", d.new_tensor_by_vector(shape, x), dim), dtype=np.float32))
        assert np.array_equal(r, m)
    r, m = run(lambda d: d.permute_dims_fw(d.new_tensor_by_vector(shape, x), [2, 0, 1]).to_vector())
    assert np.array_equal(r, m)
    r, m = run(lambda d: d.transpose_fw(d.new_tensor_by_vector(S([4, 5], 3), x[:60])).to_vector())
    assert np.array_equal(r, m)
    r, m = run(lambda d: d.broadcast_fw(d.new_tensor_by_vector(S([4, 1, 5], 2), x[:40]), 1, 3).to_vector())
    assert np.array_equal(r, m)
    r, m = run(lambda d: d.batch_pick_fw(d.new_tensor_by_vector(S([4, 3], 5), x[:60]), [4, 0, 0]).to_vector())
    assert np.array_equal(r, m)


def test_convolution_and_pooling_match_the_reference_device(naive, mine):
    rng = np.random.default_rng(23)
    x = rng.standard_normal(7 * 6 * 3 * 2).astype(np.float32)
    w = rng.standard_normal(3 * 2 * 3 * 4).astype(np.float32)
    for p in ((0, 0, 1, 1, 1, 1), (1, 1, 2, 1, 1, 1), (2, 1, 1, 2, 2, 1)):      # padding, stride, dilation
        def fw(d):
            return d.conv2d_fw(d.new_tensor_by_vector(S([7, 6, 3], 2), x), d.new_tensor_by_vector(S([3, 2, 3, 4]), w), *p).to_vector()
        r, m = _both(naive, mine, fw)
        assert r.shape == m.shape and norm_rel_err(m, r) <= 2e-6, p
        def bw(d):
            tx, tw = d.new_tensor_by_vector(S([7, 6, 3], 2), x), d.new_tensor_by_vector(S([3, 2, 3, 4]), w)
            ty = d.conv2d_fw(tx, tw, *p)
            gy = d.new_tensor_by_vector(ty.shape(), np.linspace(-1, 1, ty.shape().size()).astype(np.float32))
            gx, gw = d.new_tensor_by_constant(tx.shape(), 0), d.new_tensor_by_constant(tw.shape(), 0)
            d.conv2d_bw(tx, tw, ty, gy, *p, gx, gw)
            return np.concatenate([gx.to_vector(), gw.to_vector()])
        r, m = _both(naive, mine, bw)
        assert norm_rel_err(m, r) <= 2e-6, p
    for p in ((2, 2, 0, 0, 2, 2), (3, 2, 1, 1, 2, 1)):                          # window, padding, stride
        def fw(d):
            return d.max_pool2d_fw(d.new_tensor_by_vector(S([7, 6, 3], 2), x), *p).to_vector()
        r, m = _both(naive, mine, fw)
        assert np.array_equal(r, m), p
