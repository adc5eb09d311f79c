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
