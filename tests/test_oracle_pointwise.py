"""The CPU oracle's elementwise operations against the reference's golden vectors.

Every case of tests/golden/pointwise_vectors.json (transcribed from
test/tensor_forward_test.cc, test/tensor_backward_test.cc and
test/tensor_test.cc of the reference) is replayed on the oracle with the ULP
bound the reference's own test grants a 32-bit device.  What those tests leave
to closed forms (the pow gradients) or do not cover (larger random inputs) is
checked against float64 library routines.
"""
import numpy as np
import pytest

import oracle
from pointwise_cases import CASES, run_case_on, case_id
from util import ulp_diff


class OracleBackend:
    """Runs a golden case on the oracle."""
    unary_fw = staticmethod(oracle.unary_fw)
    unary_bw = staticmethod(oracle.unary_bw)
    const_fw = staticmethod(oracle.const_fw)
    const_bw = staticmethod(oracle.const_bw)
    pown_fw = staticmethod(oracle.pown_fw)
    pown_bw = staticmethod(oracle.pown_bw)
    scalar_fw = staticmethod(oracle.scalar_fw)
    binary_fw = staticmethod(oracle.binary_fw)
    binary_bw = staticmethod(oracle.binary_bw)
    inplace_subtract = staticmethod(oracle.inplace_subtract)
    inplace_multiply_const = staticmethod(oracle.inplace_multiply_const)
    identity = staticmethod(oracle.identity)


@pytest.mark.parametrize("case", CASES, ids=case_id)
def test_oracle_matches_reference_vectors(case):
    for got, want in run_case_on(OracleBackend, case):
        want = np.asarray(want, dtype=np.float32)
        assert got.shape == want.shape
        assert int(ulp_diff(got, want).max()) <= case["ulps"], (got, want)


def test_pow_gradients_follow_their_closed_forms():
    # test/tensor_backward_test.cc:680-728 (pow_const_r / pow_const_l) and :1477-1597
    # (pow 11/NN/1N/N1) state the expected gradients as formulas, not vectors.
    x = np.array([1, 2, 4, 8, 16, 32, 64, 128], dtype=np.float32)
    for k in (1., .5, .25, 0, -.125, -.25, -.5, -.1):
        y = oracle.const_fw("pow_const_r", x, k)
        gx = oracle.const_bw("pow_const_r", x, y, np.ones_like(x), k, np.zeros_like(x))
        want = (np.float32(k) * np.power(x.astype(np.float64), np.float64(np.float32(k)) - 1)).astype(np.float32)
        assert int(ulp_diff(gx, want).max()) <= 4
    x = np.array([1., .5, .25, 0, -.125, -.25, -.5, -1.], dtype=np.float32)
    for k in (1, 2, 4, 8, 16, 32, 64, 128):
        y = oracle.const_fw("pow_const_l", x, k)
        gx = oracle.const_bw("pow_const_l", x, y, np.ones_like(x), k, np.zeros_like(x))
        want = (np.log(np.float64(k)) * np.power(np.float64(k), x.astype(np.float64))).astype(np.float32)
        assert int(ulp_diff(gx, want).max()) <= 4
    a = np.array([1, 2, 4, 8], dtype=np.float32)
    b = np.array([2, 1, 0, -1], dtype=np.float32)
    for ba, bb in ((1, 1), (2, 2), (1, 2), (2, 1)):
        aa, bbv = np.tile(a, ba), np.tile(b, bb)
        bs = max(ba, bb)
        y = oracle.binary_fw("pow", aa, bbv, 4, ba, bb)
        ga, gb = oracle.binary_bw("pow", aa, bbv, y, np.ones(4 * bs, np.float32), np.zeros(4 * ba, np.float32),
                                  np.zeros(4 * bb, np.float32), 4, ba, bb)
        a64, b64 = a.astype(np.float64), b.astype(np.float64)
        fga = b64 * np.power(a64, b64 - 1)
        fgb = np.log(a64) * np.power(a64, b64)
        want_ga = np.tile(fga, ba) * (bs if ba == 1 else 1)
        want_gb = np.tile(fgb, bb) * (bs if bb == 1 else 1)
        assert int(ulp_diff(ga, want_ga.astype(np.float32)).max()) <= 4
        assert int(ulp_diff(gb, want_gb.astype(np.float32)).max()) <= 4


NUMPY_UNARY = {
    "negate": np.negative, "abs": np.abs, "sqrt": np.sqrt, "exp": np.exp, "log": np.log, "tanh": np.tanh,
    "sigmoid": lambda x: 1 / (1 + np.exp(-x)), "softplus": lambda x: np.logaddexp(0, x), "sin": np.sin,
    "cos": np.cos, "tan": np.tan,
}
NUMPY_UNARY_GRAD = {
    "abs": np.sign, "sqrt": lambda x: .5 / np.sqrt(x), "exp": np.exp, "log": lambda x: 1 / x,
    "tanh": lambda x: 1 - np.tanh(x) ** 2, "sigmoid": lambda x: np.exp(-x) / (1 + np.exp(-x)) ** 2,
    "softplus": lambda x: 1 / (1 + np.exp(-x)), "sin": np.cos, "cos": lambda x: -np.sin(x),
    "tan": lambda x: 1 / np.cos(x) ** 2,
}


@pytest.mark.parametrize("op", oracle.UNARY_OPS)
def test_unary_against_float64_library(op):
    rng = np.random.default_rng(7)
    x = rng.uniform(0.1, 3.0, 4096).astype(np.float32)
    if op not in ("sqrt", "log"):
        x *= rng.choice([-1, 1], x.size).astype(np.float32)
    y = oracle.unary_fw(op, x)
    want = NUMPY_UNARY[op](x.astype(np.float64))
    assert np.max(np.abs(y - want) / np.maximum(np.abs(want), 1e-30)) < 1e-5
    if op == "negate":
        return
    gy = rng.standard_normal(x.size).astype(np.float32)
    g0 = rng.standard_normal(x.size).astype(np.float32)
    gx = oracle.unary_bw(op, x, y, gy, g0)
    want = g0 + NUMPY_UNARY_GRAD[op](x.astype(np.float64)) * gy
    assert np.max(np.abs(gx - want)) < 1e-4 * max(1.0, float(np.max(np.abs(want))))


@pytest.mark.parametrize("op", oracle.BINARY_OPS)
@pytest.mark.parametrize("ba,bb", [(1, 1), (3, 3), (1, 3), (3, 1)])
def test_binary_against_float64_library(op, ba, bb):
    rng = np.random.default_rng(ba * 10 + bb)
    volume, bs = 37, max(ba, bb)
    a = rng.uniform(0.5, 2.0, volume * ba).astype(np.float32)
    b = rng.uniform(0.5, 2.0, volume * bb).astype(np.float32)
    A = np.broadcast_to(a.reshape(ba, volume).astype(np.float64), (bs, volume))
    B = np.broadcast_to(b.reshape(bb, volume).astype(np.float64), (bs, volume))
    f = {"add": A + B, "subtract": A - B, "multiply": A * B, "divide": A / B, "pow": A ** B}[op]
    y = oracle.binary_fw(op, a, b, volume, ba, bb)
    assert np.allclose(y, f.reshape(-1), rtol=1e-6)
    gy = rng.standard_normal(volume * bs).astype(np.float32)
    G = gy.reshape(bs, volume).astype(np.float64)
    da = {"add": G, "subtract": G, "multiply": G * B, "divide": G / B, "pow": G * B * A ** (B - 1)}[op]
    db = {"add": G, "subtract": -G, "multiply": G * A, "divide": -G * A / B ** 2, "pow": G * np.log(A) * A ** B}[op]
    ga0 = rng.standard_normal(a.size).astype(np.float32)
    gb0 = rng.standard_normal(b.size).astype(np.float32)
    ga, gb = oracle.binary_bw(op, a, b, y, gy, ga0, gb0, volume, ba, bb)
    want_ga = ga0 + (da.sum(axis=0) if ba == 1 and bs > 1 else da.reshape(-1))
    want_gb = gb0 + (db.sum(axis=0) if bb == 1 and bs > 1 else db.reshape(-1))
    assert np.allclose(ga, want_ga, rtol=1e-5, atol=1e-5)
    assert np.allclose(gb, want_gb, rtol=1e-5, atol=1e-5)
