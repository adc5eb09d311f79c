"""Pins the CPU oracle: reference golden vectors, float64 library products,
brute force, and algebraic invariants.  No GPU needed."""
import numpy as np
import pytest

import oracle
from util import norm_rel_err, np_matmul_bw, np_matmul_fw, vector_match

CASES = [  # di, dj, dk, ba, bb
    (1, 1, 1, 1, 1), (1, 7, 1, 1, 1), (5, 1, 3, 1, 4), (3, 4, 6, 1, 1),
    (17, 9, 5, 3, 3), (17, 9, 5, 1, 3), (17, 9, 5, 3, 1), (33, 65, 31, 2, 2),
    (200, 37, 19, 1, 5), (64, 64, 64, 4, 1), (250, 401, 7, 1, 1),
]


def _rand(rng, n):
    return rng.standard_normal(n).astype(np.float32)


def test_golden_forward(golden):
    for c in golden["matmul_fw"]:
        y = oracle.matmul_fw(c["a"], c["b"], c["di"], c["dj"], c["dk"], c["ba"], c["bb"])
        assert vector_match(c["y"], y), c["source"]
        y64 = oracle.matmul_fw_f64(c["a"], c["b"], c["di"], c["dj"], c["dk"], c["ba"], c["bb"])
        assert vector_match(c["y"], y64), c["source"]


def test_golden_forward_large(golden):
    n = golden["matmul_fw_large"]["n"]
    i = np.arange(n, dtype=np.float64)
    a = np.tile(i / 16.0, n)                 # a[i + j n] = i/16
    b = np.repeat(i / 16.0, n)               # b[i + j n] = j/16
    y1 = np.outer(i, i).T.reshape(-1) * n / 256.0   # [i + j n] = n i j / 256
    y2 = np.full(n * n, np.sum(i * i) / 256.0)
    for threads in (1, 4):
        assert vector_match(y1, oracle.matmul_fw(a, b, n, n, n, 1, 1, threads))
        assert vector_match(y2, oracle.matmul_fw(b, a, n, n, n, 1, 1, threads))
    assert vector_match(y1, oracle.matmul_fw_f64(a, b, n, n, n, 1, 1))


def test_golden_backward(golden):
    for c in golden["matmul_bw"] + [golden["matmul_operator"]]:
        z = lambda k: np.zeros(len(c[k]), dtype=np.float32)
        ga, gb = oracle.matmul_bw(c["a"], c["b"], c["gy"], z("ga"), z("gb"),
                                  c["di"], c["dj"], c["dk"], c["ba"], c["bb"])
        assert vector_match(c["ga"], ga), c["source"]
        assert vector_match(c["gb"], gb), c["source"]
        ga, gb = oracle.matmul_bw_f64(c["a"], c["b"], c["gy"], z("ga"), z("gb"),
                                      c["di"], c["dj"], c["dk"], c["ba"], c["bb"])
        assert vector_match(c["ga"], ga), c["source"]
        assert vector_match(c["gb"], gb), c["source"]
    c = golden["matmul_operator"]
    assert vector_match(c["y"], oracle.matmul_fw(c["a"], c["b"], 2, 2, 2, 3, 3))


def test_golden_shapes(golden):
    for c in golden["shape_matmul_valid"]["cases"]:
        exp = (c["y"] + [1, 1])[:2]
        for ba, bb in ((1, 1), (3, 1), (1, 3), (3, 3)):
            got = oracle.shape_matmul(c["a"], ba, c["b"], bb)
            assert got == (exp[0], exp[1], max(ba, bb)), c
    for c in golden["shape_matmul_invalid"]["cases"]:
        assert oracle.shape_matmul(c["a"], c["ba"], c["b"], c["bb"]) is None, c


def test_golden_helpers(golden):
    for c in golden["inplace_add"]:
        y = oracle.inplace_add(c["x"], c["y_in"], c["volume"], c["bx"], c["by"])
        assert vector_match(c["y_out"], y), c["source"]
    for c in golden["batch_sum"]:
        assert vector_match(c["y"], oracle.batch_sum(c["x"], c["volume"], c["bs"]))
    p = golden["pool_block_size"]
    assert [oracle.pool_block_size(s, 1) for s in p["sizes"]] == p["expected_min1"]
    assert [oracle.pool_block_size(s, 10) for s in p["sizes"]] == p["expected_min10"]
    assert oracle.pool_block_size(26_000_000, 8) == 1 << 25


@pytest.mark.parametrize("di,dj,dk,ba,bb", CASES)
def test_against_float64_library(di, dj, dk, ba, bb):
    rng = np.random.default_rng(di * 1000 + dj * 10 + dk + ba + bb)
    bs = max(ba, bb)
    a, b, gy = _rand(rng, di * dj * ba), _rand(rng, dj * dk * bb), _rand(rng, di * dk * bs)
    ga0, gb0 = _rand(rng, a.size), _rand(rng, b.size)
    ref_y = np_matmul_fw(a, b, di, dj, dk, ba, bb)
    dga, dgb = np_matmul_bw(a, b, gy, di, dj, dk, ba, bb)
    for threads in (1, 3):
        y = oracle.matmul_fw(a, b, di, dj, dk, ba, bb, threads)
        assert norm_rel_err(y, ref_y) < 2e-6
        ga, gb = oracle.matmul_bw(a, b, gy, ga0, gb0, di, dj, dk, ba, bb, threads)
        assert norm_rel_err(ga, ga0 + dga) < 2e-6
        assert norm_rel_err(gb, gb0 + dgb) < 2e-6
    y = oracle.matmul_fw_f64(a, b, di, dj, dk, ba, bb)
    assert norm_rel_err(y, ref_y) < 1.5e-7
    ga, gb = oracle.matmul_bw_f64(a, b, gy, ga0, gb0, di, dj, dk, ba, bb)
    assert norm_rel_err(ga, ga0 + dga) < 1.5e-7
    assert norm_rel_err(gb, gb0 + dgb) < 1.5e-7


def test_blocked_routine_crosses_every_block_edge():
    # sizes that straddle the 192 x 384 x 3072 blocking and the 16 x 6 tile
    rng = np.random.default_rng(7)
    di, dj, dk = 197, 389, 3079
    a, b = _rand(rng, di * dj), _rand(rng, dj * dk)
    y = oracle.matmul_fw(a, b, di, dj, dk, 1, 1, 4)
    assert norm_rel_err(y, np_matmul_fw(a, b, di, dj, dk, 1, 1)) < 3e-6


def test_invariants():
    rng = np.random.default_rng(3)
    di, dj, dk, n = 12, 7, 9, 4
    a, b = _rand(rng, di * dj), _rand(rng, dj * dk * n)
    gy = _rand(rng, di * dk * n)
    # identity
    eye = np.eye(dj, dtype=np.float32).reshape(-1)
    assert np.array_equal(oracle.matmul_fw(eye, b, dj, dj, dk, 1, n), b)
    # a broadcast operand equals the same operand tiled over the minibatch
    at = np.tile(a, n)
    assert np.array_equal(oracle.matmul_fw(a, b, di, dj, dk, 1, n),
                          oracle.matmul_fw(at, b, di, dj, dk, n, n))
    z = lambda m: np.zeros(m, dtype=np.float32)
    ga1, gb1 = oracle.matmul_bw(a, b, gy, z(a.size), z(b.size), di, dj, dk, 1, n)
    gan, gbn = oracle.matmul_bw(at, b, gy, z(at.size), z(b.size), di, dj, dk, n, n)
    assert norm_rel_err(ga1, gan.reshape(n, -1).sum(0)) < 1e-6
    assert np.array_equal(gb1, gbn)
    # backward accumulates: calling it twice doubles the increment
    ga2, gb2 = oracle.matmul_bw(a, b, gy, ga1, gb1, di, dj, dk, 1, n)
    assert norm_rel_err(ga2, 2 * ga1) < 1e-6 and norm_rel_err(gb2, 2 * gb1) < 1e-6
    # N1: the shared b's gradient is the sum of the per-sample gradients
    an, b1 = _rand(rng, di * dj * n), _rand(rng, dj * dk)
    _, gbs = oracle.matmul_bw(an, b1, gy, z(an.size), z(b1.size), di, dj, dk, n, 1)
    _, gbn = oracle.matmul_bw(an, np.tile(b1, n), gy, z(an.size), z(b1.size * n), di, dj, dk, n, n)
    assert norm_rel_err(gbs, gbn.reshape(n, -1).sum(0)) < 1e-6
