"""The CPU oracle's data-movement and reduction operations against the
reference's golden tables and against numpy's own indexing routines."""
import numpy as np
import pytest

import oracle
from indexing_cases import CASES, run_case_on, case_id
from util import ulp_diff


class OracleBackend:
    pick_fw = staticmethod(oracle.pick_fw)
    slice_fw = staticmethod(oracle.slice_fw)
    transpose_fw = staticmethod(oracle.transpose_fw)
    reduce_fw = staticmethod(oracle.reduce_fw)
    broadcast_fw = staticmethod(oracle.broadcast_fw)
    arg_extremum = staticmethod(oracle.arg_extremum)

    @staticmethod
    def batch_pick_fw(x, dims, batch, ids):
        return oracle.batch_pick_fw(x, int(np.prod(dims)), ids)

    @staticmethod
    def pick_bw(gy, gx, dims, batch, ids, dim):
        return oracle.pick_bw(gy, gx, dims, batch, ids, dim)

    @staticmethod
    def extremum_bw(op, x, y, gy, gx, dims, batch, dim):
        return oracle.extremum_bw(x, y, gy, gx, dims, batch, dim)


@pytest.mark.parametrize("case", CASES, ids=case_id)
def test_oracle_matches_reference_tables(case):
    got = run_case_on(OracleBackend, case)
    want = np.asarray(case["expected"], dtype=got.dtype)
    assert got.shape == want.shape
    if got.dtype == np.float32 and case.get("ulps", 0):
        assert int(ulp_diff(got, want).max()) <= case["ulps"]
    else:
        assert np.array_equal(got, want)


def nd(x, dims, batch):
    """Flat primitiv array -> numpy array indexed [batch, d_{k-1}, ..., d_0] (dimension 0 fastest)."""
    return np.asarray(x).reshape([batch] + list(dims)[::-1])


def ax(dims, dim):
    """numpy axis of primitiv dimension `dim` in nd()'s layout."""
    return len(dims) - dim


SHAPES = [([5], 1), ([4, 3], 2), ([3, 4, 5], 3), ([2, 3, 2, 3], 2)]


@pytest.mark.parametrize("dims,batch", SHAPES)
def test_against_numpy_indexing(dims, batch):
    rng = np.random.default_rng(len(dims) * 10 + batch)
    n = int(np.prod(dims)) * batch
    x = rng.standard_normal(n).astype(np.float32)
    X = nd(x, dims, batch)
    for dim in range(len(dims)):
        a = ax(dims, dim)
        # slice / flip / reductions / argmax / pick
        lo, up = 1 if dims[dim] > 1 else 0, dims[dim]
        assert np.array_equal(oracle.slice_fw(x, dims, batch, dim, lo, up), np.take(X, range(lo, up), axis=a).reshape(-1))
        assert np.array_equal(oracle.flip_fw(x, dims, batch, dim), np.flip(X, axis=a).reshape(-1))
        assert np.allclose(oracle.reduce_fw("sum", x, dims, batch, dim), X.astype(np.float64).sum(axis=a).reshape(-1), atol=1e-5)
        assert np.array_equal(oracle.reduce_fw("max", x, dims, batch, dim), X.max(axis=a).reshape(-1))
        assert np.array_equal(oracle.reduce_fw("min", x, dims, batch, dim), X.min(axis=a).reshape(-1))
        lse = np.log(np.exp(X.astype(np.float64)).sum(axis=a)).reshape(-1)
        assert np.allclose(oracle.reduce_fw("logsumexp", x, dims, batch, dim), lse, rtol=1e-5, atol=1e-6)
        assert np.array_equal(oracle.arg_extremum("max", x, dims, batch, dim), X.argmax(axis=a).reshape(-1))
        assert np.array_equal(oracle.arg_extremum("min", x, dims, batch, dim), X.argmin(axis=a).reshape(-1))
        ids = [int(i) for i in rng.integers(0, dims[dim], batch)]
        picked = np.stack([np.take(X[b], [ids[b]], axis=a - 1) for b in range(batch)])
        assert np.array_equal(oracle.pick_fw(x, dims, batch, ids, dim), picked.reshape(-1))
        # gradients: scatter back what forward gathered
        gy = rng.standard_normal(picked.size).astype(np.float32)
        want = np.zeros_like(X)
        for b in range(batch):
            idx = [slice(None)] * X[b].ndim
            idx[a - 1] = slice(ids[b], ids[b] + 1)
            want[b][tuple(idx)] += gy.reshape(picked.shape)[b]
        assert np.allclose(oracle.pick_bw(gy, np.zeros(n, np.float32), dims, batch, ids, dim), want.reshape(-1))
        y = oracle.reduce_fw("max", x, dims, batch, dim)
        g = oracle.extremum_bw(x, y, np.ones_like(y), np.zeros(n, np.float32), dims, batch, dim)
        G = nd(g, dims, batch)
        assert np.array_equal(G.sum(axis=a).reshape(-1), np.ones_like(y))
        assert np.array_equal(np.take_along_axis(G, np.expand_dims(X.argmax(axis=a), a), axis=a).reshape(-1), np.ones_like(y))
    # concat with itself along every dimension, broadcast of a reduced tensor
    for dim in range(len(dims) + 1):
        y, ydims, yb = oracle.concat_fw([(x, dims, batch), (x, dims, batch)], dim)
        Xp = nd(x, list(dims) + [1] * (dim + 1 - len(dims)), batch)
        assert np.array_equal(y, np.concatenate([Xp, Xp], axis=Xp.ndim - 1 - dim).reshape(-1))
    for dim in range(len(dims)):
        s = oracle.reduce_fw("sum", x, dims, batch, dim)
        rd = list(dims)
        rd[dim] = 1
        bc = oracle.broadcast_fw(s, rd, batch, dim, dims[dim])
        assert np.array_equal(bc, np.repeat(nd(s, rd, batch), dims[dim], axis=ax(dims, dim)).reshape(-1))
    # permutation (y dimension i = x dimension perm[i]) and its gradient
    perm = list(rng.permutation(len(dims)))
    y = oracle.permute_dims_fw(x, dims, perm, batch)
    axes = [0] + [len(dims) - perm[len(dims) - 1 - k] for k in range(len(dims))]
    assert np.array_equal(y, X.transpose(axes).reshape(-1))
    assert np.array_equal(oracle.permute_dims_bw(y, np.zeros(n, np.float32), dims, perm, batch), x)


def test_matrix_and_batch_ops_against_numpy():
    rng = np.random.default_rng(3)
    d1, d2, bs = 5, 7, 3
    x = rng.standard_normal(d1 * d2 * bs).astype(np.float32)
    X = x.reshape(bs, d2, d1)
    y = oracle.transpose_fw(x, d1, d2, bs)
    assert np.array_equal(y, X.transpose(0, 2, 1).reshape(-1))
    assert np.array_equal(oracle.transpose_bw(y, np.zeros_like(x), d1, d2, bs), x)
    vol = d1 * d2
    assert np.array_equal(oracle.batch_slice_fw(x, vol, 1, 3), x[vol:3 * vol])
    g = oracle.batch_slice_bw(x[:2 * vol], np.ones_like(x), vol, 1)
    assert np.array_equal(g, np.concatenate([np.ones(vol, np.float32), 1 + x[:2 * vol]]))
    ids = [2, 0, 2, 1]
    assert np.array_equal(oracle.batch_pick_fw(x, vol, ids), np.concatenate([x[i * vol:(i + 1) * vol] for i in ids]))
    gy = rng.standard_normal(vol * 4).astype(np.float32)
    want = np.zeros_like(x)
    for b, i in enumerate(ids):
        want[i * vol:(i + 1) * vol] += gy[b * vol:(b + 1) * vol]
    assert np.allclose(oracle.batch_pick_bw(gy, np.zeros_like(x), vol, ids), want)
    # slice_bw with either side broadcast
    dims = [4, 3]
    gy1 = rng.standard_normal(2 * 3).astype(np.float32)           # rows 1..2 of a 4x3, batch 1
    g = oracle.slice_bw(gy1, 1, 2, np.zeros(12 * 2, np.float32), dims, 2, 0, 1)
    G = g.reshape(2, 3, 4)
    assert np.array_equal(G[:, :, 1:3], np.broadcast_to(gy1.reshape(1, 3, 2), (2, 3, 2)))
    gy2 = rng.standard_normal(2 * 3 * 2).astype(np.float32)       # batch 2 into batch 1: summed
    g = oracle.slice_bw(gy2, 2, 2, np.zeros(12, np.float32), dims, 1, 0, 1)
    assert np.allclose(g.reshape(3, 4)[:, 1:3], gy2.reshape(2, 3, 2).sum(axis=0))
