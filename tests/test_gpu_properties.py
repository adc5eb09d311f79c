"""Size-independent properties of the operations around the matmul at sizes
where the oracle would take minutes: round trips, sortedness-style bounds and
agreement with numpy's own (independent) reductions and scatter-adds.  These
sizes reach the launch shapes that small cases never do: reductions cut into
ranges with a second merging launch, 16-byte pack copies, long index lists."""
import numpy as np
import pytest

import primitiv_amd as pa

pytestmark = pytest.mark.gpu

S = pa.Shape


@pytest.fixture(scope="module")
def dev():
    d = pa.HIP(0, rng_seed=7)
    yield d
    d.close()


@pytest.fixture(scope="module")
def big(dev):
    rng = np.random.default_rng(1)
    x = rng.standard_normal(2048 * 2048 * 4).astype(np.float32)
    return x, dev.new_tensor_by_vector(S([2048, 2048], 4), x)


def test_transpose_twice_is_identity(dev, big):
    x, tx = big
    t = dev.transpose_fw(tx)
    assert t.shape() == S([2048, 2048], 4)
    assert np.array_equal(t.to_vector().reshape(4, 2048, 2048), x.reshape(4, 2048, 2048).transpose(0, 2, 1))
    assert np.array_equal(dev.transpose_fw(t).to_vector(), x)


@pytest.mark.parametrize("dim", [0, 1])
def test_slices_concatenate_back(dev, big, dim):
    x, tx = big
    cuts = [0, 512, 520, 1999, 2048]           # aligned and ragged pieces
    parts = [dev.slice_fw(tx, dim, lo, up) for lo, up in zip(cuts[:-1], cuts[1:])]
    assert np.array_equal(dev.concat_fw(parts, dim).to_vector(), x)
    # the gradient of a slice adds into exactly its region
    g = dev.new_tensor_by_constant(S([2048, 2048], 4), 1.0)
    dev.slice_bw(parts[2], dim, cuts[2], g)
    want = np.ones((4, 2048, 2048), np.float32)
    xs = x.reshape(4, 2048, 2048)
    if dim == 0:
        want[:, :, cuts[2]:cuts[3]] += xs[:, :, cuts[2]:cuts[3]]
    else:
        want[:, cuts[2]:cuts[3], :] += xs[:, cuts[2]:cuts[3], :]
    assert np.array_equal(g.to_vector(), want.reshape(-1))


def test_batch_slices_concatenate_back(dev, big):
    x, tx = big
    parts = [dev.batch_slice_fw(tx, lo, up) for lo, up in ((0, 1), (1, 3), (3, 4))]
    assert np.array_equal(dev.batch_concat_fw(parts).to_vector(), x)


@pytest.mark.parametrize("dim", [0, 1])
def test_reductions_agree_with_numpy(dev, big, dim):
    x, tx = big
    xs = x.reshape(4, 2048, 2048).astype(np.float64)     # [batch][dim1][dim0]
    axis = 2 - dim
    got = dev.reduce_fw("sum", tx, dim).to_vector()
    assert np.allclose(got, xs.sum(axis=axis).reshape(-1), rtol=1e-4, atol=1e-3)
    got = dev.reduce_fw("logsumexp", tx, dim).to_vector()
    assert np.allclose(got, np.log(np.exp(xs).sum(axis=axis)).reshape(-1), rtol=1e-5)
    for op, fn, arg in (("max", np.max, np.argmax), ("min", np.min, np.argmin)):
        assert np.array_equal(dev.reduce_fw(op, tx, dim).to_vector(), fn(xs, axis=axis).reshape(-1).astype(np.float32))
        assert np.array_equal(dev.arg_extremum(op, tx, dim), arg(xs, axis=axis).reshape(-1).astype(np.uint32))


@pytest.mark.parametrize("dims,dim", [([64, 200000], 1), ([3000000], 0), ([3, 1000000], 1), ([100000, 48], 0)])
def test_long_reductions_agree_with_numpy(dev, dims, dim):
    # few outputs over a long extent: the extent is cut into ranges whose partial
    # states a second launch merges; ties everywhere, so the first index must win
    rng = np.random.default_rng(dims[0])
    n = int(np.prod(dims))
    x = rng.integers(-50, 51, n).astype(np.float32)
    tx = dev.new_tensor_by_vector(S(dims), x)
    xs = x.reshape(dims[::-1])
    axis = len(dims) - 1 - dim
    assert np.array_equal(dev.reduce_fw("sum", tx, dim).to_vector(), xs.sum(axis=axis, dtype=np.float64).reshape(-1))
    assert np.array_equal(dev.reduce_fw("max", tx, dim).to_vector(), xs.max(axis=axis).reshape(-1))
    assert np.array_equal(dev.arg_extremum("max", tx, dim), np.argmax(xs, axis=axis).reshape(-1).astype(np.uint32))
    assert np.array_equal(dev.arg_extremum("min", tx, dim), np.argmin(xs, axis=axis).reshape(-1).astype(np.uint32))
    lse = dev.reduce_fw("logsumexp", tx, dim).to_vector()
    m = xs.max(axis=axis, keepdims=True).astype(np.float64)
    want = (m + np.log(np.exp(xs - m).sum(axis=axis, keepdims=True))).reshape(-1)
    assert np.allclose(lse, want, rtol=1e-6)


def test_embedding_gradient_is_a_scatter_add(dev):
    # 50 000-word table, 4000 lookups with many repeats: gx[:, id] += gy[:, b] in sample order
    rng = np.random.default_rng(3)
    width, vocab, bs = 128, 50000, 4000
    ids = rng.integers(0, 300, bs).tolist()                       # heavy repetition
    table = dev.new_tensor_by_constant(S([width, vocab]), 0)
    gy = rng.integers(-8, 9, width * bs).astype(np.float32)       # integers: sums are exact in any order
    dev.pick_bw(dev.new_tensor_by_vector(S([width], bs), gy), ids, 1, table)
    want = np.zeros((vocab, width), np.float32)
    np.add.at(want, np.asarray(ids), gy.reshape(bs, width))
    assert np.array_equal(table.to_vector(), want.reshape(-1))
    picked = dev.pick_fw(table, ids, 1).to_vector().reshape(bs, width)
    assert np.array_equal(picked, want[np.asarray(ids)])


def test_elementwise_identities(dev, big):
    x, tx = big
    # (x + k) - k, x * k / k, -(-x): exact or within one rounding
    y = dev.const_fw("subtract_const_r", dev.const_fw("add_const", tx, 3.0), 3.0)
    assert np.allclose(y.to_vector(), x, atol=5e-7)
    assert np.array_equal(dev.unary_fw("negate", dev.unary_fw("negate", tx)).to_vector(), x)
    # tanh' from the kernel against the closed form on its own output
    t = dev.unary_fw("tanh", tx)
    g = dev.new_tensor_by_constant(tx.shape(), 0)
    dev.unary_bw("tanh", tx, t, dev.new_tensor_by_constant(tx.shape(), 1.0), g)
    tv = t.to_vector().astype(np.float64)
    assert np.allclose(g.to_vector(), 1.0 - tv * tv, atol=1e-6)
    # a broadcast sum equals the tiled sum
    bias = dev.new_tensor_by_vector(S([2048, 2048]), x[:2048 * 2048])
    z = dev.binary_fw("add", tx, bias).to_vector().reshape(4, -1)
    assert np.array_equal(z, x.reshape(4, -1) + x[:2048 * 2048][None, :])


def test_random_tensors_at_scale(dev):
    n = 1 << 25
    u = dev.random_uniform(S([n]), -2.0, 5.0).to_vector()
    assert u.min() > -2.0 and u.max() <= 5.0
    assert abs(u.mean() - 1.5) < 2e-3 and abs(u.var() - 49.0 / 12.0) < 1e-2
    z = dev.random_normal(S([n]), 1.0, 3.0).to_vector()
    assert abs(z.mean() - 1.0) < 3e-3 and abs(z.std() - 3.0) < 3e-3
    assert abs(np.mean(np.abs(z - 1.0) > 6.0) - 0.0455) < 1e-3          # two-sigma tail mass
    b = dev.random_bernoulli(S([n]), 0.3).to_vector()
    assert set(np.unique(b)) == {0.0, 1.0} and abs(b.mean() - 0.3) < 1e-3
