"""Data-movement and reduction operations of the HIP devices (through the C
ABI) against the reference's golden tables and the CPU oracle."""
import numpy as np
import pytest

import oracle
import primitiv_amd as pa
from indexing_cases import CASES, run_case_on, case_id
from util import ulp_diff, round_to_storage

pytestmark = pytest.mark.gpu

S = pa.Shape


class DeviceBackend:
    """Golden-case backend over a device: flat arrays in, flat arrays out."""

    def __init__(self, dev):
        self.dev = dev

    def t(self, x, dims, batch):
        return self.dev.new_tensor_by_vector(S(dims, batch), np.asarray(x, dtype=np.float32))

    def pick_fw(self, x, dims, batch, ids, dim):
        return self.dev.pick_fw(self.t(x, dims, batch), ids, dim).to_vector()

    def slice_fw(self, x, dims, batch, dim, lower, upper):
        return self.dev.slice_fw(self.t(x, dims, batch), dim, lower, upper).to_vector()

    def transpose_fw(self, x, d1, d2, batch):
        return self.dev.transpose_fw(self.t(x, [d1, d2], batch)).to_vector()

    def reduce_fw(self, op, x, dims, batch, dim):
        return self.dev.reduce_fw(op, self.t(x, dims, batch), dim).to_vector()

    def broadcast_fw(self, x, dims, batch, dim, size):
        return self.dev.broadcast_fw(self.t(x, dims, batch), dim, size).to_vector()

    def batch_pick_fw(self, x, dims, batch, ids):
        return self.dev.batch_pick_fw(self.t(x, dims, batch), ids).to_vector()

    def arg_extremum(self, op, x, dims, batch, dim):
        return np.asarray(self.dev.arg_extremum(op, self.t(x, dims, batch), dim), dtype=np.uint32)

    def pick_bw(self, gy, gx, dims, batch, ids, dim):
        g = self.t(gx, dims, batch)
        sy = pa.shape_ops.pick(g.shape(), ids, dim)
        self.dev.pick_bw(self.dev.new_tensor_by_vector(sy, gy), ids, dim, g)
        return g.to_vector()

    def extremum_bw(self, op, x, y, gy, gx, dims, batch, dim):
        tx, g = self.t(x, dims, batch), self.t(gx, dims, batch)
        sy = tx.shape().resize_dim(dim, 1)
        self.dev.extremum_bw(op, tx, self.dev.new_tensor_by_vector(sy, y), self.dev.new_tensor_by_vector(sy, gy),
                             dim, g)
        return g.to_vector()


@pytest.fixture(scope="module")
def dev():
    return pa.HIP(0)


@pytest.fixture(scope="module", params=["f16", "bf16"])
def dev16(request):
    return pa.HIP16(0, storage=request.param)


def _check_case(dev, case, exact_only):
    got = run_case_on(DeviceBackend(dev), case)
    want = np.asarray(case["expected"], dtype=got.dtype)
    assert got.shape == want.shape
    if got.dtype == np.float32 and case.get("ulps", 0):
        if exact_only:
            assert np.allclose(got, want, rtol=2e-2)
        else:
            assert int(ulp_diff(got, want).max()) <= case["ulps"]
    else:
        assert np.array_equal(got, want)


@pytest.mark.parametrize("case", CASES, ids=case_id)
def test_f32_matches_reference_tables(dev, case):
    _check_case(dev, case, False)


@pytest.mark.parametrize("case", CASES, ids=case_id)
def test_half_storage_matches_reference_tables(dev16, case):
    # the tables hold small integers, which both 16-bit types keep exactly, except
    # the long sums of ones (the reference skips those for its half device too)
    limit = 2048 if dev16._SUFFIX == "f16" else 256
    if "x_constant" in case and case["dims"][0] > limit:
        # the count exceeds what the 16-bit type represents exactly: the device sums in fp32 and rounds once,
        # so the result is the count rounded to nearest even in the storage type (65535 and up overflow in fp16)
        got = run_case_on(DeviceBackend(dev16), case)
        want = round_to_storage(case["expected"], dev16._SUFFIX)
        assert np.array_equal(got, want), (got, want)
        return
    _check_case(dev16, case, True)


SHAPES = [([7], 1), ([5, 3], 4), ([33, 65], 2), ([3, 4, 5], 3), ([2, 3, 2, 3], 2), ([300, 70], 5), ([1000], 64)]


@pytest.mark.parametrize("dims,batch", SHAPES)
def test_dimension_ops_match_oracle(dev, dims, batch):
    rng = np.random.default_rng(len(dims) * 100 + batch)
    n = int(np.prod(dims)) * batch
    x = rng.standard_normal(n).astype(np.float32)
    tx = dev.new_tensor_by_vector(S(dims, batch), x)
    for dim in range(len(dims)):
        lo, up = (1, dims[dim]) if dims[dim] > 1 else (0, 1)
        y = dev.slice_fw(tx, dim, lo, up)
        assert np.array_equal(y.to_vector(), oracle.slice_fw(x, dims, batch, dim, lo, up))
        # gradient of the slice, into gx of the same batch, of batch 1, and from gy of batch 1
        gyv = rng.standard_normal(y.shape().size()).astype(np.float32)
        g0 = rng.standard_normal(n).astype(np.float32)
        gx = dev.new_tensor_by_vector(S(dims, batch), g0)
        dev.slice_bw(dev.new_tensor_by_vector(y.shape(), gyv), dim, lo, gx)
        assert np.allclose(gx.to_vector(), oracle.slice_bw(gyv, batch, up - lo, g0, dims, batch, dim, lo), atol=1e-6)
        if batch > 1:
            g1 = g0[:n // batch].copy()
            gx1 = dev.new_tensor_by_vector(S(dims), g1)
            dev.slice_bw(dev.new_tensor_by_vector(y.shape(), gyv), dim, lo, gx1)
            assert np.allclose(gx1.to_vector(), oracle.slice_bw(gyv, batch, up - lo, g1, dims, 1, dim, lo),
                               rtol=1e-5, atol=1e-5)
            gy1 = gyv[:gyv.size // batch]
            gx = dev.new_tensor_by_vector(S(dims, batch), g0)
            dev.slice_bw(dev.new_tensor_by_vector(y.shape().resize_batch(1), gy1), dim, lo, gx)
            assert np.allclose(gx.to_vector(), oracle.slice_bw(gy1, 1, up - lo, g0, dims, batch, dim, lo), atol=1e-6)
        assert np.array_equal(dev.flip_fw(tx, dim).to_vector(), oracle.flip_fw(x, dims, batch, dim))
        gx = dev.new_tensor_by_vector(S(dims, batch), g0)
        dev.flip_bw(tx, dim, gx)
        assert np.allclose(gx.to_vector(), oracle.flip_bw(x, g0, dims, batch, dim), atol=1e-6)
        for op in pa.HIP.REDUCE_OPS:
            got = dev.reduce_fw(op, tx, dim).to_vector()
            want = oracle.reduce_fw(op, x, dims, batch, dim)
            if op in ("max", "min"):
                assert np.array_equal(got, want)
            else:
                assert np.allclose(got, want, rtol=1e-5, atol=1e-4)
        for op in ("max", "min"):
            assert np.array_equal(dev.arg_extremum(op, tx, dim), oracle.arg_extremum(op, x, dims, batch, dim))
            yv = oracle.reduce_fw(op, x, dims, batch, dim)
            gyv = rng.standard_normal(yv.size).astype(np.float32)
            sy = tx.shape().resize_dim(dim, 1)
            gx = dev.new_tensor_by_vector(S(dims, batch), g0)
            dev.extremum_bw(op, tx, dev.new_tensor_by_vector(sy, yv), dev.new_tensor_by_vector(sy, gyv), dim, gx)
            assert np.allclose(gx.to_vector(), oracle.extremum_bw(x, yv, gyv, g0, dims, batch, dim), atol=1e-6)
        # pick with one index per sample, with a shared index, and from a tensor of batch 1
        for ids in ([int(i) for i in rng.integers(0, dims[dim], batch)], [int(rng.integers(0, dims[dim]))]):
            got = dev.pick_fw(tx, ids, dim)
            assert np.array_equal(got.to_vector(), oracle.pick_fw(x, dims, batch, ids, dim))
            gyv = rng.standard_normal(got.shape().size()).astype(np.float32)
            gx = dev.new_tensor_by_vector(S(dims, batch), g0)
            dev.pick_bw(dev.new_tensor_by_vector(got.shape(), gyv), ids, dim, gx)
            assert np.allclose(gx.to_vector(), oracle.pick_bw(gyv, g0, dims, batch, ids, dim), atol=1e-6)
        ids = [int(i) for i in rng.integers(0, dims[dim], 6)]   # repeated indices into a tensor of batch 1
        x1, t1 = x[:n // batch], dev.new_tensor_by_vector(S(dims), x[:n // batch])
        got = dev.pick_fw(t1, ids, dim)
        assert np.array_equal(got.to_vector(), oracle.pick_fw(x1, dims, 1, ids, dim))
        gyv = rng.standard_normal(got.shape().size()).astype(np.float32)
        gx = dev.new_tensor_by_vector(S(dims), g0[:n // batch])
        dev.pick_bw(dev.new_tensor_by_vector(got.shape(), gyv), ids, dim, gx)
        assert np.allclose(gx.to_vector(), oracle.pick_bw(gyv, g0[:n // batch], dims, 1, ids, dim), rtol=1e-5, atol=1e-5)
        # broadcast of the reduced tensor back along dim
        rd = list(dims)
        rd[dim] = 1
        s = oracle.reduce_fw("sum", x, dims, batch, dim)
        got = dev.broadcast_fw(dev.new_tensor_by_vector(S(rd, batch), s), dim, dims[dim])
        assert got.shape() == S(dims, batch)
        assert np.array_equal(got.to_vector(), oracle.broadcast_fw(s, rd, batch, dim, dims[dim]))
    for dim in range(len(dims) + 1):
        other = dev.new_tensor_by_vector(S(dims), x[:n // batch])   # batch 1 joins batch N
        got = dev.concat_fw([tx, other, tx], dim)
        want, wd, wb = oracle.concat_fw([(x, dims, batch), (x[:n // batch], dims, 1), (x, dims, batch)], dim)
        assert got.shape() == S(wd, wb)
        assert np.array_equal(got.to_vector(), want)
    perm = [int(p) for p in rng.permutation(len(dims))]
    y = dev.permute_dims_fw(tx, perm)
    assert np.array_equal(y.to_vector(), oracle.permute_dims_fw(x, dims, perm, batch))
    g0 = rng.standard_normal(n).astype(np.float32)
    gx = dev.new_tensor_by_vector(S(dims, batch), g0)
    dev.permute_dims_bw(tx, y, y, perm, gx)
    assert np.allclose(gx.to_vector(), oracle.permute_dims_bw(y.to_vector(), g0, dims, perm, batch), atol=1e-6)


# One shape per launch shape of the reduction (wavefront per contiguous run, lanes
# along base with n split, workgroup per output, thread per output), ragged sizes.
REDUCE_SHAPES = [([100, 300], 2, 0), ([33, 1031], 1, 0), ([70, 100], 3, 1), ([129, 517], 2, 1), ([20, 50], 40, 1),
                 ([17, 1000, 3], 1, 1), ([5000], 3, 0), ([20011], 2, 0), ([3, 9000], 2, 1), ([40, 20], 30, 0), ([4, 64, 2], 5, 1),
                 # a contiguous run taken 16 bytes per lane (length a multiple of 4, at least 256, many outputs)
                 ([256, 520], 1, 0), ([260, 300], 2, 0), ([1028, 530], 1, 0),
                 # two columns per lane (even stride of at least 128 below the reduced dimension)
                 ([128, 517], 2, 1), ([130, 300], 2, 1), ([386, 40, 3], 1, 1)]


@pytest.mark.parametrize("dims,batch,dim", REDUCE_SHAPES)
def test_reduction_launch_shapes_match_oracle(dev, dims, batch, dim):
    rng = np.random.default_rng(dims[0] * 7 + batch)
    n = int(np.prod(dims)) * batch
    # few distinct values: ties everywhere, so the first-occurrence rule is exercised
    for x in (rng.standard_normal(n).astype(np.float32), rng.integers(-3, 4, n).astype(np.float32)):
        tx = dev.new_tensor_by_vector(S(dims, batch), x)
        for op in pa.HIP.REDUCE_OPS:
            got = dev.reduce_fw(op, tx, dim).to_vector()
            want = oracle.reduce_fw(op, x, dims, batch, dim)
            if op in ("max", "min"):
                assert np.array_equal(got, want)
            else:
                assert np.allclose(got, want, rtol=1e-5, atol=2e-4)
        for op in ("max", "min"):
            assert np.array_equal(dev.arg_extremum(op, tx, dim), oracle.arg_extremum(op, x, dims, batch, dim))
            yv = oracle.reduce_fw(op, x, dims, batch, dim)
            gyv = rng.standard_normal(yv.size).astype(np.float32)
            g0 = rng.standard_normal(n).astype(np.float32)
            sy = tx.shape().resize_dim(dim, 1)
            gx = dev.new_tensor_by_vector(S(dims, batch), g0)
            dev.extremum_bw(op, tx, dev.new_tensor_by_vector(sy, yv), dev.new_tensor_by_vector(sy, gyv), dim, gx)
            assert np.allclose(gx.to_vector(), oracle.extremum_bw(x, yv, gyv, g0, dims, batch, dim), atol=1e-6)


@pytest.mark.parametrize("d1,d2,bs", [(1, 1, 1), (5, 7, 3), (64, 32, 2), (100, 257, 4), (1000, 33, 1), (130, 258, 2), (256, 66, 3),
                                      (2, 2, 1), (2, 1000, 2)])
def test_transpose_and_batch_ops_match_oracle(dev, d1, d2, bs):
    rng = np.random.default_rng(d1 + d2)
    x = rng.standard_normal(d1 * d2 * bs).astype(np.float32)
    tx = dev.new_tensor_by_vector(S([d1, d2], bs), x)
    y = dev.transpose_fw(tx)
    assert y.shape() == S([d2, d1], bs)
    assert np.array_equal(y.to_vector(), oracle.transpose_fw(x, d1, d2, bs))
    g0 = rng.standard_normal(x.size).astype(np.float32)
    gx = dev.new_tensor_by_vector(S([d1, d2], bs), g0)
    dev.transpose_bw(tx, y, y, gx)
    assert np.allclose(gx.to_vector(), oracle.transpose_bw(y.to_vector(), g0, d1, d2, bs), atol=1e-6)
    vol = d1 * d2
    if bs > 1:
        part = dev.batch_slice_fw(tx, 1, bs)
        assert np.array_equal(part.to_vector(), oracle.batch_slice_fw(x, vol, 1, bs))
        gx = dev.new_tensor_by_vector(S([d1, d2], bs), g0)
        dev.batch_slice_bw(part, 1, gx)
        assert np.allclose(gx.to_vector(), oracle.batch_slice_bw(part.to_vector(), g0, vol, 1), atol=1e-6)
    ids = [int(i) for i in rng.integers(0, bs, 5)]
    picked = dev.batch_pick_fw(tx, ids)
    assert np.array_equal(picked.to_vector(), oracle.batch_pick_fw(x, vol, ids))
    gx = dev.new_tensor_by_vector(S([d1, d2], bs), g0)
    dev.batch_pick_bw(picked, ids, gx)
    assert np.allclose(gx.to_vector(), oracle.batch_pick_bw(picked.to_vector(), g0, vol, ids), rtol=1e-5, atol=1e-5)
    joined = dev.batch_concat_fw([tx, picked, tx])
    assert joined.shape() == S([d1, d2], 2 * bs + 5)
    assert np.array_equal(joined.to_vector(), oracle.batch_concat_fw([x, picked.to_vector(), x]))


@pytest.mark.parametrize("bs", [700, 1500])
def test_long_index_lists_go_through_device_memory(dev, bs):
    # more indices than travel in the kernel arguments (700), and more than get a
    # workgroup row each in the gradient (1500); many samples share an index
    rng = np.random.default_rng(5)
    vocab, width = 500, 48
    table = rng.standard_normal(width * vocab).astype(np.float32)
    ids = [int(i) for i in rng.integers(0, vocab, bs)]
    t = dev.new_tensor_by_vector(S([width, vocab]), table)
    got = dev.pick_fw(t, ids, 1)
    assert got.shape() == S([width], bs)
    assert np.array_equal(got.to_vector(), oracle.pick_fw(table, [width, vocab], 1, ids, 1))
    g = dev.new_tensor_by_constant(S([width, vocab]), 0)
    dev.pick_bw(got, ids, 1, g)
    # fp32, samples added in order: the same sums as the sequential restatement
    assert np.array_equal(g.to_vector(), oracle.pick_bw(got.to_vector(), np.zeros_like(table), [width, vocab], 1, ids, 1))
    # the same lists through batch_pick: a table of `vocab` samples
    tb = dev.new_tensor_by_vector(S([width], vocab), table)
    gotb = dev.batch_pick_fw(tb, ids)
    assert np.array_equal(gotb.to_vector(), got.to_vector())
    gb = dev.new_tensor_by_constant(S([width], vocab), 0)
    dev.batch_pick_bw(gotb, ids, gb)
    assert np.array_equal(gb.to_vector(), g.to_vector())


def test_softmax_cross_entropy_pieces(dev):
    # logsumexp + broadcast + pick, the way primitiv builds softmax cross entropy
    # (primitiv/core/tensor_funcs.cc:310-329), at a vocabulary-sized dimension
    rng = np.random.default_rng(9)
    vocab, bs = 10000, 64
    x = rng.standard_normal(vocab * bs).astype(np.float32) * 3
    tx = dev.new_tensor_by_vector(S([vocab], bs), x)
    lse = dev.reduce_fw("logsumexp", tx, 0)
    want = np.log(np.exp(x.reshape(bs, vocab).astype(np.float64)).sum(axis=1))
    assert np.allclose(lse.to_vector(), want, rtol=1e-6)
    log_softmax = dev.binary_fw("subtract", tx, dev.broadcast_fw(lse, 0, vocab))
    ids = [int(i) for i in rng.integers(0, vocab, bs)]
    picked = dev.pick_fw(log_softmax, ids, 0).to_vector()
    assert np.allclose(picked, x.reshape(bs, vocab)[np.arange(bs), ids] - want, rtol=1e-5, atol=1e-5)


def test_errors(dev):
    x = dev.new_tensor_by_constant(S([2, 2, 2], 3), 0)
    for ids, dim in (([], 0), ([2], 0), ([0, 1], 0), ([2], 1), ([1], 3)):
        with pytest.raises(pa.Error):
            dev.pick_fw(x, ids, dim)          # test/tensor_forward_test.cc:171-191
    with pytest.raises(pa.Error):
        dev.slice_fw(x, 0, 1, 1)
    with pytest.raises(pa.Error):
        dev.slice_fw(x, 0, 0, 3)
    with pytest.raises(pa.Error):
        dev.transpose_fw(x)
    with pytest.raises(pa.Error):
        dev.permute_dims_fw(x, [0, 0, 1])
    with pytest.raises(pa.Error):
        dev.batch_pick_fw(x, [3])
    with pytest.raises(pa.Error):
        dev.broadcast_fw(x, 0, 2)
    with pytest.raises(pa.Error):
        dev.concat_fw([x, dev.new_tensor_by_constant(S([3, 2, 2], 3), 0)], 1)


def test_half_storage_matches_oracle(dev16):
    rng = np.random.default_rng(11)
    dims, batch = [40, 30], 3
    n = 40 * 30 * batch
    x = rng.standard_normal(n).astype(np.float32)
    tx = dev16.new_tensor_by_vector(S(dims, batch), x)
    xr = tx.to_vector()                       # what the device holds after rounding
    for dim in (0, 1):
        assert np.array_equal(dev16.slice_fw(tx, dim, 2, 9).to_vector(), oracle.slice_fw(xr, dims, batch, dim, 2, 9))
        assert np.array_equal(dev16.flip_fw(tx, dim).to_vector(), oracle.flip_fw(xr, dims, batch, dim))
        assert np.array_equal(dev16.reduce_fw("max", tx, dim).to_vector(), oracle.reduce_fw("max", xr, dims, batch, dim))
        assert np.array_equal(dev16.arg_extremum("min", tx, dim), oracle.arg_extremum("min", xr, dims, batch, dim))
        for op in ("sum", "logsumexp"):
            want = oracle.reduce_fw(op, xr, dims, batch, dim)
            assert np.max(np.abs(dev16.reduce_fw(op, tx, dim).to_vector() - want)) <= 2e-2 * np.max(np.abs(want))
        ids = [3, 0, 7]
        assert np.array_equal(dev16.pick_fw(tx, ids, dim).to_vector(), oracle.pick_fw(xr, dims, batch, ids, dim))
    assert np.array_equal(dev16.transpose_fw(tx).to_vector(), oracle.transpose_fw(xr, 40, 30, batch))
    assert np.array_equal(dev16.permute_dims_fw(tx, [1, 0]).to_vector(), oracle.permute_dims_fw(xr, dims, [1, 0], batch))
    assert np.array_equal(dev16.batch_pick_fw(tx, [2, 2, 0]).to_vector(), oracle.batch_pick_fw(xr, 1200, [2, 2, 0]))


@pytest.mark.parametrize("d1,d2,bs", [(2, 2, 1), (40, 30, 3), (130, 258, 2), (128, 128, 1), (256, 66, 3), (41, 30, 2),
                                      (40, 31, 2), (1, 64, 1)])
def test_half_storage_transpose(dev16, d1, d2, bs):
    # even extents move as 2 x 2 blocks of elements (tiles of 128 x 128 elements of 16-bit storage), odd ones one element per lane
    rng = np.random.default_rng(d1 * 1000 + d2)
    x = rng.standard_normal(d1 * d2 * bs).astype(np.float32)
    tx = dev16.new_tensor_by_vector(S([d1, d2], bs), x)
    xr = tx.to_vector()
    y = dev16.transpose_fw(tx)
    assert y.shape() == S([d2, d1], bs)
    assert np.array_equal(y.to_vector(), oracle.transpose_fw(xr, d1, d2, bs))
    g0 = round_to_storage(rng.standard_normal(x.size).astype(np.float32), dev16._SUFFIX)
    gx = dev16.new_tensor_by_vector(S([d1, d2], bs), g0)
    dev16.transpose_bw(tx, y, y, gx)                    # gx += transpose(gy), rounded once per element
    want = round_to_storage(oracle.transpose_bw(y.to_vector(), g0, d1, d2, bs), dev16._SUFFIX)
    assert np.array_equal(gx.to_vector(), want)


def _aligned_copies(dev, exact_sum):
    # extents and offsets that are multiples of 16 bytes in every storage type: the
    # copies then move whole 16-byte packs
    rng = np.random.default_rng(21)
    dims, batch = [64, 48], 3
    n = 64 * 48 * batch
    tx = dev.new_tensor_by_vector(S(dims, batch), rng.standard_normal(n).astype(np.float32))
    xr = tx.to_vector()
    for dim, lo, up in ((0, 16, 56), (1, 8, 40), (0, 0, 64)):
        y = dev.slice_fw(tx, dim, lo, up)
        assert np.array_equal(y.to_vector(), oracle.slice_fw(xr, dims, batch, dim, lo, up))
        g0 = dev.new_tensor_by_vector(S(dims, batch), rng.standard_normal(n).astype(np.float32))
        g0v, yv = g0.to_vector(), y.to_vector()
        dev.slice_bw(y, dim, lo, g0)
        want = oracle.slice_bw(yv, batch, up - lo, g0v, dims, batch, dim, lo)
        if exact_sum:
            assert np.array_equal(g0.to_vector(), want)
        else:
            assert np.max(np.abs(g0.to_vector() - want)) <= 2e-2 * np.max(np.abs(want))
    for dim in (0, 1, 2):
        got = dev.concat_fw([tx, tx], dim)
        want, wd, wb = oracle.concat_fw([(xr, dims, batch), (xr, dims, batch)], dim)
        assert got.shape() == S(wd, wb)
        assert np.array_equal(got.to_vector(), want)
    assert np.array_equal(dev.batch_slice_fw(tx, 1, 3).to_vector(), xr[64 * 48:])


def test_aligned_copies_match_oracle(dev):
    _aligned_copies(dev, True)


def test_half_storage_aligned_copies_match_oracle(dev16):
    _aligned_copies(dev16, False)


@pytest.mark.parametrize("dims,batch,dim", [([256, 4096], 1, 1), ([20000], 3, 0), ([130, 3000], 2, 1), ([16, 70000], 1, 1)])
def test_long_reductions_cut_into_ranges_are_reproducible(dev, dims, batch, dim):
    # few outputs over a long dimension: the dimension is cut into ranges reduced by different workgroups, and the
    # one that finishes last merges them in order - the same bits whichever that is
    rng = np.random.default_rng(dims[0] + batch)
    n = int(np.prod(dims)) * batch
    x = rng.standard_normal(n).astype(np.float32)
    tx = dev.new_tensor_by_vector(S(dims, batch), x)
    for op in ("sum", "logsumexp", "max"):
        first = dev.reduce_fw(op, tx, dim).to_vector()
        want = oracle.reduce_fw(op, x, dims, batch, dim)
        if op == "max":
            assert np.array_equal(first, want)
        elif op == "logsumexp":
            assert np.allclose(first, want, rtol=1e-5, atol=1e-4)
        else:
            # against the sum in float64; an fp32 sum of n values of unit variance, in whatever order, is good to
            # a few times 1e-7 n at the very worst
            exact = np.moveaxis(x.astype(np.float64).reshape([batch] + dims[::-1]), len(dims) - dim, -1).sum(-1).reshape(-1)
            assert np.max(np.abs(first - exact)) <= 3e-7 * dims[dim]
        for _ in range(10):
            assert np.array_equal(dev.reduce_fw(op, tx, dim).to_vector(), first)
    idx = oracle.arg_extremum("max", x, dims, batch, dim)
    for _ in range(5):
        assert np.array_equal(dev.arg_extremum("max", tx, dim), idx)


@pytest.mark.parametrize("dims,batch,dim", [([130, 517], 2, 1), ([256, 40, 3], 1, 1), ([129, 300], 1, 1), ([64, 1031], 3, 0),
                                            ([260, 300], 2, 1), ([516, 70, 2], 1, 1), ([512, 520], 1, 0), ([520, 300], 2, 0),
                                            ([1032, 515], 1, 0)])
def test_half_storage_reduction_launch_shapes(dev16, dims, batch, dim):
    # 16-bit storage reduces four columns per lane when the stride below the reduced
    # dimension is a multiple of 4 and at least 256, two when it is even and at least
    # 128; odd and short strides take one. A leading-dimension reduction walks each
    # run 8 elements per lane when its length is a multiple of 8 and at least 512.
    rng = np.random.default_rng(dims[0] + batch)
    n = int(np.prod(dims)) * batch
    for x in (rng.standard_normal(n).astype(np.float32), rng.integers(-3, 4, n).astype(np.float32)):
        tx = dev16.new_tensor_by_vector(S(dims, batch), x)
        xr = tx.to_vector()
        for op in ("max", "min"):
            assert np.array_equal(dev16.reduce_fw(op, tx, dim).to_vector(), oracle.reduce_fw(op, xr, dims, batch, dim))
            assert np.array_equal(dev16.arg_extremum(op, tx, dim), oracle.arg_extremum(op, xr, dims, batch, dim))
        for op in ("sum", "logsumexp"):
            want = oracle.reduce_fw(op, xr, dims, batch, dim)
            got = dev16.reduce_fw(op, tx, dim).to_vector()
            assert np.max(np.abs(got - want)) <= 2e-2 * np.max(np.abs(want))
