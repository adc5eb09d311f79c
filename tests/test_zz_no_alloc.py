"""phip_matmul_fw_f32_noalloc against phip_matmul_fw_f32, through the C ABI.

The allocation-free entry point runs the same kernels with the partial tiles and
tile counters of a split product in the library's fixed device array, so its
result must equal the allocating entry point's bit for bit (the fp32 gate of the
matmul tests, max|x - ref| / max|ref| <= 1e-4, is checked as well, against the
CPU oracle).  Calls follow one another on one context, the later ones smaller
than the first, so what an earlier call left in the array is there when the
next one runs.
"""
import ctypes

import numpy as np
import pytest

import oracle
import primitiv_amd as pa
from primitiv_amd import _lib
from util import norm_rel_err

pytestmark = pytest.mark.gpu

F32_TOL = 1e-4

# (di, dj, dk, ba, bb): products whose K range is cut between workgroups (partial
# tiles + tile counters in scratch), the output projection's forward product (a
# launch that mixes whole tiles with tiles cut in K ranges: partial tiles of the
# latter in scratch) and an unsplit one.
SEQUENCE = [
    (2048, 512, 1, 1, 64),     # recurrent gate forward
    (256, 784, 1, 1, 128),     # dense forward: smaller, right after the larger one
    (96, 1000, 5, 1, 3),       # ragged, split
    (10000, 650, 1, 1, 64),    # streamed operand: whole tiles beside split ones
    (1024, 4096, 512, 1, 1),   # mid-size, long K: large tiles, K cut in 8: exactly 16 MiB of partial tiles
    (768, 4096, 96, 1, 1),     # few tiles, long K
    (200, 3000, 40, 2, 2),     # per-sample products, split
    (64, 64, 64, 1, 1),        # unsplit, no scratch at all
]


def _pool_stats(dev):
    s, r = ctypes.c_uint64(0), ctypes.c_uint64(0)
    _lib.call("phip_pool_stats", dev.ctx(), ctypes.byref(s), ctypes.byref(r))
    return s.value, r.value


def _both(dev, rng, di, dj, dk, ba, bb):
    bs = max(ba, bb)
    a = rng.standard_normal(di * dj * ba).astype(np.float32)
    b = rng.standard_normal(dj * dk * bb).astype(np.float32)
    ta = dev.new_tensor_by_vector(pa.Shape([di, dj], ba), a)
    tb = dev.new_tensor_by_vector(pa.Shape([dj, dk], bb), b)
    y_ref = dev.matmul_fw(ta, tb)                       # allocating entry point
    y_new = dev.new_tensor_by_constant(pa.Shape([di, dk], bs), float("nan"))
    before = _pool_stats(dev)
    _lib.call("phip_matmul_fw_f32_noalloc", dev.ctx(), ta.handle(), tb.handle(), y_new.mutable_handle(),
              di, dj, dk, ba, bb)
    assert _pool_stats(dev) == before, "the allocation-free call touched the pool"
    return a, b, y_ref.to_vector(), y_new.to_vector()


def test_noalloc_forward_matches_allocating_entry_point():
    dev = pa.HIP(0)
    rng = np.random.default_rng(7)
    for case in SEQUENCE:
        print("noalloc case", case, flush=True)
        di, dj, dk, ba, bb = case
        a, b, y_ref, y_new = _both(dev, rng, *case)
        assert np.array_equal(y_ref, y_new), case
        want = oracle.matmul_fw(a, b, di, dj, dk, ba, bb)
        assert norm_rel_err(y_new, want) <= F32_TOL, case
    dev.close()


def test_noalloc_two_calls_second_smaller_fresh_context():
    # the pair the entry point is specified by: two calls in a row, the second smaller
    dev = pa.HIP(0)
    rng = np.random.default_rng(11)
    for case in [(2048, 512, 1, 1, 64), (300, 520, 1, 1, 33)]:
        print("noalloc pair", case, flush=True)
        di, dj, dk, ba, bb = case
        a, b, y_ref, y_new = _both(dev, rng, *case)
        assert np.array_equal(y_ref, y_new), case
        assert norm_rel_err(y_new, oracle.matmul_fw(a, b, di, dj, dk, ba, bb)) <= F32_TOL, case
    dev.close()


def test_noalloc_rejects_what_does_not_fit():
    # 1024 x 1024 with K = 4096 is cut into 8 ranges: 32 MiB of partial tiles, the array holds 16
    dev = pa.HIP(0)
    di, dj, dk = 1024, 4096, 1024
    ta = dev.new_tensor_by_constant(pa.Shape([di, dj]), 1.0)
    tb = dev.new_tensor_by_constant(pa.Shape([dj, dk]), 1.0)
    y = dev.new_tensor_by_constant(pa.Shape([di, dk]), -3.0)
    with pytest.raises(pa.Error) as e:
        _lib.call("phip_matmul_fw_f32_noalloc", dev.ctx(), ta.handle(), tb.handle(), y.mutable_handle(),
                  di, dj, dk, 1, 1)
    assert e.value.code == _lib.PHIP_ERR_INVALID_ARGUMENT and "scratch" in str(e.value)
    assert np.all(y.to_vector() == -3.0)    # nothing was written
    # the allocating entry point takes the same product, and the context still works afterwards
    got = dev.matmul_fw(ta, tb).to_vector()
    assert np.all(got == float(dj))
    y2 = dev.new_tensor_by_constant(pa.Shape([64, 64]), 0.0)
    _lib.call("phip_matmul_fw_f32_noalloc", dev.ctx(), ta.handle(), tb.handle(), y2.mutable_handle(), 64, 64, 64, 1, 1)
    assert np.all(y2.to_vector() == 64.0)
    dev.close()
