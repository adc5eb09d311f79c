"""The helpers around the matmul path (fill, copies, in-place add with
minibatch broadcasting, minibatch sum, the memory pool), through the C ABI,
against the reference's golden vectors and the oracle."""
import ctypes

import numpy as np
import pytest

import oracle
import primitiv_amd as pa
from primitiv_amd import _lib
from util import norm_rel_err, vector_match

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def devs():
    ds = [pa.HIP(0), pa.HIP16(0, storage="f16"), pa.HIP16(0, storage="bf16")]
    yield ds
    for d in ds:
        d.close()


def test_device_identity(devs):
    assert pa.HIP.num_devices() >= 1
    assert pa.HIP.check_support(0)
    assert not pa.HIP.check_support(pa.HIP.num_devices())
    with pytest.raises(pa.Error):
        pa.HIP(pa.HIP.num_devices())          # test/cuda_device_test.cc:45-48
    info = devs[0].info()
    assert info.arch.decode().startswith("gfx950")
    assert info.wavefront_size == 64 and info.compute_units > 0
    assert "Type: HIP" in devs[0].dump_description()
    assert devs[0].type() == pa.DeviceType.HIP and devs[1].type() == pa.DeviceType.HIP16


def test_new_tensor_and_reset(devs):
    # test/tensor_test.cc:73-143,391-465
    for d in devs:
        x = d.new_tensor_by_constant(pa.Shape([2, 2], 3), 5)
        assert vector_match([5] * 12, x.to_vector())
        d.reset_tensor(-2.5, x)
        assert vector_match([-2.5] * 12, x.to_vector())
        data = [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12]
        x = d.new_tensor_by_vector(pa.Shape([2, 2], 3), data)
        assert vector_match(data, x.to_vector())
        d.reset_tensor_by_array(np.arange(12, 0, -1), x)
        assert vector_match(np.arange(12, 0, -1), x.to_vector())
        with pytest.raises(pa.Error):
            d.new_tensor_by_vector(pa.Shape([2, 2], 3), [1, 2, 3])
        # odd element count on the half devices (even-rounded storage)
        x = d.new_tensor_by_vector([3], [1, 2, 3])
        assert vector_match([1, 2, 3], x.to_vector())
        s = d.new_tensor_by_constant([], 7)
        assert s.to_float() == 7.0
    assert not pa.Tensor().valid()
    with pytest.raises(pa.Error):
        pa.Tensor().shape()


def test_allocated_size_and_pool(devs, golden):
    d = devs[0]
    # power-of-two blocks of at least 8 bytes (test/tensor_test.cc:114-143)
    for n, expect in ((1, 8), (2, 8), (3, 16), (4, 16), (5, 32), (1024, 4096), (1025, 8192)):
        assert d.new_raw_tensor([n]).allocated_size() == expect
    p = golden["pool_block_size"]
    for size, exp in zip(p["sizes"], p["expected_min1"]):
        ptr, got = ctypes.c_void_p(), ctypes.c_size_t(77)
        _lib.call("phip_pool_alloc", d.ctx(), size, ctypes.byref(ptr), ctypes.byref(got))
        want = 0 if size == 0 else max(exp, 8)
        assert got.value == want == oracle.pool_block_size(size, 8)
        assert (ptr.value is None) == (size == 0)
        _lib.call("phip_pool_free", d.ctx(), ptr)
    # a freed block is handed out again for the same size class
    p1, p2 = ctypes.c_void_p(), ctypes.c_void_p()
    _lib.call("phip_pool_alloc", d.ctx(), 1000, ctypes.byref(p1), None)
    _lib.call("phip_pool_free", d.ctx(), p1)
    _lib.call("phip_pool_alloc", d.ctx(), 600, ctypes.byref(p2), None)
    assert p1.value == p2.value
    _lib.call("phip_pool_free", d.ctx(), p2)
    with pytest.raises(pa.Error):
        _lib.call("phip_pool_free", d.ctx(), ctypes.c_void_p(12345))  # unknown handle
    # more than the device holds: error, not a crash; the pool retries after
    # releasing its idle blocks (primitiv/core/memory_pool.cc:53-63)
    huge = ctypes.c_void_p()
    rc = _lib.lib().phip_pool_alloc(d.ctx(), 1 << 40, ctypes.byref(huge), None)
    assert rc == _lib.PHIP_ERR_OUT_OF_MEMORY and not huge.value
    sup, res = ctypes.c_uint64(), ctypes.c_uint64()
    _lib.call("phip_pool_stats", d.ctx(), ctypes.byref(sup), ctypes.byref(res))
    assert res.value == 0
    _lib.call("phip_pool_release_reserved", d.ctx())


def test_out_of_memory_reclaims_idle_blocks_of_every_context_on_the_gpu(devs):
    # a fp32 and a 16-bit device object on one GPU each cache idle blocks; when an allocation fails, the retry
    # (primitiv/core/memory_pool.cc:53-63) must be able to use what the other one holds
    a, b = devs[0], devs[1]

    def reserved(d):
        sup, res = ctypes.c_uint64(), ctypes.c_uint64()
        _lib.call("phip_pool_stats", d.ctx(), ctypes.byref(sup), ctypes.byref(res))
        return res.value

    p = ctypes.c_void_p()
    _lib.call("phip_pool_alloc", a.ctx(), 1 << 20, ctypes.byref(p), None)
    _lib.call("phip_pool_free", a.ctx(), p)
    assert reserved(a) >= 1 << 20
    huge = ctypes.c_void_p()
    assert _lib.lib().phip_pool_alloc(b.ctx(), 1 << 40, ctypes.byref(huge), None) == _lib.PHIP_ERR_OUT_OF_MEMORY
    assert reserved(a) == 0 and reserved(b) == 0
    _lib.call("phip_pool_alloc", a.ctx(), 1 << 20, ctypes.byref(p), None)
    _lib.call("phip_pool_free", a.ctx(), p)
    assert _lib.lib().phip_malloc(b.ctx(), 1 << 40, ctypes.byref(huge)) == _lib.PHIP_ERR_OUT_OF_MEMORY
    assert reserved(a) == 0
    x = a.new_tensor_by_constant([1000], 2.0)          # both contexts still work
    assert float(x.to_vector()[999]) == 2.0


def test_tensor_outlives_device():
    # test/cuda_device_test.cc:66-78: dropping a tensor after its device is fine
    d = pa.HIP(0)
    x = d.new_tensor_by_constant([4], 1)
    d.close()
    with pytest.raises(pa.Error):
        x.to_vector()
    del x


def test_copy_between_devices(devs):
    # test/tensor_forward_test.cc:67-84
    data = [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12]
    for src in devs:
        x = src.new_tensor_by_vector(pa.Shape([2, 2], 3), data)
        for dst in devs:
            y = dst.copy_tensor(x)
            assert y.device() is dst and y.shape() == x.shape()
            assert vector_match(data, y.to_vector())
    other = pa.HIP(0)
    x = devs[0].new_tensor_by_vector([2], [1, 2])
    with pytest.raises(pa.Error):
        other.matmul_fw(x, x)                   # "Device mismatched"
    other.close()


def test_copy_between_devices_waits_for_the_source(devs):
    # every device object has a stream of its own: a copy to another object must
    # see the kernels still queued on the source, and the source may be dropped at once
    src, other = devs[0], pa.HIP(0)
    n = 1 << 22
    x = src.new_tensor_by_constant([n], 1.0)
    for _ in range(20):
        x = src.const_fw("add_const", x, 1.0)
    y = other.copy_tensor(x)
    del x
    assert np.array_equal(y.to_vector(), np.full(n, 21, np.float32))
    for d16 in devs[1:]:
        z = d16.copy_tensor(other.const_fw("add_const", y, 1.0))     # fp32 -> 16-bit on the GPU
        assert np.array_equal(z.to_vector(), np.full(n, 22, np.float32))
        back = other.copy_tensor(d16.const_fw("multiply_const", z, 2.0))   # and back
        assert np.array_equal(back.to_vector(), np.full(n, 44, np.float32))
    other.close()


def test_checkpoint_round_trip(devs, tmp_path):
    # a parameter file written from one device loads into any other
    # (test/parameter_test.cc:284-322 runs the same round trip on one device);
    # the file holds float32, so a 16-bit device rounds once on load and
    # its own values survive save + load unchanged
    from primitiv_amd import parameter_file as pf
    rng = np.random.default_rng(3)
    value = rng.standard_normal(300 * 70).astype(np.float32)
    m1 = rng.standard_normal(300 * 70).astype(np.float32)
    path = str(tmp_path / "param.data")
    for src in devs:
        v = src.new_tensor_by_vector(pa.Shape([300, 70]), value)
        stats = {"adam-m1": src.new_tensor_by_vector(pa.Shape([300, 70]), m1),
                 "adam-m2": src.new_tensor_by_constant(pa.Shape([300, 70]), 0.25)}
        pf.save(path, v, stats)
        held = v.to_vector()
        for dst in devs:
            got, st = pf.load(path, dst)
            assert got.device() is dst and got.shape() == v.shape() and sorted(st) == ["adam-m1", "adam-m2"]
            if dst is src or dst is devs[0]:
                assert np.array_equal(got.to_vector(), held)              # nothing is lost
                assert np.array_equal(st["adam-m1"].to_vector(), stats["adam-m1"].to_vector())
            else:
                assert np.allclose(got.to_vector(), held, rtol=8e-3, atol=1e-6)   # one rounding to 16 bits
            assert np.array_equal(st["adam-m2"].to_vector(), np.full(300 * 70, 0.25, np.float32))
            # the loaded tensor is a working operand on its device
            y = dst.matmul_fw(dst.transpose_fw(got), got)
            assert y.shape() == pa.Shape([70, 70])


def test_inplace_add_golden(devs, golden):
    for d in devs:
        for c in golden["inplace_add"]:
            y = d.new_tensor_by_vector(pa.Shape([2, 2], c["by"]), c["y_in"])
            x = d.new_tensor_by_vector(pa.Shape([2, 2], c["bx"]), c["x"])
            y.inplace_add(x)
            assert vector_match(c["y_out"], y.to_vector()), c["source"]
            y2 = d.new_tensor_by_vector(pa.Shape([2, 2], c["by"]), c["y_in"])
            y2 += x
            assert vector_match(c["y_out"], y2.to_vector()), c["source"]
        # copy-on-write (test/tensor_test.cc:604-631)
        c = golden["inplace_add"][0]
        a = d.new_tensor_by_vector(pa.Shape([2, 2], 3), c["y_in"])
        b = d.new_tensor_by_vector(pa.Shape([2, 2], 3), c["x"])
        copied = a.copy()
        a += b
        assert vector_match(c["y_out"], a.to_vector())
        assert vector_match(c["y_in"], copied.to_vector())
        with pytest.raises(pa.Error):
            a.inplace_add(d.new_tensor_by_constant(pa.Shape([2, 2], 2), 0))
        with pytest.raises(pa.Error):
            a.inplace_add(d.new_tensor_by_constant(pa.Shape([2, 3], 3), 0))


def test_batch_sum_golden(devs, golden):
    for d in devs:
        for c in golden["batch_sum"]:
            x = d.new_tensor_by_vector(pa.Shape([2, 2, 2], c["bs"]), c["x"])
            y = d.batch_sum_fw(x)
            assert y.shape() == pa.Shape([2, 2, 2])
            assert vector_match(c["y"], y.to_vector())


@pytest.mark.parametrize("volume,bx,by", [(1, 1, 1), (1000, 1, 1), (1000, 7, 7), (1001, 7, 1), (999, 1, 7),
                                          (1 << 20, 3, 3), (65537, 33, 1)])
def test_inplace_add_and_batch_sum_random(devs, volume, bx, by):
    rng = np.random.default_rng(volume + bx + by)
    x = rng.standard_normal(volume * bx).astype(np.float32)
    y = rng.standard_normal(volume * by).astype(np.float32)
    want = oracle.inplace_add(x, y, volume, bx, by)
    want_sum = oracle.batch_sum(x, volume, bx)
    for d, tol in zip(devs, (1e-6, 2e-3, 1.6e-2)):
        ty = d.new_tensor_by_vector(pa.Shape([volume], by), y)
        tx = d.new_tensor_by_vector(pa.Shape([volume], bx), x)
        ty += tx
        assert norm_rel_err(ty.to_vector(), want) <= tol
        assert norm_rel_err(d.batch_sum_fw(tx).to_vector(), want_sum) <= tol


def test_storage_conversion_rounds_to_nearest_even(devs):
    x = np.array([1.0, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 65504.0, 1e-8, -2.5, 0.333333], dtype=np.float32)
    got = devs[1].new_tensor_by_vector([x.size], x).to_vector()
    assert np.array_equal(got, x.astype(np.float16).astype(np.float32))
    xb = np.array([1.0, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 3.0e38, -2.5, 0.333333], dtype=np.float32)
    got = devs[2].new_tensor_by_vector([xb.size], xb).to_vector()
    u = xb.view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    assert np.array_equal(got, u.astype(np.uint32).view(np.float32))
