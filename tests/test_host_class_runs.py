"""The C++ class primitiv::devices::HIP and its C-API constructors, LINKED with
the real primitiv core and RUN on the CPU of the build container.

libphip is replaced by a host stand-in (tests/host_class/phip_host_stub.cc), so
what these tests exercise is the class itself: which libphip entry each Device
virtual calls and with which arguments in which order, handles and
copy-on-write, the memory pool wiring, the error convention, the C-API
constructors - everything a GPU run through the Python mirror cannot see.  The
golden vectors are the reference's own (tests/golden/*.json); the cases are the
ones the GPU tests replay through the mirror, run here through
Device::matmul_fw / matmul_bw / ... as primitiv's Graph and Tensor code calls
them.  Skipped where the primitiv source tree is absent (any GPU box).
"""
import ctypes

import numpy as np
import pytest

import host_class_lib as hc
import primitiv_amd as pa
from util import norm_rel_err, ulp_diff, vector_match

pytestmark = pytest.mark.skipif(not hc.available(), reason=hc.REASON)

S = pa.Shape
STORAGES = ["f32", "f16", "bf16"]


@pytest.fixture(scope="module")
def dev():
    d = hc.HostDevice("f32")
    yield d
    d.close()


@pytest.fixture(scope="module", params=STORAGES)
def anydev(request):
    d = hc.HostDevice(request.param)
    yield d
    d.close()


# ---- identity, construction, lifetime ------------------------------------------------

def test_device_identity_and_invalid_ids():
    n = ctypes.c_uint32(0)
    hc.call("hc_num_devices", ctypes.byref(n))
    assert n.value == 1
    ok = ctypes.c_int(-1)
    hc.call("hc_check_support", 0, ctypes.byref(ok))
    assert ok.value == 1
    hc.call("hc_check_support", n.value, ctypes.byref(ok))
    assert ok.value == 0
    # test/cuda_device_test.cc:45-48
    for bad in (n.value, 12345678):
        with pytest.raises(hc.HostError) as e:
            hc.HostDevice("f32", device_id=bad)
        assert "Invalid device ID" in str(e.value)
    d32, d16, dbf = hc.HostDevice("f32"), hc.HostDevice("f16"), hc.HostDevice("bf16")
    assert d32.type() == pa.DeviceType.HIP == 0x00030000
    assert d16.type() == dbf.type() == pa.DeviceType.HIP16 == 0x00030001
    hc.call("hc_device_dump_description", d32.ptr)
    hc.call("hc_device_set_deterministic", d32.ptr, 1)
    hc.call("hc_device_set_overlap", d32.ptr, 0)
    hc.call("hc_device_set_overlap", d32.ptr, 1)
    hc.call("hc_device_set_deferred_zero_fill", d32.ptr, 0)
    hc.call("hc_device_set_deferred_zero_fill", d32.ptr, 1)
    p = ctypes.c_void_p()
    hc.call("hc_device_new_hip16", 0, 5, ctypes.byref(p))       # the CUDA16-shaped constructor
    t = ctypes.c_uint32(0)
    hc.call("hc_device_type", p, ctypes.byref(t))
    assert t.value == pa.DeviceType.HIP16
    hc.call("hc_device_delete", p)
    for d in (d32, d16, dbf):
        d.close()


def test_tensor_outlives_device_and_nothing_leaks():
    # test/cuda_device_test.cc:50-78
    before = hc.stub_stats()
    for storage in range(3):
        hc.call("hc_scenario_tensor_outlives_device", storage)
    d = hc.HostDevice("f32")
    x1 = d.new_tensor_by_constant(S([]), 0)
    x2 = d.new_tensor_by_constant(S([16, 16]), 0)
    x3 = d.new_tensor_by_constant(S([16, 16, 16], 16), 0)
    assert hc.stub_stats()["live_blocks"] == before["live_blocks"] + 3
    del x1, x2, x3
    d.close()
    after = hc.stub_stats()
    assert after["live_blocks"] == before["live_blocks"] and after["live_bytes"] == before["live_bytes"]
    assert after["live_contexts"] == before["live_contexts"]


def test_new_tensor_reset_and_allocated_blocks(anydev):
    # test/tensor_test.cc:73-143,391-465
    d = anydev
    x = d.new_tensor_by_constant(S([2, 2], 3), 5)
    assert vector_match([5] * 12, x.to_vector())
    x.reset(-2.5)
    assert vector_match([-2.5] * 12, x.to_vector())
    data = [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12]
    x = d.new_tensor_by_vector(S([2, 2], 3), data)
    assert x.shape() == S([2, 2], 3) and vector_match(data, x.to_vector())
    x.reset_by_array(np.arange(12, 0, -1))
    assert vector_match(np.arange(12, 0, -1), x.to_vector())
    with pytest.raises(hc.HostError):
        d.new_tensor_by_vector(S([2, 2], 3), [1, 2, 3])
    x = d.new_tensor_by_vector([3], [1, 2, 3])      # odd count: even-rounded storage on the 16-bit devices
    assert vector_match([1, 2, 3], x.to_vector())
    assert d.new_tensor_by_constant([], 7).to_float() == 7.0
    inv = ctypes.c_void_p()
    hc.call("hc_tensor_invalid", ctypes.byref(inv))
    t = hc.HostTensor(inv)
    assert not t.valid()
    with pytest.raises(hc.HostError):
        t.shape()


def test_pool_blocks_are_powers_of_two_and_reused():
    # primitiv::MemoryPool over phip_malloc: 2^k bytes, at least 8 (test/tensor_test.cc:114-143)
    d = hc.HostDevice("f32")
    base = hc.stub_stats()
    keep = []
    expect = 0
    for n, block in ((1, 8), (2, 8), (3, 16), (4, 16), (5, 32), (1024, 4096), (1025, 8192)):
        keep.append(d.new_tensor_by_constant([n], 0))
        expect += block
        assert hc.stub_stats()["live_bytes"] - base["live_bytes"] == expect
    calls = hc.stub_stats()["malloc_calls"]
    del keep
    again = [d.new_tensor_by_constant([n], 1) for n in (1, 3, 5, 1024, 1025)]
    assert hc.stub_stats()["malloc_calls"] == calls          # every block came back out of the pool
    del again
    d.close()
    assert hc.stub_stats()["live_bytes"] == base["live_bytes"]


def test_out_of_memory_releases_idle_blocks_and_retries():
    # primitiv/core/memory_pool.cc:53-63: a failed allocation frees the pool's idle blocks and is tried again;
    # the class also hands back libphip's own cached scratch before the retry
    d = hc.HostDevice("f32")
    base = hc.stub_stats()
    big = d.new_tensor_by_constant([1 << 18], 0)             # 1 MiB, then idle in the pool
    del big
    assert hc.stub_stats()["live_bytes"] - base["live_bytes"] == 1 << 20
    hc.stub_set_memory_limit(base["live_bytes"] + (1 << 20) + (1 << 18))
    try:
        x = d.new_tensor_by_constant([1 << 17], 3)           # 512 KiB: does not fit beside the idle MiB
        now = hc.stub_stats()
        # first try fails, libphip's scratch pool is released, second try fails, the tensor pool frees its
        # idle MiB, third try succeeds
        assert now["failed_mallocs"] == base["failed_mallocs"] + 2
        assert now["release_calls"] == base["release_calls"] + 1
        assert now["live_bytes"] - base["live_bytes"] == 1 << 19
        assert float(x.to_vector()[-1]) == 3.0
        with pytest.raises(hc.HostError) as e:                # truly too large: the error surfaces
            d.new_tensor_by_constant([1 << 20], 0)
        assert "Memory allocation failed" in str(e.value) or "exhausted" in str(e.value)
        del x
    finally:
        hc.stub_set_memory_limit(0)
    d.close()


# ---- the matmul path: the reference's golden vectors through Device::matmul_fw / matmul_bw ---------

def test_matmul_forward_golden(dev, golden):
    # test/tensor_forward_test.cc:1798-1870
    for c in golden["matmul_fw"]:
        a = dev.new_tensor_by_vector(S([c["di"], c["dj"]], c["ba"]), c["a"])
        b = dev.new_tensor_by_vector(S([c["dj"], c["dk"]], c["bb"]), c["b"])
        y = dev.matmul_fw(a, b)
        assert y.shape() == S([c["di"], c["dk"]], max(c["ba"], c["bb"])), c["source"]
        assert vector_match(c["y"], y.to_vector()), c["source"]


def test_matmul_forward_large_golden(dev, golden):
    # test/tensor_forward_test.cc:1872-1905: non-square use would be caught by a != b
    n = golden["matmul_fw_large"]["n"]
    i = np.arange(n, dtype=np.float64)
    a = dev.new_tensor_by_vector([n, n], np.tile(i / 16.0, n))
    b = dev.new_tensor_by_vector([n, n], np.repeat(i / 16.0, n))
    assert vector_match(np.outer(i, i).T.reshape(-1) * n / 256.0, dev.matmul_fw(a, b).to_vector())
    assert vector_match(np.full(n * n, np.sum(i * i) / 256.0), dev.matmul_fw(b, a).to_vector())


def test_matmul_backward_golden(anydev, golden):
    # test/tensor_backward_test.cc:1599-1668, test/operator_impl_test.cc:1132-1144; small integers are
    # exact in the 16-bit formats too
    d = anydev
    for c in golden["matmul_bw"] + [golden["matmul_operator"]]:
        a = d.new_tensor_by_vector(S([c["di"], c["dj"]], c["ba"]), c["a"])
        b = d.new_tensor_by_vector(S([c["dj"], c["dk"]], c["bb"]), c["b"])
        y = d.matmul_fw(a, b)
        gy = d.new_tensor_by_vector(y.shape(), c["gy"])
        ga = d.new_tensor_by_constant(a.shape(), 0)
        gb = d.new_tensor_by_constant(b.shape(), 0)
        d.matmul_bw(a, b, y, gy, ga, gb)
        assert vector_match(c["ga"], ga.to_vector()), c["source"]
        assert vector_match(c["gb"], gb.to_vector()), c["source"]
        d.matmul_bw(a, b, y, gy, ga, gb)                      # gradients accumulate
        assert vector_match(2 * np.asarray(c["ga"]), ga.to_vector()), c["source"]


def test_matmul_rectangular_random_against_float64(anydev):
    # distinct di, dj, dk and batch sizes: any swapped argument changes the result or its shape
    d = anydev
    tol = 1e-5 if d.storage == "f32" else 2e-2
    rng = np.random.default_rng(3)
    for di, dj, dk, ba, bb in [(3, 5, 7, 1, 1), (4, 6, 5, 3, 3), (5, 3, 2, 1, 4), (2, 7, 3, 4, 1)]:
        bs = max(ba, bb)
        a = rng.standard_normal(di * dj * ba).astype(np.float32)
        b = rng.standard_normal(dj * dk * bb).astype(np.float32)
        gy = rng.standard_normal(di * dk * bs).astype(np.float32)
        ta, tb = d.new_tensor_by_vector(S([di, dj], ba), a), d.new_tensor_by_vector(S([dj, dk], bb), b)
        ty = d.matmul_fw(ta, tb)
        ga, gb = d.new_tensor_by_constant(ta.shape(), 0), d.new_tensor_by_constant(tb.shape(), 0)
        d.matmul_bw(ta, tb, ty, d.new_tensor_by_vector(ty.shape(), gy), ga, gb)
        A = a.astype(np.float64).reshape(ba, dj, di).transpose(0, 2, 1)
        B = b.astype(np.float64).reshape(bb, dk, dj).transpose(0, 2, 1)
        G = gy.astype(np.float64).reshape(bs, dk, di).transpose(0, 2, 1)
        Y = np.matmul(A, B)
        GA, GB = np.matmul(G, B.transpose(0, 2, 1)), np.matmul(A.transpose(0, 2, 1), G)
        if ba == 1:
            GA = GA.sum(axis=0, keepdims=True)
        if bb == 1:
            GB = GB.sum(axis=0, keepdims=True)
        flat = lambda M: M.transpose(0, 2, 1).reshape(-1)
        assert norm_rel_err(ty.to_vector(), flat(Y)) <= tol
        assert norm_rel_err(ga.to_vector(), flat(GA)) <= tol
        assert norm_rel_err(gb.to_vector(), flat(GB)) <= tol


def test_matmul_shape_errors(dev, golden):
    # test/tensor_forward_test.cc:1907-1927 and the checks of Device::matmul_bw (core/device.cc:277-301)
    for c in golden["shape_matmul_invalid"]["cases"]:
        a = dev.new_tensor_by_constant(S(c["a"], c["ba"]), 0)
        b = dev.new_tensor_by_constant(S(c["b"], c["bb"]), 0)
        with pytest.raises(hc.HostError):
            dev.matmul_fw(a, b)
    a, b = dev.new_tensor_by_constant([2, 3], 0), dev.new_tensor_by_constant([3, 4], 0)
    y = dev.matmul_fw(a, b)
    bad = dev.new_tensor_by_constant([2, 5], 0)
    with pytest.raises(hc.HostError):
        dev.matmul_bw(a, b, y, y, bad, b)
    other = hc.HostDevice("f32")
    foreign = other.new_tensor_by_constant([3, 4], 0)
    with pytest.raises(hc.HostError) as e:
        dev.matmul_fw(a, foreign)
    assert "Device mismatched" in str(e.value)
    del foreign
    other.close()


def test_gradient_into_a_shared_block_is_copied_first(anydev):
    # primitiv/core/tensor.cc:33-41: a Tensor that shares its block with another gets a private copy
    # before it is written; matmul_bw takes its writable handles before anything is enqueued
    d = anydev
    a = d.new_tensor_by_vector([2, 2], [1, 2, 3, 4])
    b = d.new_tensor_by_vector([2, 2], [1, 0, 0, 1])
    y = d.matmul_fw(a, b)
    gy = d.new_tensor_by_vector([2, 2], [1, 1, 1, 1])
    ga = d.new_tensor_by_constant([2, 2], 10)
    gb = d.new_tensor_by_constant([2, 2], 20)
    ga_twin, gb_twin = ga.share(), gb.share()
    d.matmul_bw(a, b, y, gy, ga, gb)
    assert vector_match([10] * 4, ga_twin.to_vector()) and vector_match([20] * 4, gb_twin.to_vector())
    assert vector_match([11] * 4, ga.to_vector())            # gy . b^T = ones
    assert vector_match([23, 27, 23, 27], gb.to_vector())    # a^T . gy = [[3,3],[7,7]]


def test_inplace_add_golden_and_copy_on_write(anydev, golden):
    # test/tensor_test.cc:541-631
    d = anydev
    for c in golden["inplace_add"]:
        for via_tensor in (True, False):
            y = d.new_tensor_by_vector(S([c["volume"]], c["by"]), c["y_in"])
            x = d.new_tensor_by_vector(S([c["volume"]], c["bx"]), c["x"])
            twin = y.share()
            if via_tensor:
                y.inplace_add(x)                              # Tensor::inplace_add
            else:
                d.inplace_add(x, y)                           # Device::inplace_add
            assert vector_match(c["y_out"], y.to_vector()), c["source"]
            assert vector_match(c["y_in"], twin.to_vector()), c["source"]


def test_batch_sum_golden(anydev, golden):
    # test/tensor_forward_test.cc:2920-2934
    for c in golden["batch_sum"]:
        x = anydev.new_tensor_by_vector(S([c["volume"]], c["bs"]), c["x"])
        y = anydev.batch_sum_fw(x)
        assert y.shape() == S([c["volume"]]) and vector_match(c["y"], y.to_vector())


def test_copies(anydev):
    # test/tensor_forward_test.cc:67-84: within a device, between device objects of every storage pair, and
    # to and from one of the reference's own host devices
    data = np.arange(1, 13, dtype=np.float32)
    x = anydev.new_tensor_by_vector(S([2, 2], 3), data)
    same = anydev.copy_tensor(x)
    assert same.shape() == x.shape() and vector_match(data, same.to_vector())
    for storage in STORAGES:
        other = hc.HostDevice(storage)
        y = other.copy_tensor(x)
        assert y.shape() == x.shape() and vector_match(data, y.to_vector())
        del y
        other.close()
    out = np.zeros(12, dtype=np.float32)
    hc.call("hc_scenario_copy_through_naive", anydev.ptr, data.ctypes.data_as(ctypes.c_void_p), 12,
            out.ctypes.data_as(ctypes.c_void_p))
    assert vector_match(data, out)


# ---- the C API ----------------------------------------------------------------------------

def test_c_api_constructors_and_matmul(golden):
    # primitivCreateHipDeviceWithSeed -> primitivApplyTensorInput -> primitivApplyTensorMatmul
    # (primitiv/c/functions.cc:334-343) -> primitivEvaluateTensorAsArray, all through primitiv's C API
    L = hc.lib()
    n = ctypes.c_uint32(99)
    hc.c_api("primitivGetNumHipDevices", ctypes.byref(n))
    assert n.value == 1
    dev = ctypes.c_void_p()
    hc.c_api("primitivCreateHipDeviceWithSeed", 0, 1234, ctypes.byref(dev))
    c = golden["matmul_fw"][1]                                # CheckMatMulAB: 3x4 . 4x6

    def tensor(dims, batch, values):
        arr = (ctypes.c_uint32 * len(dims))(*dims)
        shape = ctypes.c_void_p()
        hc.c_api("primitivCreateShapeWithDims", arr, ctypes.c_size_t(len(dims)), ctypes.c_uint32(batch),
                 ctypes.byref(shape))
        v = np.asarray(values, dtype=np.float32)
        t = ctypes.c_void_p()
        hc.c_api("primitivApplyTensorInput", shape, v.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(v.size), dev,
                 ctypes.byref(t))
        hc.c_api("primitivDeleteShape", shape)
        return t

    a = tensor([c["di"], c["dj"]], c["ba"], c["a"])
    b = tensor([c["dj"], c["dk"]], c["bb"], c["b"])
    y = ctypes.c_void_p()
    hc.c_api("primitivApplyTensorMatmul", a, b, ctypes.byref(y))
    size = ctypes.c_size_t(0)
    hc.c_api("primitivEvaluateTensorAsArray", y, None, ctypes.byref(size))
    out = np.zeros(size.value, dtype=np.float32)
    hc.c_api("primitivEvaluateTensorAsArray", y, out.ctypes.data_as(ctypes.c_void_p), ctypes.byref(size))
    assert vector_match(c["y"], out)
    for t in (a, b, y):
        hc.c_api("primitivDeleteTensor", t)
    hc.c_api("primitivDeleteDevice", dev)

    # the other constructors, and the error convention of the C API (status + message, no exception)
    for ctor, args in (("primitivCreateHipDevice", (0,)), ("primitivCreateHip16DeviceWithSeed", (0, 7, 0)),
                       ("primitivCreateHip16DeviceWithSeed", (0, 7, 1))):
        p = ctypes.c_void_p()
        hc.c_api(ctor, *args, ctypes.byref(p))
        hc.c_api("primitivDeleteDevice", p)
    assert L.primitivCreateHipDeviceWithSeed(0, 1, None) != 0
    L.primitivResetStatus()
    with pytest.raises(hc.HostError) as e:
        hc.c_api("primitivCreateHipDevice", 12345678, ctypes.byref(ctypes.c_void_p()))
    assert "Invalid device ID" in str(e.value)
    d = hc.HostDevice("bf16", via_c_api=True)
    assert d.type() == pa.DeviceType.HIP16
    hc.c_api("primitivDeleteDevice", d.ptr)
    d.ptr = ctypes.c_void_p()


# ---- primitiv's own Graph / Parameter / Optimizer on the device ------------------------------

def test_graph_parameter_optimizer_training_step(anydev):
    # the network of test/graph_test.cc:362-435; its node values are golden there
    f32 = anydev.storage == "f32"
    values, grads, updated = (np.zeros(n, dtype=np.float32) for n in (62, 9, 9))
    eta = 0.25
    hc.call("hc_scenario_xor_training_step", anydev.ptr, ctypes.c_float(eta),
            *[v.ctypes.data_as(ctypes.c_void_p) for v in (values, grads, updated)])
    h1, h2, h3, h4 = .76159416, .99505475, -.23346060, -1.5231883
    h5, h6, h7 = .76653940, -.52318831, .47681169
    expected = [
        [1, 1, 1, -1, -1, 1, -1, -1], [1, -1, 1, -1], [-1, -1], [1, 1], [1], [2, -2, 0, 0, 0, 0, -2, 2],
        [1, -3, -1, -1, -1, -1, -3, 1], [h1, -h2, -h1, -h1, -h1, -h1, -h2, h1], [h3, h4, h4, h3], [h5, h6, h6, h5],
        [1, -1, -1, 1], [h3, h7, h7, h3], [h3 * h3, h7 * h7, h7 * h7, h3 * h3], [2 * (h3 * h3 + h7 * h7)],
    ]
    want = np.concatenate([np.asarray(e, dtype=np.float32) for e in expected])
    assert np.allclose(values, want, rtol=0, atol=2e-7 if f32 else 2e-2)
    # the derivative in float64
    X = np.array([[1, 1], [1, -1], [-1, 1], [-1, -1]], dtype=np.float64)
    W1 = np.array([[1, 1], [-1, -1]], dtype=np.float64)
    B1, W2, B2, T = np.array([-1., -1.]), np.array([1., 1.]), 1.0, np.array([1., -1., -1., 1.])
    H = np.tanh(X @ W1.T + B1)
    D = 2 * ((H @ W2 + B2) - T)
    GA = np.outer(D, W2) * (1 - H ** 2)
    G = np.concatenate([(GA.T @ X).T.reshape(-1), GA.sum(axis=0), D @ H, [D.sum()]])
    tol = 1e-5 if f32 else 3e-2
    assert np.allclose(grads, G, atol=tol)
    P0 = np.array([1, -1, 1, -1, -1, -1, 1, 1, 1], dtype=np.float64)
    assert np.allclose(updated, P0 - eta * G, atol=tol)


def test_xor_perceptron_op_by_op(anydev):
    import test_gpu_graph
    test_gpu_graph.test_xor_perceptron_forward_and_backward(anydev)
    test_gpu_graph.test_matmul_gradients_of_one_tensor_used_twice(anydev)


def test_lstm_graphs_op_by_op(anydev):
    # test/graph_test.cc:437-646 through Device's front, operator by operator
    import test_gpu_graph
    test_gpu_graph.test_lstm_with_separate_gate_weights(anydev)
    test_gpu_graph.test_lstm_with_stacked_gate_weights(anydev)


@pytest.mark.parametrize("stacked", [0, 1])
def test_lstm_graphs_with_the_reference_graph(anydev, stacked):
    # the same two tests built with primitiv's own Graph / Node / Parameter on devices::HIP:
    # operator count, the four golden losses at the test's 1e-6, gradients against float64
    import test_gpu_graph as tg
    case = tg.GRAPH_VECTORS["CheckConcatLSTM" if stacked else "CheckLSTM"]
    ref = tg._lstm_float64(tg.GRAPH_VECTORS["CheckConcatLSTM"])
    order = (["pWx", "pWh", "pb"] if stacked else
             ["pWix", "pWfx", "pWox", "pWjx", "pWih", "pWfh", "pWoh", "pWjh", "pbi", "pbf", "pbo", "pbj"])
    params = np.concatenate([np.asarray(case["parameters"][k]["values"], dtype=np.float32) for k in order])
    x = np.asarray(case["inputs"]["x"]["values"], dtype=np.float32)
    h = np.asarray(case["inputs"]["h"]["values"], dtype=np.float32)
    losses, grads = np.zeros(4, np.float32), np.zeros(40, np.float32)
    total, nops = ctypes.c_float(0), ctypes.c_uint32(0)
    vp = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    hc.call("hc_scenario_lstm_step", anydev.ptr, stacked, vp(params), vp(x), vp(h), vp(losses), ctypes.byref(total),
            ctypes.byref(nops), vp(grads))
    assert nops.value == case["num_operators"]
    loss_tol, grad_tol = tg._lstm_tolerances(anydev)
    want = np.asarray(case["expected_losses"], dtype=np.float32)
    assert np.allclose(losses, want, rtol=0, atol=loss_tol)
    assert abs(total.value - float(want.sum())) <= 4 * loss_tol
    if stacked:
        G = np.concatenate([tg._colmajor(ref["gWx"]), tg._colmajor(ref["gWh"]), ref["gb"]])
    else:
        rows = [slice(0, 2), slice(2, 4), slice(4, 6), slice(6, 8)]
        G = np.concatenate([tg._colmajor(ref["gWx"][r]) for r in rows] + [tg._colmajor(ref["gWh"][r]) for r in rows] +
                           [ref["gb"][r] for r in rows])
    assert np.allclose(grads, G, rtol=0, atol=grad_tol)
