#!/usr/bin/env python3
"""Benchmark of the matmul path (fw + bw) on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W [--workload NAME] [--skip-cpu]

A step is one pass of the hot path over one batch of synthetic seeded input:
one matmul_fw + matmul_bw call pair, or, for the recurrent workloads, their
whole sequence of per-timestep call pairs.  Inputs are resident in HBM before
the timed region starts.  Prints ONE JSON line; `value` is for the headline
workload (square batched fp32), `workloads` carries the same figures for all
five.  The CPU figures come from the CPU oracle timed on this host.
"""
import argparse
import copy
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import primitiv_amd as pa  # noqa: E402
from primitiv_amd import _lib  # noqa: E402
from primitiv_amd.configs import WORKLOADS  # noqa: E402

# Published MI355X peaks (dense).
PEAK_TFLOPS = {"f32": 157.3, "f16": 2516.6, "bf16": 2516.6}
PEAK_HBM_GBS = 8000.0
HEADLINE = "square_batched"
# HBM bytes per step by rocprofv3's counters, from profiles/matmul_workloads_kernel_times_traffic_counters.txt
# section 2: per dispatch FETCH_SIZE x 2.0 KiB + WRITE_SIZE x 1.0 KiB (the factors read off a streaming
# y += x of known size in the same runs), summed over a step's launches ("HBM bytes per step by the
# counters" there).  Algorithmic bytes for comparison are Workload.bytes_per_step().
COUNTER_TRAFFIC_BYTES_PER_STEP = {
    "square_batched": 762.4e6,       # 206.14 + 283.93 + 272.32 MB: the three gemm_f32_lds_kernel launches
    "dense": 14.58e6,                # gemm_f32_tile16_kernel 7.06 + gemm_f32_pair_kernel 7.52 MB
    "rnn_gate": 872.4e6,             # 30 x (9.64 + 19.44 MB)
    "output_projection": 4473.4e6,   # 35 x (gemm_f32_slab_kernel 34.65 + gemm_f32_stream_pair_kernel 93.16 MB)
    "half_storage": 6273.2e6,        # 2 x 2122.67 + 1960.7 + 67.17 MB (transposed copy of a)
}
# per launch of the headline kernel (average of its three operand-layout instantiations)
HEADLINE_TRAFFIC_BYTES = COUNTER_TRAFFIC_BYTES_PER_STEP["square_batched"] / 3


class Resident:
    """One workload with every input already on the device."""

    def __init__(self, dev, w, seed=0):
        self.dev, self.w = dev, w
        a, bs, gys = w.inputs(seed=seed)
        S = pa.Shape
        self.a = dev.new_tensor_by_vector(S([w.di, w.dj], w.ba), a)
        self.b = [dev.new_tensor_by_vector(S([w.dj, w.dk], w.bb), x) for x in bs]
        self.gy = [dev.new_tensor_by_vector(S([w.di, w.dk], w.bs), x) for x in gys]
        self.y = [dev.new_raw_tensor(S([w.di, w.dk], w.bs)) for _ in range(w.steps)]
        # gradient of the shared / persistent operand accumulates across the
        # timesteps; the per-timestep operand gets its own zeroed gradient
        self.ga = dev.new_tensor_by_constant(self.a.shape(), 0)
        self.gb = [dev.new_tensor_by_constant(S([w.dj, w.dk], w.bb), 0) for _ in range(w.steps)]
        l = _lib.lib()
        self.fw = getattr(l, "phip_matmul_fw_" + w.storage)
        self.bw = getattr(l, "phip_matmul_bw_" + w.storage)
        self.dims = (w.di, w.dj, w.dk, w.ba, w.bb)
        self.ptrs = [(self.b[t].handle(), self.gy[t].handle(), self.y[t].handle(), self.gb[t].handle())
                     for t in range(w.steps)]
        dev.sync()

    def step(self):
        ctx, a, ga = self.dev.ctx(), self.a.handle(), self.ga.handle()
        fw, bw, dims = self.fw, self.bw, self.dims
        for b, gy, y, gb in self.ptrs:
            rc = fw(ctx, a, b, y, *dims)
            rc |= bw(ctx, a, b, gy, ga, gb, *dims)
            if rc:
                _lib.check(rc)


# The GPU's clocks take tens of milliseconds of load to settle (square_batched: 114 TFLOP/s behind
# 3 warm-up steps of 0.9 ms, 122 behind 10, 129.6 behind 30 or 100): the untimed warm-up is the
# requested number of steps and at least this much time.
WARMUP_MIN_SECONDS = 0.06


def _warm_up(dev, step, warmup):
    t0 = time.perf_counter()
    for _ in range(warmup):
        step()
    dev.sync()
    while time.perf_counter() - t0 < WARMUP_MIN_SECONDS:
        for _ in range(8):
            step()
        dev.sync()


def time_gpu(dev, res, steps, warmup):
    """(host seconds, event seconds) for `steps` steps."""
    ctx = dev.ctx()
    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    _lib.call("phip_event_create", ctx, ctypes.byref(e0))
    _lib.call("phip_event_create", ctx, ctypes.byref(e1))
    _warm_up(dev, res.step, warmup)
    t0 = time.perf_counter()
    _lib.call("phip_event_record", ctx, e0)
    for _ in range(steps):
        res.step()
    _lib.call("phip_event_record", ctx, e1)
    dev.sync()
    host = time.perf_counter() - t0
    ms = ctypes.c_float()
    _lib.call("phip_event_elapsed_ms", e0, e1, ctypes.byref(ms))
    _lib.call("phip_event_destroy", e0)
    _lib.call("phip_event_destroy", e1)
    return host, ms.value * 1e-3


class _Dims(ctypes.Structure):
    _fields_ = [(n, ctypes.c_uint32) for n in ("di", "dj", "dk", "ba", "bb")]


_bench_lib = None


def _native():
    """libphip_bench.so: the same loops in native code (primitiv_amd/bench_front.cc)."""
    global _bench_lib
    if _bench_lib is None:
        _lib.lib()
        path = os.path.join(ROOT, "primitiv_amd", "libphip_bench.so")
        if not os.path.exists(path):
            raise _lib.Error("libphip_bench.so is not built; run `python -m primitiv_amd.build`")
        l = ctypes.CDLL(path)
        vp, pp, i = ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p), ctypes.c_int
        out = [ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_double)]
        # device pointers are 64-bit: without these ctypes would pass them as C ints
        l.phip_bench_raw_loop.argtypes = [vp, vp, vp, pp, pp, pp, pp, ctypes.POINTER(_Dims), i, i, i] + out
        l.phip_bench_front_loop.argtypes = [vp, vp, vp, pp, pp, ctypes.POINTER(_Dims), i, i, i] + out
        l.phip_bench_raw_loop.restype = l.phip_bench_front_loop.restype = i
        _bench_lib = l
    return _bench_lib


def time_front(dev, res, steps, warmup):
    """Per-step milliseconds of the fp32 workload `res` in native loops: the two entry points on
    preallocated outputs ("raw", what the Python loop above times), and with what primitiv's Device
    front does around them per call ("front": y from the pool, the per-timestep gradient from the pool
    and zero-filled, both handed back; primitiv/core/device.cc:20-24,268-301)."""
    w = res.w
    n = w.steps
    arr = lambda ptrs: (ctypes.c_void_p * n)(*ptrs)
    b, gy = arr([p[0] for p in res.ptrs]), arr([p[1] for p in res.ptrs])
    y, gb = arr([p[2] for p in res.ptrs]), arr([p[3] for p in res.ptrs])
    d = _Dims(w.di, w.dj, w.dk, w.ba, w.bb)
    ev, host = ctypes.c_float(), ctypes.c_double()
    out = {}
    L = _native()
    _lib.check(L.phip_bench_raw_loop(dev.ctx(), res.a.handle(), res.ga.handle(), b, gy, y, gb, ctypes.byref(d), n,
                                     steps, warmup, ctypes.byref(ev), ctypes.byref(host)))
    out["ms_per_step_native_raw"] = ev.value / steps
    out["ms_per_step_native_raw_host_clock"] = host.value / steps
    _lib.check(L.phip_bench_front_loop(dev.ctx(), res.a.handle(), res.ga.handle(), b, gy, ctypes.byref(d), n,
                                       steps, warmup, ctypes.byref(ev), ctypes.byref(host)))
    out["ms_per_step_front"] = ev.value / steps
    out["ms_per_step_front_host_clock"] = host.value / steps
    return out


def cpu_baseline(w, threads=1):
    """Times the CPU oracle (a port of the reference's Eigen device, one
    thread, as the reference builds Eigen without OpenMP) on a bounded sample
    of the workload and scales to TFLOP/s."""
    import oracle
    steps, bb, repeats, sample = w.steps, w.bb, 2, "full workload"
    if w.name.startswith("half_storage"):
        bb, repeats, sample = 1, 1, "1 of the 8 minibatch samples (a shared), fp32"
    elif w.name == "square_batched":
        sample = "one fw+bw call, all 16 samples"
    elif w.name in ("dense",):
        repeats = 5
    rng = np.random.default_rng(0)
    bs = max(w.ba, bb)
    a = rng.standard_normal(w.di * w.dj * w.ba).astype(np.float32)
    b = rng.standard_normal(w.dj * w.dk * bb).astype(np.float32)
    gy = rng.standard_normal(w.di * w.dk * bs).astype(np.float32)
    ga, gb = np.zeros_like(a), np.zeros_like(b)
    best = float("inf")
    for _ in range(repeats):
        t0 = time.perf_counter()
        for _ in range(steps):
            oracle.matmul_fw(a, b, w.di, w.dj, w.dk, w.ba, bb, threads)
            oracle.matmul_bw(a, b, gy, ga, gb, w.di, w.dj, w.dk, w.ba, bb, threads)
        best = min(best, time.perf_counter() - t0)
    flops = 3 * 2 * w.di * w.dj * w.dk * bs * steps
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count()
    return {"value": flops / best / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "host_cores_online": os.cpu_count(), "host_cores_usable": usable,
            "sample": "%s, best of %d, %.2f s" % (sample, repeats, best)}


def _workload(name):
    """A workload of the table, or its half-storage entry with bfloat16 storage (same shapes, same
    inputs; not one of the reference's configurations, reported next to them)."""
    if name == "half_storage_bf16":
        w = copy.copy(WORKLOADS["half_storage"])
        w.name, w.storage = name, "bf16"
        return w
    return WORKLOADS[name]


def measure(name, steps, warmup, skip_cpu, deterministic=False, in_order=False):
    w = _workload(name)
    dev = pa.HIP(0) if w.storage == "f32" else pa.HIP16(0, storage=w.storage)
    dev.set_deterministic(deterministic)
    dev.set_overlap(not in_order)
    res = Resident(dev, w)
    host_s, ev_s = time_gpu(dev, res, steps, warmup)
    front = {}
    if w.storage == "f32":
        # The fp32 workloads are timed by a C++ caller as well (primitiv's callers are C++): the same
        # calls on the same buffers.  That loop is the step of record; the interpreter's loop above is
        # reported beside it (on the dispatch-bound workloads it adds up to a microsecond per call).
        front = time_front(dev, res, steps, warmup)
        front["ms_per_step_python_loop"] = ev_s / steps * 1e3
        front["ms_per_step_python_loop_host_clock"] = host_s / steps * 1e3
        ev_s = front["ms_per_step_native_raw"] * 1e-3 * steps
        host_s = front["ms_per_step_native_raw_host_clock"] * 1e-3 * steps
        # the same loops with every launch on one stream: what the library's second lane for runs of
        # independent matmul calls (phip_set_overlap) contributes
        dev.set_overlap(False)
        one_stream = time_front(dev, res, steps, warmup)
        dev.set_overlap(not in_order)
        front["ms_per_step_in_order"] = one_stream["ms_per_step_native_raw"]
        front["ms_per_step_front_in_order"] = one_stream["ms_per_step_front"]
    del res
    dev.close()
    per_step = ev_s / steps
    tflops = w.flops_per_step() * w.steps / per_step / 1e12
    gbs = w.bytes_per_step() * w.steps / per_step / 1e9
    f_mfma, f_hbm = tflops / PEAK_TFLOPS[w.storage], gbs / PEAK_HBM_GBS
    launches = 3 * w.steps
    out = {
        "workload": name, "dtype": w.storage, "calls_per_step": w.steps,
        "ms_per_step": per_step * 1e3, "ms_per_step_host_clock": host_s / steps * 1e3,
        "us_per_kernel_launch": per_step / launches * 1e6,
        "tflops": tflops, "frac_mfma_peak": f_mfma, "gbs": gbs, "frac_hbm_peak": f_hbm,
        "binding_roofline": "mfma" if f_mfma >= f_hbm else "hbm",
        "frac_binding_roofline": max(f_mfma, f_hbm),
    }
    out.update(front)
    # HBM traffic per step by the counters (profiles/), next to the algorithmic bytes above
    if name in COUNTER_TRAFFIC_BYTES_PER_STEP:
        traffic = COUNTER_TRAFFIC_BYTES_PER_STEP[name]
        out["counter_traffic_bytes_per_step"] = traffic
        out["counter_gbs"] = traffic / per_step / 1e9
        out["counter_frac_hbm_peak"] = traffic / per_step / 1e9 / PEAK_HBM_GBS
    if not skip_cpu:
        out["cpu_baseline"] = cpu_baseline(w)
    return out


def _event_seconds(dev, fn, reps):
    """Average seconds of one fn() over `reps` back-to-back calls, by events on the library's stream."""
    ctx = dev.ctx()
    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    _lib.call("phip_event_create", ctx, ctypes.byref(e0))
    _lib.call("phip_event_create", ctx, ctypes.byref(e1))
    for _ in range(2):
        fn()
    dev.sync()
    _lib.call("phip_event_record", ctx, e0)
    for _ in range(reps):
        fn()
    _lib.call("phip_event_record", ctx, e1)
    ms = ctypes.c_float()
    _lib.call("phip_event_elapsed_ms", e0, e1, ctypes.byref(ms))
    _lib.call("phip_event_destroy", e0)
    _lib.call("phip_event_destroy", e1)
    return ms.value * 1e-3 / reps


def _wall_seconds(dev, fn, reps):
    """Average seconds of one blocking fn() (a call that waits for the device itself) by the host clock."""
    for _ in range(2):
        fn()
    dev.sync()
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    dev.sync()
    return (time.perf_counter() - t0) / reps


def measure_pointwise(reps=20):
    """Streaming rate of the elementwise kernels: algorithmic bytes (every operand the
    operation needs read once, every result written once, a gradient read and written)
    over the event time, against the 8 TB/s HBM peak.  Large cases are 64 Mi elements per
    tensor; the bias cases use a 1 Mi-element bias over a minibatch of 64, and the
    recurrent-layer shape (2048 x 64) shows the latency floor."""
    S = pa.Shape
    out = []
    for storage, item in (("f32", 4), ("f16", 2)):
        dev = pa.HIP(0) if storage == "f32" else pa.HIP16(0, storage=storage)
        n = 64 << 20
        x = dev.new_tensor_by_constant(S([n]), 0.5)
        y = dev.new_tensor_by_constant(S([n]), 0.25)
        g = dev.new_tensor_by_constant(S([n]), 0.0)
        g2 = dev.new_tensor_by_constant(S([n]), 0.0)
        vol, bs = 1 << 20, 64
        bias = dev.new_tensor_by_constant(S([vol]), 0.5)
        gbias = dev.new_tensor_by_constant(S([vol]), 0.0)
        xb = dev.new_tensor_by_constant(S([vol], bs), 0.5)
        gxb = dev.new_tensor_by_constant(S([vol], bs), 0.0)
        sv, sb = 2048, 64
        sbias = dev.new_tensor_by_constant(S([sv]), 0.5)
        sx = dev.new_tensor_by_constant(S([sv], sb), 0.5)
        sg = dev.new_tensor_by_constant(S([sv], sb), 0.0)
        sgb = dev.new_tensor_by_constant(S([sv]), 0.0)
        big, med = n * item, vol * bs * item
        cases = [
            ("tanh_fw", lambda: dev.unary_fw("tanh", x), 2 * big),
            ("tanh_bw", lambda: dev.unary_bw("tanh", x, y, x, g), 4 * big),
            ("prelu_fw", lambda: dev.const_fw("prelu", x, 0.01), 2 * big),
            ("add_fw", lambda: dev.binary_fw("add", x, y), 3 * big),
            ("multiply_bw", lambda: dev.binary_bw("multiply", x, y, x, y, g, g2), 7 * big),
            ("bias_add_fw", lambda: dev.binary_fw("add", xb, bias), 2 * med + vol * item),
            ("bias_add_bw", lambda: dev.binary_bw("add", xb, bias, xb, xb, gxb, gbias), 3 * med + 2 * vol * item),
            ("inplace_add", lambda: dev.inplace_add(x, y), 3 * big),
            ("inplace_multiply_const", lambda: dev.inplace_multiply_const(1.0, y), 2 * big),
            ("bias_add_fw_2048x64", lambda: dev.binary_fw("add", sx, sbias), (2 * sv * sb + sv) * item),
            ("bias_add_bw_2048x64", lambda: dev.binary_bw("add", sx, sbias, sx, sx, sg, sgb),
             (3 * sv * sb + 2 * sv) * item),
        ]
        for name, fn, nbytes in cases:
            sec = _event_seconds(dev, fn, reps)
            out.append({"kernel": name, "dtype": storage, "bytes": nbytes, "us": sec * 1e6,
                        "gbs": nbytes / sec / 1e9, "frac_hbm_peak": nbytes / sec / 1e9 / PEAK_HBM_GBS})
            print("# %-24s %s  %9.1f us  %7.0f GB/s (%.1f%% of HBM peak)"
                  % (name, storage, sec * 1e6, out[-1]["gbs"], 100 * out[-1]["frac_hbm_peak"]),
                  file=sys.stderr, flush=True)
        del x, y, g, g2, bias, gbias, xb, gxb, sbias, sx, sg, sgb, cases
        # moving and reducing along a dimension: a 4096 x 4096 matrix with a minibatch of 4
        # (64 Mi elements) and the softmax of a 10000-word vocabulary over a minibatch of 64
        r, bs = 4096, 4
        m = dev.new_tensor_by_constant(S([r, r], bs), 0.5)
        gm = dev.new_tensor_by_constant(S([r, r], bs), 0.0)
        whole = r * r * bs * item
        logits = dev.new_tensor_by_constant(S([10000], 64), 0.5)
        table = dev.new_tensor_by_constant(S([650, 10000]), 0.5)
        gtable = dev.new_tensor_by_constant(S([650, 10000]), 0.0)
        ids = [(7919 * i) % 10000 for i in range(64)]
        picked = dev.pick_fw(table, ids, 1)
        half = dev.slice_fw(m, 0, 0, r // 2)
        cases = [
            ("slice_fw_rows", lambda: dev.slice_fw(m, 0, 0, r // 2), whole),
            ("slice_bw_rows", lambda: dev.slice_bw(half, 0, 0, gm), whole // 2 * 3),
            ("concat_fw_cols", lambda: dev.concat_fw([half, half], 1), whole * 2),
            ("transpose_fw", lambda: dev.transpose_fw(m), 2 * whole),
            ("sum_fw_dim0", lambda: dev.reduce_fw("sum", m, 0), whole + whole // r),
            ("sum_fw_dim1", lambda: dev.reduce_fw("sum", m, 1), whole + whole // r),
            ("max_fw_dim1", lambda: dev.reduce_fw("max", m, 1), whole + whole // r),
            ("logsumexp_fw_vocab", lambda: dev.reduce_fw("logsumexp", logits, 0), (640000 + 64) * item),
            ("broadcast_fw_vocab", lambda: dev.broadcast_fw(dev.reduce_fw("sum", logits, 0), 0, 10000),
             (2 * 640000 + 128) * item),
            ("pick_fw_embedding", lambda: dev.pick_fw(table, ids, 1), 2 * 650 * 64 * item),
            ("pick_bw_embedding", lambda: dev.pick_bw(picked, ids, 1, gtable), 3 * 650 * 64 * item),
        ]
        for name, fn, nbytes in cases:
            sec = _event_seconds(dev, fn, reps)
            out.append({"kernel": name, "dtype": storage, "bytes": nbytes, "us": sec * 1e6,
                        "gbs": nbytes / sec / 1e9, "frac_hbm_peak": nbytes / sec / 1e9 / PEAK_HBM_GBS})
            print("# %-24s %s  %9.1f us  %7.0f GB/s (%.1f%% of HBM peak)"
                  % (name, storage, sec * 1e6, out[-1]["gbs"], 100 * out[-1]["frac_hbm_peak"]),
                  file=sys.stderr, flush=True)
        del m, gm, logits, table, gtable, picked, half, cases
        # random tensors (results written once) and copies between device objects on this GPU
        # (one read, one write; to the other storage width: converted on the way)
        n = 64 << 20
        other = pa.HIP16(0, storage="f16") if storage == "f32" else pa.HIP(0)
        other_item = 2 if storage == "f32" else 4
        src = dev.new_tensor_by_constant(S([n]), 0.5)
        cases = [
            ("random_uniform", lambda: dev.random_uniform(S([n]), -1.0, 1.0), n * item),
            ("random_normal", lambda: dev.random_normal(S([n]), 0.0, 1.0), n * item),
            ("random_bernoulli", lambda: dev.random_bernoulli(S([n]), 0.5), n * item),
            ("copy_tensor_same_storage", lambda: dev.copy_tensor(src), 2 * n * item),
            # to another device object: the call drains both streams itself, so the host clock times it
            ("copy_tensor_to_" + ("f16" if storage == "f32" else "f32"), lambda: other.copy_tensor(src),
             n * (item + other_item)),
        ]
        for name, fn, nbytes in cases:
            sec = (_wall_seconds if name.startswith("copy_tensor_to") else _event_seconds)(dev, fn, reps)
            out.append({"kernel": name, "dtype": storage, "bytes": nbytes, "us": sec * 1e6,
                        "gbs": nbytes / sec / 1e9, "frac_hbm_peak": nbytes / sec / 1e9 / PEAK_HBM_GBS})
            print("# %-24s %s  %9.1f us  %7.0f GB/s (%.1f%% of HBM peak)"
                  % (name, storage, sec * 1e6, out[-1]["gbs"], 100 * out[-1]["frac_hbm_peak"]),
                  file=sys.stderr, flush=True)
        del src, cases
        other.close()
        dev.close()
    return out


def measure_conv(reps=10):
    """conv2d (2 * outputs * taps flops forward, twice that backward, against the MFMA peak of the
    storage type) and max_pool2d (x read, y written; backward: x, y, gy read, gx read and written,
    against the HBM peak) on image-model layer shapes."""
    S = pa.Shape
    out = []
    layers = [  # name, x dims, w dims, minibatch, (pad0, pad1, str0, str1, dil0, dil1)
        ("vgg16_conv1_2", [224, 224, 64], [3, 3, 64, 64], 8, (1, 1, 1, 1, 1, 1)),
        ("vgg16_conv4_2", [28, 28, 512], [3, 3, 512, 512], 32, (1, 1, 1, 1, 1, 1)),
        ("pointwise_1x1", [56, 56, 256], [1, 1, 256, 64], 32, (0, 0, 1, 1, 1, 1)),
        ("mnist_conv1", [28, 28, 1], [5, 5, 1, 8], 200, (2, 2, 1, 1, 1, 1)),
    ]
    for storage, item in (("f32", 4), ("f16", 2)):
        dev = pa.HIP(0, rng_seed=1) if storage == "f32" else pa.HIP16(0, rng_seed=1, storage=storage)
        for name, xd, wd, bs, a in layers:
            x = dev.random_normal(S(xd, bs), 0.0, 1.0)
            w = dev.random_normal(S(wd), 0.0, 0.05)
            y = dev.conv2d_fw(x, w, *a)
            gx = dev.new_tensor_by_constant(x.shape(), 0.0)
            gw = dev.new_tensor_by_constant(w.shape(), 0.0)
            flops = 2.0 * y.shape().size() * wd[0] * wd[1] * wd[2]
            for tag, fn, work in (("fw", lambda: dev.conv2d_fw(x, w, *a), flops),
                                  ("bw", lambda: dev.conv2d_bw(x, w, y, y, *a, gx, gw), 2 * flops)):
                sec = _event_seconds(dev, fn, reps)
                out.append({"kernel": "conv2d_%s_%s" % (tag, name), "dtype": storage, "flops": work, "us": sec * 1e6,
                            "tflops": work / sec / 1e12, "frac_mfma_peak": work / sec / 1e12 / PEAK_TFLOPS[storage]})
                print("# %-28s %s  %9.1f us  %7.1f TFLOP/s (%.1f%% of MFMA peak)"
                      % (out[-1]["kernel"], storage, sec * 1e6, out[-1]["tflops"], 100 * out[-1]["frac_mfma_peak"]),
                      file=sys.stderr, flush=True)
            del x, w, y, gx, gw
        x = dev.random_normal(S([224, 224, 64], 8), 0.0, 1.0)
        a = (2, 2, 0, 0, 2, 2)
        y = dev.max_pool2d_fw(x, *a)
        gx = dev.new_tensor_by_constant(x.shape(), 0.0)
        nx, ny = x.shape().size() * item, y.shape().size() * item
        for tag, fn, nbytes in (("fw", lambda: dev.max_pool2d_fw(x, *a), nx + ny),
                                ("bw", lambda: dev.max_pool2d_bw(x, y, y, *a, gx), 3 * nx + 2 * ny)):
            sec = _event_seconds(dev, fn, reps)
            out.append({"kernel": "max_pool2d_%s_2x2" % tag, "dtype": storage, "bytes": nbytes, "us": sec * 1e6,
                        "gbs": nbytes / sec / 1e9, "frac_hbm_peak": nbytes / sec / 1e9 / PEAK_HBM_GBS})
            print("# %-28s %s  %9.1f us  %7.0f GB/s (%.1f%% of HBM peak)"
                  % (out[-1]["kernel"], storage, sec * 1e6, out[-1]["gbs"], 100 * out[-1]["frac_hbm_peak"]),
                  file=sys.stderr, flush=True)
        del x, y, gx
        dev.close()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="all",
                    help="all or one of: " + ", ".join(list(WORKLOADS) + ["half_storage_bf16"]))
    ap.add_argument("--skip-cpu", action="store_true", help="do not time the CPU oracle")
    ap.add_argument("--in-order", action="store_true",
                    help="every launch on one stream (phip_set_overlap off): per-kernel durations under a profiler")
    ap.add_argument("--deterministic", action="store_true",
                    help="gradients of split products added in a fixed order (phip_set_deterministic)")
    ap.add_argument("--traffic-calibration", action="store_true",
                    help="first run one streaming y += x over 64 Mi floats (reads 512 MiB, writes 256 MiB): "
                         "the known-size kernel that scales rocprofv3's FETCH_SIZE / WRITE_SIZE")
    ap.add_argument("--pointwise", action="store_true",
                    help="measure the elementwise kernels' streaming rates instead of the matmul workloads")
    ap.add_argument("--conv", action="store_true",
                    help="measure conv2d and max_pool2d on image-model layer shapes instead of the matmul workloads")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this backend has no multi-GPU path "
                 "(run with --gpus 1).")
    if args.pointwise:
        print(json.dumps({"metric": "elementwise kernels, algorithmic GB/s", "unit": "GB/s", "n_gpus": 1,
                          "peak": PEAK_HBM_GBS, "data": "synthetic", "kernels": measure_pointwise()}))
        return

    if args.conv:
        print(json.dumps({"metric": "conv2d TFLOP/s, max_pool2d algorithmic GB/s", "n_gpus": 1,
                          "data": "synthetic", "kernels": measure_conv()}))
        return

    if args.traffic_calibration:
        dev = pa.HIP(0)
        n = 64 << 20
        x, y = dev.new_tensor_by_constant([n], 1.0), dev.new_tensor_by_constant([n], 2.0)
        y += x
        dev.sync()
        del x, y
        dev.close()

    names = list(WORKLOADS) + ["half_storage_bf16"] if args.workload == "all" else [args.workload]
    if HEADLINE not in names and args.workload == "all":
        names.append(HEADLINE)
    results = {}
    for n in names:
        steps = args.steps if not n.startswith("half_storage") else max(1, min(args.steps, 5))
        # the CPU figure of the bf16 variant would repeat the fp16 one: same shapes, fp32 on the CPU
        results[n] = measure(n, steps, args.warmup, args.skip_cpu or n == "half_storage_bf16", args.deterministic, args.in_order)
        print("# %s: %.3f ms/step  %.2f TFLOP/s (%.1f%% of MFMA peak)  %.0f GB/s (%.1f%% of HBM peak)%s"
              % (n, results[n]["ms_per_step"], results[n]["tflops"], 100 * results[n]["frac_mfma_peak"],
                 results[n]["gbs"], 100 * results[n]["frac_hbm_peak"],
                 "  [%.3f ms/step with every launch on one stream]" % results[n]["ms_per_step_in_order"]
                 if "ms_per_step_in_order" in results[n] else ""), file=sys.stderr, flush=True)

    head = results.get(HEADLINE) or results[names[0]]
    w = WORKLOADS[head["workload"]]
    # Dominant kernel of the headline workload: the 128x128x32 fp32 MFMA GEMM
    # with global-to-LDS loads (three operand-layout instantiations, one launch
    # each per step, equal flops); its average launch duration is the event
    # time over the launches.
    launch_s = head["ms_per_step"] * 1e-3 / (3 * w.steps)
    flops_per_launch = w.flops_per_step() / 3
    roofline = {
        "bound": "mfma", "achieved": flops_per_launch / launch_s / 1e12, "peak": PEAK_TFLOPS[w.storage],
        "unit": "TFLOP/s", "frac": flops_per_launch / launch_s / 1e12 / PEAK_TFLOPS[w.storage],
        "traffic": HEADLINE_TRAFFIC_BYTES if head["workload"] == HEADLINE else None,
        "kernel": "gemm_f32_lds_kernel<A_KMAJOR,B_KMAJOR,false> (fw, ga, gb)",
        "flops_per_launch": flops_per_launch, "avg_launch_ms": launch_s * 1e3,
    }
    line = {
        "metric": "matmul fw+bw TFLOP/s", "value": head["tflops"], "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32" if w.storage == "f32" else w.storage, "data": "synthetic",
        "config": {"workload": "%s: a,b,gy {%d,%d}x%d fp32, fw + both gradients"
                   % (head["workload"], w.di, w.dj, w.bs),
                   "streams": "one (--in-order)" if args.in_order else
                              "library default: a second stream for runs of independent matmul calls of at most 4 GFLOP (%s)"
                              % ("this workload's products are larger and run in order" if w.flops_per_step() / 3 > 4e9
                                 else "this workload's calls use it"),
                   "tolerance": "max|x-ref|/max|ref| <= %.0e vs CPU oracle" % w.tolerance},
        "frac_of_mfma_peak": head["frac_mfma_peak"],
        "roofline": roofline,
        "cpu_baseline": head.get("cpu_baseline"),
        "workloads": results,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
