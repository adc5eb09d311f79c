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
import collections
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
STORAGE_CODE = {"f32": 0, "f16": 1, "bf16": 2}
# HBM bytes per step by rocprofv3's counters, from profiles/matmul_workloads_kernel_times_traffic_counters.txt
# section 2: per dispatch FETCH_SIZE x 2.0 KiB + WRITE_SIZE x 1.0 KiB (the factors read off a streaming
# y += x of known size in the same runs), summed over a step's launches ("HBM bytes per step by the
# counters" there).  Algorithmic bytes for comparison are Workload.bytes_per_step().
COUNTER_TRAFFIC_BYTES_PER_STEP = {
    "square_batched": 762.9e6,       # the three gemm_f32_lds_kernel launches: 206 + 284 + 272 MB: the three gemm_f32_lds_kernel launches
    "dense": 14.58e6,                # gemm_f32_tile16_kernel 7.06 + gemm_f32_pair_kernel 7.52 MB
    "rnn_gate": 872.4e6,             # 30 x (9.64 + 19.44 MB)
    "output_projection": 4469.8e6,   # 35 x (gemm_f32_slab_kernel 34.65 + gemm_f32_stream_pair_kernel 93.06 MB)
    "half_storage": 6293.6e6,        # two launches of 2.12 GB, one of 1.98 GB, 67 MB for the transposed copy of a
    "rnn_gate:f16": 487.4e6,         # 30 x (gemm_h16_skinny_kernel 4.83 + gemm_h16_skinny_pair_kernel 11.41 MB)
    "output_projection:f16": 3284.8e6,  # 35 x (30.46 + 36.68 + 26.71 MB: three gemm_h16_skinny_kernel launches)
}
# per launch of the headline kernel (average of its three operand-layout instantiations)
HEADLINE_TRAFFIC_BYTES = COUNTER_TRAFFIC_BYTES_PER_STEP["square_batched"] / 3
# Workloads whose products are small enough for the library's second lane (at most 4 GFLOP each): the
# step of record is taken with every launch on one stream, which is what a graph with other operations
# between its products sees; the figure with independent calls on two lanes is reported beside it.
PER_TIMESTEP = ("dense", "rnn_gate", "output_projection")

NATIVE_SRC = os.path.join(ROOT, "bench_native.cc")
NATIVE_LIB = os.path.join(ROOT, "libphip_bench.so")


def build_native():
    """Compiles the native timing loops (bench_native.cc, host code) against libphip.so."""
    import subprocess
    lib_dir = os.path.join(ROOT, "primitiv_amd")
    subprocess.check_call(["g++", "-O2", "-std=c++11", "-fPIC", "-shared", "-Wall", "-Wextra", NATIVE_SRC, "-o",
                           NATIVE_LIB, "-L" + lib_dir, "-lphip", "-Wl,-rpath,$ORIGIN/primitiv_amd"])
    return NATIVE_LIB


class Resident:
    """One workload with every input already on the device."""

    def __init__(self, dev, w, seed=0):
        self.dev, self.w = dev, w
        a, bs, gys = w.inputs(seed=seed)
        self.host = (a, bs, gys)
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
# "Sustains": the two MFMA-bound workloads are also timed over at least this long a run of back-to-back steps.
SUSTAINED_MIN_SECONDS = 1.0


class _Dims(ctypes.Structure):
    _fields_ = [(n, ctypes.c_uint32) for n in ("di", "dj", "dk", "ba", "bb")]


class _LstmDims(ctypes.Structure):
    _fields_ = [(n, ctypes.c_uint32) for n in ("in_size", "hidden", "batch", "timesteps")]


_bench_lib = None


def _native():
    """libphip_bench.so: the timing loops in native code (bench_native.cc)."""
    global _bench_lib
    if _bench_lib is None:
        _lib.lib()
        if not os.path.exists(NATIVE_LIB):
            raise _lib.Error("libphip_bench.so is not built; run `python __graft_entry__.py` or bench.build_native()")
        l = ctypes.CDLL(NATIVE_LIB)
        vp, pp, i = ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p), ctypes.c_int
        out = [ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_double)]
        # device pointers are 64-bit: without these ctypes would pass them as C ints
        l.phip_bench_raw_loop.argtypes = [vp, i, i, vp, vp, pp, pp, pp, pp, ctypes.POINTER(_Dims), i, i, i] + out
        l.phip_bench_front_loop.argtypes = [vp, i, vp, vp, pp, pp, ctypes.POINTER(_Dims), i, i, i] + out
        l.phip_bench_lstm_loop.argtypes = [vp, i, ctypes.POINTER(_LstmDims), vp, vp, vp, vp, pp, pp, vp, vp, i, i, i] + out
        l.phip_bench_raw_loop.restype = l.phip_bench_front_loop.restype = l.phip_bench_lstm_loop.restype = i
        l.phip_bench_last_enqueue_ms.restype = ctypes.c_double
        _bench_lib = l
    return _bench_lib


class Loops:
    """The native loops over one resident workload: raw (the two entry points on preallocated
    outputs) and front (what primitiv's Device front does around them per call: y from the pool,
    the per-timestep gradient from the pool and zero-filled, both handed back;
    primitiv/core/device.cc:20-24,268-301).  Each call returns milliseconds per step by the
    events on the library's stream and by the host clock."""

    def __init__(self, dev, res):
        self.dev, self.res, w = dev, res, res.w
        n = w.steps
        arr = lambda ptrs: (ctypes.c_void_p * n)(*ptrs)
        self.b, self.gy = arr([p[0] for p in res.ptrs]), arr([p[1] for p in res.ptrs])
        self.y, self.gb = arr([p[2] for p in res.ptrs]), arr([p[3] for p in res.ptrs])
        self.d = _Dims(w.di, w.dj, w.dk, w.ba, w.bb)
        self.n, self.code = n, STORAGE_CODE[w.storage]

    def raw(self, steps, warmup, which=0):
        """which: 0 = forward and backward calls, 1 = forward only, 2 = backward only."""
        ev, host = ctypes.c_float(), ctypes.c_double()
        r = self.res
        _lib.check(_native().phip_bench_raw_loop(self.dev.ctx(), self.code, which, r.a.handle(), r.ga.handle(), self.b, self.gy,
                                                 self.y, self.gb, ctypes.byref(self.d), self.n, steps, warmup,
                                                 ctypes.byref(ev), ctypes.byref(host)))
        return ev.value / steps, host.value / steps

    def front(self, steps, warmup):
        ev, host = ctypes.c_float(), ctypes.c_double()
        r = self.res
        _lib.check(_native().phip_bench_front_loop(self.dev.ctx(), self.code, r.a.handle(), r.ga.handle(), self.b,
                                                   self.gy, ctypes.byref(self.d), self.n, steps, warmup,
                                                   ctypes.byref(ev), ctypes.byref(host)))
        return ev.value / steps, host.value / steps

    def settle(self, warmup, which=0):
        """Untimed steps: the requested number and at least WARMUP_MIN_SECONDS.  Returns (steps, seconds)."""
        t0, done = time.perf_counter(), 0
        if warmup:
            self.raw(warmup, 0, which)
            done = warmup
        chunk = 8
        while time.perf_counter() - t0 < WARMUP_MIN_SECONDS:
            self.raw(chunk, 0, which)
            done += chunk
            chunk = min(2 * chunk, 1024)   # short calls: fewer trips through the interpreter
        return done, time.perf_counter() - t0


def time_python_loop(dev, res, steps):
    """Milliseconds per step (events, host clock) of the same calls issued by the interpreter."""
    ctx = dev.ctx()
    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    _lib.call("phip_event_create", ctx, ctypes.byref(e0))
    _lib.call("phip_event_create", ctx, ctypes.byref(e1))
    dev.sync()
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
    return ms.value / steps, host / steps * 1e3


def _rel(x, ref):
    return float(np.max(np.abs(np.asarray(x, dtype=np.float64) - ref)) / np.max(np.abs(ref)))


def cpu_baseline(w, res, threads=1):
    """The CPU leg.  Times the CPU oracle (a port of the reference's Eigen device, one thread, as the
    reference builds Eigen without OpenMP) on a bounded sample of the workload's own seeded inputs
    and scales to TFLOP/s; and uses the same oracle as the checker of this run's timed buffers:
    the forward result that the timed loop left on the device for timestep 0 (a strip of it for the
    large workloads) against the oracle's, by the workload's tolerance."""
    import oracle
    a, bs_, gys = res.host
    steps, bb, repeats, sample = w.steps, w.bb, 2, "full workload"
    b_list, gy_list = bs_, gys
    if w.name.startswith("half_storage"):
        bb, repeats, sample = 1, 1, "1 of the 8 minibatch samples (a shared), fp32"
        nb, ny = w.dj * w.dk, w.di * w.dk
        b_list, gy_list = [bs_[0][:nb]], [gys[0][:ny]]
    elif w.name == "square_batched":
        sample = "one fw+bw call, all 16 samples"
    elif w.name in ("dense",):
        repeats = 5
    bs = max(w.ba, bb)
    ga, gb = np.zeros_like(a), np.zeros_like(b_list[0])
    best = float("inf")
    for _ in range(repeats):
        t0 = time.perf_counter()
        for t in range(steps):
            oracle.matmul_fw(a, b_list[t], w.di, w.dj, w.dk, w.ba, bb, threads)
            oracle.matmul_bw(a, b_list[t], gy_list[t], ga, gb, w.di, w.dj, w.dk, w.ba, bb, threads)
        best = min(best, time.perf_counter() - t0)
    flops = 3 * 2 * w.di * w.dj * w.dk * bs * steps
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count()
    base = {"value": flops / best / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "host_cores_online": os.cpu_count(), "host_cores_usable": usable,
            "sample": "%s, seeded inputs of the workload, best of %d, %.2f s" % (sample, repeats, best)}
    # parity of the buffers this run timed
    if w.ba > 1:       # per-sample products: sample 0
        na, nb, ny = w.di * w.dj, w.dj * w.dk, w.di * w.dk
        want = oracle.matmul_fw(a[:na], bs_[0][:nb], w.di, w.dj, w.dk, 1, 1, threads)
        got = res.y[0].to_vector()[:ny]
        what = "y of sample 0"
    else:              # shared a: the first columns of y (all of it when small)
        cols = min(w.dk * w.bb, 64 if w.di * w.dj >= (1 << 24) else w.dk * w.bb)
        want = oracle.matmul_fw(a, bs_[0][:w.dj * cols], w.di, w.dj, cols, 1, 1, threads)
        got = res.y[0].to_vector()[:w.di * cols]
        what = "y of timestep 0" + ("" if cols == w.dk * w.bb else ", first %d columns" % cols)
    err = _rel(got, want)
    parity = {"checked": what, "max_abs_err_over_max_abs_ref": err, "tolerance": w.tolerance, "ok": bool(err <= w.tolerance)}
    return base, parity


def _workload(name):
    """A workload of the table; `<name>:<storage>` is the same workload (shapes, seeded inputs) with
    another storage type, e.g. half_storage:bf16, rnn_gate:f16.  Those are not among the reference's
    configurations and are reported next to them."""
    if name == "half_storage_bf16":
        name = "half_storage:bf16"
    if ":" in name:
        base, storage = name.split(":")
        w = copy.copy(WORKLOADS[base])
        w.name, w.storage = name, storage
        if storage != "f32":
            w.tolerance = 2e-2
        return w
    return WORKLOADS[name]


def _figures(w, per_step_s):
    tflops = w.flops_per_step() * w.steps / per_step_s / 1e12
    gbs = w.bytes_per_step() * w.steps / per_step_s / 1e9
    f_mfma, f_hbm = tflops / PEAK_TFLOPS[w.storage], gbs / PEAK_HBM_GBS
    return {"tflops": tflops, "frac_mfma_peak": f_mfma, "gbs": gbs, "frac_hbm_peak": f_hbm,
            "binding_roofline": "mfma" if f_mfma >= f_hbm else "hbm", "frac_binding_roofline": max(f_mfma, f_hbm)}


def measure(name, steps, warmup, skip_cpu, deterministic=False, in_order=False, sustained=False):
    w = _workload(name)
    base = name.split(":")[0]
    dev = pa.HIP(0) if w.storage == "f32" else pa.HIP16(0, storage=w.storage)
    dev.set_deterministic(deterministic)
    per_timestep = base in PER_TIMESTEP
    lanes_for_record = not in_order and not per_timestep
    dev.set_overlap(lanes_for_record)
    res = Resident(dev, w)
    loops = Loops(dev, res)
    dev.gemm_trace(True)
    loops.raw(1, 0)
    trace = dev.gemm_trace(False)      # every kernel that the step's matmul calls launched, helpers included
    kernels = trace[:8]
    warm_steps, warm_s = loops.settle(warmup)
    ms, host_ms = loops.raw(steps, 0)                       # the step of record: a C++ caller's loop
    out = {"workload": name, "dtype": w.storage, "calls_per_step": w.steps, "steps_timed": steps,
           "warmup_effective_steps": warm_steps, "warmup_effective_s": warm_s,
           "ms_per_step": ms, "ms_per_step_host_clock": host_ms,
           "streams": "one" if not lanes_for_record else "library default (two lanes for runs of independent products)",
           "gemm_kernels_first_timestep": kernels}
    launches = len(trace)
    out["kernel_launches_per_step"] = launches
    out["us_per_kernel_launch"] = ms * 1e3 / launches
    out.update(_figures(w, ms * 1e-3))
    out["ms_per_step_front"], out["ms_per_step_front_host_clock"] = loops.front(steps, 2)
    out["ms_per_step_python_loop"], out["ms_per_step_python_loop_host_clock"] = time_python_loop(dev, res, steps)
    if per_timestep or w.flops_per_step() / 3 <= 4e9:
        # the same loops the other way: both lanes (when the record is in order) or one stream
        dev.set_overlap(not lanes_for_record)
        loops.raw(max(2, warmup), 0)
        other, _ = loops.raw(steps, 0)
        other_front, _ = loops.front(steps, 2)
        dev.set_overlap(lanes_for_record)
        two, one = (other, ms) if not lanes_for_record else (ms, other)
        two_front, one_front = (other_front, out["ms_per_step_front"]) if not lanes_for_record else (out["ms_per_step_front"], other_front)
        out["ms_per_step_in_order"], out["ms_per_step_front_in_order"] = one, one_front
        out["frac_binding_roofline_in_order"] = _figures(w, one * 1e-3)["frac_binding_roofline"]
        out["ms_per_step_two_lanes"], out["ms_per_step_front_two_lanes"] = two, two_front
        out["frac_binding_roofline_two_lanes"] = _figures(w, two * 1e-3)["frac_binding_roofline"]
    if per_timestep and w.storage == "f32" and not deterministic:
        dev.set_deterministic(True)
        loops.raw(max(2, warmup), 0)
        out["ms_per_step_deterministic"], _ = loops.raw(steps, 0)
        dev.set_deterministic(False)
    if sustained:
        n = max(steps, int(SUSTAINED_MIN_SECONDS / (ms * 1e-3)) + 1)
        s_ms, _ = loops.raw(n, 0)
        fig = _figures(w, s_ms * 1e-3)
        out["sustained"] = {"steps": n, "seconds": s_ms * 1e-3 * n, "ms_per_step": s_ms, "tflops": fig["tflops"],
                            "frac_mfma_peak": fig["frac_mfma_peak"]}
    # HBM traffic per step by the counters (profiles/), next to the algorithmic bytes above
    if name in COUNTER_TRAFFIC_BYTES_PER_STEP:
        traffic = COUNTER_TRAFFIC_BYTES_PER_STEP[name]
        out["counter_traffic_bytes_per_step"] = traffic
        out["counter_gbs"] = traffic / (ms * 1e-3) / 1e9
        out["counter_frac_hbm_peak"] = traffic / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS
    if not skip_cpu:
        out["cpu_baseline"], out["parity_in_run"] = cpu_baseline(w, res)
    del loops, res
    dev.close()
    return out


def _event_seconds(dev, fn, reps, warm=2):
    """Average seconds of one fn() over `reps` back-to-back calls, by events on the library's stream."""
    ctx = dev.ctx()
    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    _lib.call("phip_event_create", ctx, ctypes.byref(e0))
    _lib.call("phip_event_create", ctx, ctypes.byref(e1))
    for _ in range(warm):
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


def _wall_seconds(dev, fn, reps, warm=2):
    """Average seconds of one blocking fn() (a call that waits for the device itself) by the host clock."""
    for _ in range(warm):
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
    recurrent-layer shape (2048 x 64) shows the latency floor.
    The large cases walk round several sets of operands, so that no call finds its operands in the 256 MB
    Infinity Cache from the call before: repeated over ONE set, a copy of 256 MiB reads 5.4 TB/s, the same copy
    with streaming stores 8.6 TB/s (the source then stays in the cache between calls), and one of 1 GiB 5.1
    either way - the rate of HBM is what the rotation shows.  Results rotate too: each case keeps its last
    SETS results alive, so the memory pool hands a call the block of the oldest one and not the block the
    call before has just written (a 128 MiB result written over and over stays in that cache: the 16-bit
    transpose then reads 6.2 TB/s, with results of 256 MiB and more 5.2)."""
    S = pa.Shape
    out = []
    SETS = 4

    def kept(fn):
        """fn, with its last SETS results held."""
        held = collections.deque(maxlen=SETS)
        return lambda: held.append(fn())

    class Ring:
        """SETS tensors of one shape, handed out in turn."""
        def __init__(self, make):
            self.t, self.i = [make() for _ in range(SETS)], 0

        def __call__(self):
            self.i = (self.i + 1) % SETS
            return self.t[self.i]

    for storage, item in (("f32", 4), ("f16", 2)):
        dev = pa.HIP(0) if storage == "f32" else pa.HIP16(0, storage=storage)
        n = 64 << 20
        xs = Ring(lambda: dev.new_tensor_by_constant(S([n]), 0.5))
        ys = Ring(lambda: dev.new_tensor_by_constant(S([n]), 0.25))
        gs = Ring(lambda: dev.new_tensor_by_constant(S([n]), 0.0))
        g2s = Ring(lambda: dev.new_tensor_by_constant(S([n]), 0.0))
        vol, bs = 1 << 20, 64
        bias = dev.new_tensor_by_constant(S([vol]), 0.5)
        gbias = dev.new_tensor_by_constant(S([vol]), 0.0)
        xbs = Ring(lambda: dev.new_tensor_by_constant(S([vol], bs), 0.5))
        gxbs = Ring(lambda: dev.new_tensor_by_constant(S([vol], bs), 0.0))
        sv, sb = 2048, 64
        sbias = dev.new_tensor_by_constant(S([sv]), 0.5)
        sx = dev.new_tensor_by_constant(S([sv], sb), 0.5)
        sg = dev.new_tensor_by_constant(S([sv], sb), 0.0)
        sgb = dev.new_tensor_by_constant(S([sv]), 0.0)
        big, med = n * item, vol * bs * item
        cases = [
            ("tanh_fw", lambda: dev.unary_fw("tanh", xs()), 2 * big),
            ("tanh_bw", lambda: (lambda x: dev.unary_bw("tanh", x, ys(), x, gs()))(xs()), 4 * big),
            ("prelu_fw", lambda: dev.const_fw("prelu", xs(), 0.01), 2 * big),
            ("add_fw", lambda: dev.binary_fw("add", xs(), ys()), 3 * big),
            ("multiply_bw", lambda: (lambda x, y: dev.binary_bw("multiply", x, y, x, y, gs(), g2s()))(xs(), ys()), 7 * big),
            ("bias_add_fw", lambda: dev.binary_fw("add", xbs(), bias), 2 * med + vol * item),
            ("bias_add_bw", lambda: (lambda xb: dev.binary_bw("add", xb, bias, xb, xb, gxbs(), gbias))(xbs()),
             3 * med + 2 * vol * item),
            ("inplace_add", lambda: dev.inplace_add(xs(), ys()), 3 * big),
            ("inplace_multiply_const", lambda: dev.inplace_multiply_const(1.0, ys()), 2 * big),
            ("bias_add_fw_2048x64", lambda: dev.binary_fw("add", sx, sbias), (2 * sv * sb + sv) * item),
            ("bias_add_bw_2048x64", lambda: dev.binary_bw("add", sx, sbias, sx, sx, sg, sgb),
             (3 * sv * sb + 2 * sv) * item),
        ]
        for name, fn, nbytes in cases:
            sec = _event_seconds(dev, kept(fn), reps, warm=SETS + 2)
            out.append({"kernel": name, "dtype": storage, "bytes": nbytes, "us": sec * 1e6,
                        "gbs": nbytes / sec / 1e9, "frac_hbm_peak": nbytes / sec / 1e9 / PEAK_HBM_GBS})
            print("# %-24s %s  %9.1f us  %7.0f GB/s (%.1f%% of HBM peak)"
                  % (name, storage, sec * 1e6, out[-1]["gbs"], 100 * out[-1]["frac_hbm_peak"]),
                  file=sys.stderr, flush=True)
        del xs, ys, gs, g2s, bias, gbias, xbs, gxbs, sbias, sx, sg, sgb, cases
        # moving and reducing along a dimension: a 4096 x 4096 matrix with a minibatch of 4
        # (64 Mi elements) and the softmax of a 10000-word vocabulary over a minibatch of 64
        r, bs = 4096, 4
        ms = Ring(lambda: dev.new_tensor_by_constant(S([r, r], bs), 0.5))
        gms = Ring(lambda: dev.new_tensor_by_constant(S([r, r], bs), 0.0))
        whole = r * r * bs * item
        logits = dev.new_tensor_by_constant(S([10000], 64), 0.5)
        table = dev.new_tensor_by_constant(S([650, 10000]), 0.5)
        gtable = dev.new_tensor_by_constant(S([650, 10000]), 0.0)
        ids = [(7919 * i) % 10000 for i in range(64)]
        picked = dev.pick_fw(table, ids, 1)
        halves = Ring(lambda: dev.slice_fw(ms(), 0, 0, r // 2))
        cases = [
            ("slice_fw_rows", lambda: dev.slice_fw(ms(), 0, 0, r // 2), whole),
            ("slice_bw_rows", lambda: dev.slice_bw(halves(), 0, 0, gms()), whole // 2 * 3),
            ("concat_fw_cols", lambda: dev.concat_fw([halves(), halves()], 1), whole * 2),
            ("transpose_fw", lambda: dev.transpose_fw(ms()), 2 * whole),
            ("sum_fw_dim0", lambda: dev.reduce_fw("sum", ms(), 0), whole + whole // r),
            ("sum_fw_dim1", lambda: dev.reduce_fw("sum", ms(), 1), whole + whole // r),
            ("max_fw_dim1", lambda: dev.reduce_fw("max", ms(), 1), whole + whole // r),
            ("logsumexp_fw_vocab", lambda: dev.reduce_fw("logsumexp", logits, 0), (640000 + 64) * item),
            ("broadcast_fw_vocab", lambda: dev.broadcast_fw(dev.reduce_fw("sum", logits, 0), 0, 10000),
             (2 * 640000 + 128) * item),
            ("pick_fw_embedding", lambda: dev.pick_fw(table, ids, 1), 2 * 650 * 64 * item),
            ("pick_bw_embedding", lambda: dev.pick_bw(picked, ids, 1, gtable), 3 * 650 * 64 * item),
        ]
        for name, fn, nbytes in cases:
            sec = _event_seconds(dev, kept(fn), reps, warm=SETS + 2)
            out.append({"kernel": name, "dtype": storage, "bytes": nbytes, "us": sec * 1e6,
                        "gbs": nbytes / sec / 1e9, "frac_hbm_peak": nbytes / sec / 1e9 / PEAK_HBM_GBS})
            print("# %-24s %s  %9.1f us  %7.0f GB/s (%.1f%% of HBM peak)"
                  % (name, storage, sec * 1e6, out[-1]["gbs"], 100 * out[-1]["frac_hbm_peak"]),
                  file=sys.stderr, flush=True)
        del ms, gms, logits, table, gtable, picked, halves, cases
        # random tensors (results written once) and copies between device objects on this GPU
        # (one read, one write; to the other storage width: converted on the way)
        n = 64 << 20
        other = pa.HIP16(0, storage="f16") if storage == "f32" else pa.HIP(0)
        other_item = 2 if storage == "f32" else 4
        srcs = Ring(lambda: dev.new_tensor_by_constant(S([n]), 0.5))
        cases = [
            ("random_uniform", lambda: dev.random_uniform(S([n]), -1.0, 1.0), n * item),
            ("random_normal", lambda: dev.random_normal(S([n]), 0.0, 1.0), n * item),
            ("random_bernoulli", lambda: dev.random_bernoulli(S([n]), 0.5), n * item),
            ("copy_tensor_same_storage", lambda: dev.copy_tensor(srcs()), 2 * n * item),
            # to another device object: the call drains both streams itself, so the host clock times it
            ("copy_tensor_to_" + ("f16" if storage == "f32" else "f32"), lambda: other.copy_tensor(srcs()),
             n * (item + other_item)),
        ]
        for name, fn, nbytes in cases:
            sec = (_wall_seconds if name.startswith("copy_tensor_to") else _event_seconds)(dev, kept(fn), reps, warm=SETS + 2)
            out.append({"kernel": name, "dtype": storage, "bytes": nbytes, "us": sec * 1e6,
                        "gbs": nbytes / sec / 1e9, "frac_hbm_peak": nbytes / sec / 1e9 / PEAK_HBM_GBS})
            print("# %-24s %s  %9.1f us  %7.0f GB/s (%.1f%% of HBM peak)"
                  % (name, storage, sec * 1e6, out[-1]["gbs"], 100 * out[-1]["frac_hbm_peak"]),
                  file=sys.stderr, flush=True)
        del srcs, cases
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


def _timed_native(fn, steps, warmup):
    ev, host = ctypes.c_float(), ctypes.c_double()
    _lib.check(fn(steps, warmup, ctypes.byref(ev), ctypes.byref(host)))
    return ev.value / steps, host.value / steps


# Device calls of one LSTM timestep as primitiv's graph issues them (bench_native.cc: phip_bench_lstm_loop).
LSTM_CALLS_FORWARD = 17      # 2 strided copies (concat), matmul, bias add, 4 slices, 4 activations, 5 elementwise
LSTM_CALLS_BACKWARD = 40     # 17 zero fills, 10 elementwise gradients, 4 + 2 strided copies, matmul_bw, 3 in-place adds ... per timestep


def measure_lstm(storage, steps, warmup, hidden=650, batch=64, timesteps=35):
    """One LSTM layer of the reference's language model (examples/ptb/ptb_rnnlm_lstm.cc:69-112:
    W {4*hidden, 2*hidden}, minibatch 64, 35 timesteps unrolled), forward through the timesteps and
    backward through time, every device call as primitiv's Graph would make it (zero-filled gradients
    included).  A step is the whole sequence; reported per timestep, in order and with the library's
    default (which engages its second lane only in runs of matmul calls, so here it should not differ)."""
    from primitiv_amd.configs import Randomizer
    S = pa.Shape
    dev = pa.HIP(0) if storage == "f32" else pa.HIP16(0, storage=storage)
    rng = Randomizer(0)
    H, I, B, T = hidden, hidden, batch, timesteps
    W = dev.new_tensor_by_vector(S([4 * H, I + H]), rng.uniform(-0.1, 0.1, 4 * H * (I + H)))
    b = dev.new_tensor_by_vector(S([4 * H]), rng.uniform(-0.1, 0.1, 4 * H))
    xs = [dev.new_tensor_by_vector(S([I], B), rng.uniform(-0.1, 0.1, I * B)) for _ in range(T)]
    gys = [dev.new_tensor_by_vector(S([H], B), rng.normal(0.0, 1e-2, H * B)) for _ in range(T)]
    gW = dev.new_tensor_by_constant(W.shape(), 0)
    gb = dev.new_tensor_by_constant(b.shape(), 0)
    arr = lambda ts: (ctypes.c_void_p * T)(*[t.handle() for t in ts])
    px, pgy = arr(xs), arr(gys)
    d = _LstmDims(I, H, B, T)
    L, code = _native(), STORAGE_CODE[storage]

    def loop(forward_only):
        return lambda n, wu, ev, host: L.phip_bench_lstm_loop(dev.ctx(), code, ctypes.byref(d), W.handle(), b.handle(),
                                                              gW.handle(), gb.handle(), px, pgy, None, None,
                                                              int(forward_only), n, wu, ev, host)

    out = {"layer": "LSTM %d -> %d, minibatch %d, %d timesteps, W {%d,%d}" % (I, H, B, T, 4 * H, I + H), "dtype": storage,
           "device_calls_per_timestep": {"forward": LSTM_CALLS_FORWARD, "backward": LSTM_CALLS_BACKWARD},
           "steps_timed": steps}
    for key, overlap in (("in_order", False), ("library_default", True)):
        dev.set_overlap(overlap)
        _timed_native(loop(False), max(2, warmup), 0)
        fw_ms, fw_host = _timed_native(loop(True), steps, 1)
        all_ms, all_host = _timed_native(loop(False), steps, 1)
        enqueue = L.phip_bench_last_enqueue_ms() / steps
        out[key] = {"us_per_timestep_forward": fw_ms * 1e3 / T, "us_per_timestep_forward_backward": all_ms * 1e3 / T,
                    "us_per_timestep_forward_backward_host_enqueue_only": enqueue * 1e3 / T,
                    "us_per_timestep_forward_backward_host_clock": all_host * 1e3 / T,
                    "us_per_timestep_forward_host_clock": fw_host * 1e3 / T}
    flops = 3 * 2 * (4 * H) * (I + H) * B
    t = out["in_order"]["us_per_timestep_forward_backward"] * 1e-6
    out["matmul_tflops_of_the_timestep"] = flops / t / 1e12
    out["us_per_device_call"] = out["in_order"]["us_per_timestep_forward_backward"] / (LSTM_CALLS_FORWARD + LSTM_CALLS_BACKWARD)
    dev.gemm_trace(True)
    _timed_native(loop(False), 1, 0)
    names = dev.gemm_trace(False)
    out["gemm_kernels"] = sorted(set(names))
    del W, b, xs, gys, gW, gb
    dev.close()
    return out


SWEEP_SQUARES = [256, 384, 512, 768, 1024, 1536, 2048, 3072, 4096]
# layers of the reference's examples: (name, di, dj, minibatch)
SWEEP_LAYERS = [
    ("mnist_hidden", 800, 784, 200),        # examples/mnist/mnist.cc:58-80
    ("mnist_output", 10, 800, 200),
    ("ptb_lstm_b20", 2600, 1300, 20),       # examples/ptb/ptb_rnnlm_lstm.cc:86-101, minibatch 20
    ("ptb_lstm_b64", 2600, 1300, 64),
    ("ptb_projection_b20", 10000, 650, 20),  # :125
]


def measure_sweep(reps=20):
    """Shape sweep, every launch on one stream: unbatched squares M = N = K and the reference examples' layers
    (a shared, minibatch folded into columns), forward and backward timed apart, fp32 and fp16 storage, with
    the kernels each went to.  Neighbouring squares whose efficiency differs by more than 1.5x are flagged."""
    from primitiv_amd.configs import Workload
    rows = []
    for storage in ("f32", "f16"):
        dev = pa.HIP(0) if storage == "f32" else pa.HIP16(0, storage=storage)
        dev.set_overlap(False)
        cases = [("square_%d" % n, n, n, n, 1, 1) for n in SWEEP_SQUARES]
        cases += [(name, di, dj, 1, 1, bs) for name, di, dj, bs in SWEEP_LAYERS]
        prev = None
        for name, di, dj, dk, ba, bb in cases:
            dist = ("normal", 0.0, 1.0)
            w = Workload(name, di, dj, dk, ba, bb, 1, ("uniform", -0.1, 0.1), dist, dist, storage=storage)
            res = Resident(dev, w)
            loops = Loops(dev, res)
            row = {"shape": name, "dtype": storage, "di": di, "dj": dj, "dk": dk * bb}
            third = w.flops_per_step() / 3
            for which, key, flops in ((1, "fw", third), (2, "bw", 2 * third)):
                dev.gemm_trace(True)
                loops.raw(1, 0, which)
                row[key + "_kernels"] = "+".join(dev.gemm_trace(False))
                n = max(3, min(reps, int(0.05 / max(1e-6, flops / 50e12))))
                # the clocks settle only under tens of milliseconds of load (1536^3 forward reads 78 us
                # behind 20 calls and 68 us behind 200): every figure is taken behind at least 60 ms of it
                loops.settle(n, which)
                ms, _ = loops.raw(n, 0, which)
                row[key + "_us"] = ms * 1e3
                row[key + "_tflops"] = flops / (ms * 1e-3) / 1e12
                row[key + "_frac_mfma_peak"] = row[key + "_tflops"] / PEAK_TFLOPS[storage]
            if name.startswith("square") and prev is not None:
                for key in ("fw", "bw"):
                    r = row[key + "_frac_mfma_peak"] / prev[key + "_frac_mfma_peak"]
                    if r > 1.5 or r < 1 / 1.5:
                        row.setdefault("cliff", []).append("%s x%.2f vs %s" % (key, r, prev["shape"]))
            prev = row if name.startswith("square") else None
            rows.append(row)
            print("# %-20s %s  fw %8.1f us %7.1f TF (%4.1f%%) %-22s  bw %8.1f us %7.1f TF (%4.1f%%) %-30s %s"
                  % (name, storage, row["fw_us"], row["fw_tflops"], 100 * row["fw_frac_mfma_peak"], row["fw_kernels"],
                     row["bw_us"], row["bw_tflops"], 100 * row["bw_frac_mfma_peak"], row["bw_kernels"],
                     " ".join(row.get("cliff", []))), file=sys.stderr, flush=True)
            del loops, res
        dev.close()
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="all",
                    help="all or one of: " + ", ".join(list(WORKLOADS)) + "; name:storage runs a workload with "
                         "another storage type (half_storage:bf16, rnn_gate:f16, ...)")
    ap.add_argument("--skip-cpu", action="store_true", help="do not time the CPU oracle (nor check against it)")
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
    ap.add_argument("--lstm", action="store_true",
                    help="one LSTM layer of the reference's language model, forward and backward through time, "
                         "device call by device call")
    ap.add_argument("--storage", default="all", help="with --lstm: f32, f16, bf16 or all")
    ap.add_argument("--sweep", action="store_true",
                    help="shape sweep (unbatched squares, the reference examples' layers), fp32 and fp16, with kernel names")
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

    if args.lstm:
        layers = [measure_lstm(st, max(2, min(args.steps, 10)), args.warmup) for st in (("f32", "f16", "bf16") if args.storage == "all" else (args.storage,))]
        for l in layers:
            print("# lstm %s: %.1f us / timestep forward + backward in order (%.1f forward), %.1f library default; "
                  "%.2f us per device call" % (l["dtype"], l["in_order"]["us_per_timestep_forward_backward"],
                                                l["in_order"]["us_per_timestep_forward"],
                                                l["library_default"]["us_per_timestep_forward_backward"],
                                                l["us_per_device_call"]), file=sys.stderr, flush=True)
        print(json.dumps({"metric": "LSTM layer, microseconds per timestep (forward + backward through time)",
                          "unit": "us", "n_gpus": 1, "data": "synthetic", "higher_is_better": False, "layers": layers}))
        return

    if args.sweep:
        print(json.dumps({"metric": "matmul shape sweep, TFLOP/s and fraction of the MFMA peak", "n_gpus": 1,
                          "data": "synthetic", "peaks_tflops": PEAK_TFLOPS, "rows": measure_sweep()}))
        return

    if args.traffic_calibration:
        dev = pa.HIP(0)
        n = 64 << 20
        x, y = dev.new_tensor_by_constant([n], 1.0), dev.new_tensor_by_constant([n], 2.0)
        y += x
        dev.sync()
        del x, y
        dev.close()

    # the reference's five configurations, then the same shapes with other storage types (reported extras)
    extras = ["half_storage:bf16", "rnn_gate:f16", "rnn_gate:bf16", "output_projection:f16", "output_projection:bf16"]
    names = list(WORKLOADS) + extras if args.workload == "all" else [args.workload]
    results = {}
    for n in names:
        steps = args.steps if not n.startswith("half_storage") else max(1, min(args.steps, 5))
        # the CPU figure of a storage variant would repeat its fp32 / fp16 one: same shapes, fp32 on the CPU
        base = n.split(":")[0]
        results[n] = measure(n, steps, args.warmup, args.skip_cpu or (":" in n and base != "half_storage"),
                             args.deterministic, args.in_order, sustained=base in (HEADLINE, "half_storage"))
        r = results[n]
        print("# %s: %.3f ms/step  %.2f TFLOP/s (%.1f%% of MFMA peak)  %.0f GB/s (%.1f%% of HBM peak)  [%s]%s%s"
              % (n, r["ms_per_step"], r["tflops"], 100 * r["frac_mfma_peak"], r["gbs"], 100 * r["frac_hbm_peak"],
                 "+".join(r["gemm_kernels_first_timestep"]),
                 "  [%.3f ms/step on two lanes]" % r["ms_per_step_two_lanes"] if "ms_per_step_two_lanes" in r else "",
                 "  [sustained %.1f s: %.2f TFLOP/s]" % (r["sustained"]["seconds"], r["sustained"]["tflops"])
                 if "sustained" in r else ""), file=sys.stderr, flush=True)

    head = results.get(HEADLINE) or results[names[0]]
    w = _workload(head["workload"])
    # Dominant kernel of the headline workload: the 128x128x32 fp32 MFMA GEMM
    # with global-to-LDS loads (three operand-layout instantiations, one launch
    # each per step, equal flops); its average launch duration is the event
    # time over the launches.
    launch_s = head["ms_per_step"] * 1e-3 / head["kernel_launches_per_step"]
    flops_per_launch = w.flops_per_step() * w.steps / head["kernel_launches_per_step"]
    roofline = {
        "bound": "mfma", "achieved": flops_per_launch / launch_s / 1e12, "peak": PEAK_TFLOPS[w.storage],
        "unit": "TFLOP/s", "frac": flops_per_launch / launch_s / 1e12 / PEAK_TFLOPS[w.storage],
        "traffic": HEADLINE_TRAFFIC_BYTES if head["workload"] == HEADLINE else None,
        "kernel": "gemm_f32_lds_kernel<A_KMAJOR,B_KMAJOR,0> (fw, ga, gb)" if head["workload"] == HEADLINE
                  else "+".join(head["gemm_kernels_first_timestep"]),
        "flops_per_launch": flops_per_launch, "avg_launch_ms": launch_s * 1e3,
    }
    line = {
        "metric": "matmul fw+bw TFLOP/s", "value": head["tflops"], "unit": "TFLOP/s",
        "n_gpus": 1, "steps": head["steps_timed"], "warmup": args.warmup,
        "warmup_effective_steps": head["warmup_effective_steps"], "warmup_effective_s": head["warmup_effective_s"],
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": w.storage, "data": "synthetic",
        "config": {"workload": "%s: a,b,gy {%d,%d}x%d %s, fw + both gradients"
                   % (head["workload"], w.di, w.dj, w.bs, w.storage),
                   "streams": head["streams"],
                   "tolerance": "max|x-ref|/max|ref| <= %.0e vs CPU oracle" % w.tolerance},
        "frac_of_mfma_peak": head["frac_mfma_peak"],
        "sustained": head.get("sustained"),
        "parity_in_run": head.get("parity_in_run"),
        "roofline": roofline,
        "cpu_baseline": head.get("cpu_baseline"),
        "workloads": results,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
