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
# HBM bytes per launch of the headline kernel (average of its three operand-layout
# instantiations): rocprofv3 FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0, the factors read
# off a streaming y += x of known size (the summary under profiles/ holds both runs).
HEADLINE_TRAFFIC_BYTES = 195.9e6 + 67.1e6


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


def time_gpu(dev, res, steps, warmup):
    """(host seconds, event seconds) for `steps` steps."""
    ctx = dev.ctx()
    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    _lib.call("phip_event_create", ctx, ctypes.byref(e0))
    _lib.call("phip_event_create", ctx, ctypes.byref(e1))
    for _ in range(warmup):
        res.step()
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
    return host, ms.value * 1e-3


def cpu_baseline(w, threads=1):
    """Times the CPU oracle (a port of the reference's Eigen device, one
    thread, as the reference builds Eigen without OpenMP) on a bounded sample
    of the workload and scales to TFLOP/s."""
    import oracle
    steps, bb, repeats, sample = w.steps, w.bb, 2, "full workload"
    if w.name == "half_storage":
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
    return {"value": flops / best / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": "%s, best of %d, %.2f s" % (sample, repeats, best)}


def measure(name, steps, warmup, skip_cpu):
    w = WORKLOADS[name]
    dev = pa.HIP(0) if w.storage == "f32" else pa.HIP16(0, storage=w.storage)
    res = Resident(dev, w)
    host_s, ev_s = time_gpu(dev, res, steps, warmup)
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
    if not skip_cpu:
        out["cpu_baseline"] = cpu_baseline(w)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="all", help="all or one of: " + ", ".join(WORKLOADS))
    ap.add_argument("--skip-cpu", action="store_true", help="do not time the CPU oracle")
    ap.add_argument("--traffic-calibration", action="store_true",
                    help="first run one streaming y += x over 64 Mi floats (reads 512 MiB, writes 256 MiB): "
                         "the known-size kernel that scales rocprofv3's FETCH_SIZE / WRITE_SIZE")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this backend has no multi-GPU path "
                 "(run with --gpus 1).")

    if args.traffic_calibration:
        dev = pa.HIP(0)
        n = 64 << 20
        x, y = dev.new_tensor_by_constant([n], 1.0), dev.new_tensor_by_constant([n], 2.0)
        y += x
        dev.sync()
        del x, y
        dev.close()

    names = list(WORKLOADS) if args.workload == "all" else [args.workload]
    if HEADLINE not in names and args.workload == "all":
        names.append(HEADLINE)
    results = {}
    for n in names:
        steps = args.steps if n != "half_storage" else max(1, min(args.steps, 5))
        results[n] = measure(n, steps, args.warmup, args.skip_cpu)
        print("# %s: %.3f ms/step  %.2f TFLOP/s (%.1f%% of MFMA peak)  %.0f GB/s (%.1f%% of HBM peak)"
              % (n, results[n]["ms_per_step"], results[n]["tflops"], 100 * results[n]["frac_mfma_peak"],
                 results[n]["gbs"], 100 * results[n]["frac_hbm_peak"]), file=sys.stderr, flush=True)

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
        "kernel": "gemm_f32_lds_kernel<A_KMAJOR,B_KMAJOR> (fw, ga, gb)",
        "flops_per_launch": flops_per_launch, "avg_launch_ms": launch_s * 1e3,
    }
    line = {
        "metric": "matmul fw+bw TFLOP/s", "value": head["tflops"], "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32" if w.storage == "f32" else w.storage, "data": "synthetic",
        "config": {"workload": "%s: a,b,gy {%d,%d}x%d fp32, fw + both gradients"
                   % (head["workload"], w.di, w.dj, w.bs),
                   "tolerance": "max|x-ref|/max|ref| <= %.0e vs CPU oracle" % w.tolerance},
        "frac_of_mfma_peak": head["frac_mfma_peak"],
        "roofline": roofline,
        "cpu_baseline": head.get("cpu_baseline"),
        "workloads": results,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
