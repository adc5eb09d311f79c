"""The LSTM layer that bench.py --lstm times (bench_native.cc: phip_bench_lstm_loop, the layer of the
reference's examples/ptb/ptb_rnnlm_lstm.cc:69-112 unrolled device call by device call, forward and
backward through time) against the same recurrence and its derivative in float64 numpy."""
import ctypes
import os
import sys

import numpy as np
import pytest

import primitiv_amd as pa
from primitiv_amd import _lib
from util import norm_rel_err

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import bench  # noqa: E402

pytestmark = pytest.mark.gpu

S = pa.Shape


def _lstm_float64(W, b, xs, gys):
    """W [4H x (I+H)], b [4H], xs / gys lists of [B x I] / [B x H]; returns h_T, gW, gb, gx_0."""
    sig = lambda v: 1 / (1 + np.exp(-v))
    H = W.shape[0] // 4
    B = xs[0].shape[0]
    h, c = np.zeros((B, H)), np.zeros((B, H))
    tape = []
    for x in xs:
        xh = np.concatenate([x, h], axis=1)
        u = xh @ W.T + b
        i, f, o, j = sig(u[:, :H]), sig(u[:, H:2 * H]), sig(u[:, 2 * H:3 * H]), np.tanh(u[:, 3 * H:])
        c_new = i * j + f * c
        tc = np.tanh(c_new)
        h = o * tc
        tape.append((xh, i, f, o, j, c, tc))
        c = c_new
    gW, gb = np.zeros_like(W), np.zeros_like(b)
    gh, gc = gys[-1].copy(), np.zeros((B, H))
    gx0 = None
    for t in range(len(xs) - 1, -1, -1):
        xh, i, f, o, j, c_prev, tc = tape[t]
        go, gtc = gh * tc, gh * o
        gc = gc + gtc * (1 - tc * tc)
        gi, gj, gf, gc_prev = gc * j, gc * i, gc * c_prev, gc * f
        gu = np.concatenate([gi * i * (1 - i), gf * f * (1 - f), go * o * (1 - o), gj * (1 - j * j)], axis=1)
        gW += gu.T @ xh
        gb += gu.sum(axis=0)
        gxh = gu @ W
        I = xh.shape[1] - H
        gx0 = gxh[:, :I]
        gh = gxh[:, I:] + (gys[t - 1] if t > 0 else 0)
        gc = gc_prev
    return h, gW, gb, gx0


@pytest.mark.parametrize("storage", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("I,H,B,T", [(16, 24, 5, 4), (650, 650, 8, 3)])
def test_lstm_layer_forward_and_backward_through_time(storage, I, H, B, T):
    rng = np.random.default_rng(3)
    W = rng.uniform(-0.3, 0.3, (4 * H, I + H)) / np.sqrt((I + H) / 40)
    b = rng.uniform(-0.1, 0.1, 4 * H)
    xs = [rng.standard_normal((B, I)) for _ in range(T)]
    gys = [rng.standard_normal((B, H)) * 0.1 for _ in range(T)]
    f32 = lambda m: np.asarray(m, dtype=np.float32)
    dev = pa.HIP(0) if storage == "f32" else pa.HIP16(0, storage=storage)
    try:
        tW = dev.new_tensor_by_vector(S([4 * H, I + H]), f32(W).T.reshape(-1))      # column-major
        tb = dev.new_tensor_by_vector(S([4 * H]), f32(b))
        txs = [dev.new_tensor_by_vector(S([I], B), f32(x).reshape(-1)) for x in xs]
        tgys = [dev.new_tensor_by_vector(S([H], B), f32(g).reshape(-1)) for g in gys]
        gW, gb = dev.new_tensor_by_constant(tW.shape(), 0), dev.new_tensor_by_constant(tb.shape(), 0)
        h_last, gx_first = dev.new_tensor_by_constant(S([H], B), 0), dev.new_tensor_by_constant(S([I], B), 0)
        arr = lambda ts: (ctypes.c_void_p * T)(*[t.handle() for t in ts])
        d = bench._LstmDims(I, H, B, T)
        ev, host = ctypes.c_float(), ctypes.c_double()
        rc = bench._native().phip_bench_lstm_loop(dev.ctx(), bench.STORAGE_CODE[storage], ctypes.byref(d), tW.handle(),
                                                  tb.handle(), gW.mutable_handle(), gb.mutable_handle(), arr(txs),
                                                  arr(tgys), h_last.mutable_handle(), gx_first.mutable_handle(), 0, 1, 0,
                                                  ctypes.byref(ev), ctypes.byref(host))
        assert rc == 0, _lib.lib().phip_last_error()
        # the reference rounds its inputs the way the device stores them
        r = lambda t, shape: t.to_vector().astype(np.float64).reshape(shape)
        Wd, bd = r(tW, (I + H, 4 * H)).T, r(tb, (4 * H,))
        want_h, want_gW, want_gb, want_gx0 = _lstm_float64(Wd, bd, [r(t, (B, I)) for t in txs], [r(t, (B, H)) for t in tgys])
        tol = 1e-4 if storage == "f32" else 2e-2
        assert norm_rel_err(h_last.to_vector(), want_h.reshape(-1)) <= tol
        assert norm_rel_err(gW.to_vector(), want_gW.T.reshape(-1)) <= tol
        assert norm_rel_err(gb.to_vector(), want_gb) <= tol
        assert norm_rel_err(gx_first.to_vector(), want_gx0.reshape(-1)) <= tol
        # the graph was cleared: every node value and gradient went back to the pool
        sup, res = ctypes.c_uint64(), ctypes.c_uint64()
        _lib.call("phip_pool_stats", dev.ctx(), ctypes.byref(sup), ctypes.byref(res))
        held = sum(t.allocated_size() for t in [tW, tb, gW, gb, h_last, gx_first] + txs + tgys)
        assert sup.value == held
    finally:
        dev.close()
