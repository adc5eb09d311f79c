"""ctypes front of ``libref_primitiv.so`` (see ``ref_primitiv.c``).

Test infrastructure only.  Arrays are flat float32 numpy arrays in primitiv's
layout: column-major matrices, minibatch outermost.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libref_primitiv.so")
_lib = None

__all__ = [
    "build", "lib", "shape_matmul", "matmul_fw", "matmul_bw", "matmul_fw_f64",
    "matmul_bw_f64", "inplace_add", "batch_sum", "pool_block_size",
    "num_threads_available",
]

_F = ctypes.POINTER(ctypes.c_float)
_U = ctypes.c_uint32


def build(force=False):
    """Compile the oracle with gcc (always recompiles when ``force``)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libref_primitiv.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        l = ctypes.CDLL(_LIB_PATH)
        l.ref_shape_matmul.argtypes = [ctypes.POINTER(_U), _U, _U,
                                       ctypes.POINTER(_U), _U, _U,
                                       ctypes.POINTER(_U)]
        l.ref_shape_matmul.restype = ctypes.c_int
        l.ref_matmul_fw.argtypes = [_F, _F, _F, _U, _U, _U, _U, _U, ctypes.c_int]
        l.ref_matmul_fw.restype = None
        l.ref_matmul_bw.argtypes = [_F, _F, _F, _F, _F, _U, _U, _U, _U, _U,
                                    ctypes.c_int]
        l.ref_matmul_bw.restype = None
        l.ref_matmul_fw_f64.argtypes = [_F, _F, _F, _U, _U, _U, _U, _U]
        l.ref_matmul_fw_f64.restype = None
        l.ref_matmul_bw_f64.argtypes = [_F, _F, _F, _F, _F, _U, _U, _U, _U, _U]
        l.ref_matmul_bw_f64.restype = None
        l.ref_inplace_add.argtypes = [_F, _F, _U, _U, _U]
        l.ref_inplace_add.restype = None
        l.ref_batch_sum.argtypes = [_F, _F, _U, _U]
        l.ref_batch_sum.restype = None
        l.ref_pool_block_size.argtypes = [ctypes.c_uint64, ctypes.c_uint64]
        l.ref_pool_block_size.restype = ctypes.c_uint64
        l.ref_num_threads_available.argtypes = []
        l.ref_num_threads_available.restype = ctypes.c_int
        _lib = l
    return _lib


def _f32(x):
    return np.ascontiguousarray(np.asarray(x, dtype=np.float32).reshape(-1))


def _p(x):
    return x.ctypes.data_as(_F)


def shape_matmul(adims, abatch, bdims, bbatch):
    """Returns (rows, cols, batch) or None where the reference throws."""
    a = (_U * max(1, len(adims)))(*adims)
    b = (_U * max(1, len(bdims)))(*bdims)
    out = (_U * 3)()
    rc = lib().ref_shape_matmul(a, len(adims), abatch, b, len(bdims), bbatch, out)
    return None if rc != 0 else (out[0], out[1], out[2])


def _check(a, b, di, dj, dk, ba, bb):
    assert ba == bb or ba == 1 or bb == 1
    assert a.size == di * dj * ba, (a.size, di, dj, ba)
    assert b.size == dj * dk * bb, (b.size, dj, dk, bb)


def matmul_fw(a, b, di, dj, dk, ba, bb, threads=1):
    a, b = _f32(a), _f32(b)
    _check(a, b, di, dj, dk, ba, bb)
    y = np.empty(di * dk * max(ba, bb), dtype=np.float32)
    lib().ref_matmul_fw(_p(a), _p(b), _p(y), di, dj, dk, ba, bb, threads)
    return y


def matmul_bw(a, b, gy, ga, gb, di, dj, dk, ba, bb, threads=1):
    """Returns new (ga, gb) = inputs plus the accumulated gradients."""
    a, b, gy = _f32(a), _f32(b), _f32(gy)
    _check(a, b, di, dj, dk, ba, bb)
    assert gy.size == di * dk * max(ba, bb)
    ga, gb = _f32(ga).copy(), _f32(gb).copy()
    assert ga.size == a.size and gb.size == b.size
    lib().ref_matmul_bw(_p(a), _p(b), _p(gy), _p(ga), _p(gb), di, dj, dk, ba, bb,
                        threads)
    return ga, gb


def matmul_fw_f64(a, b, di, dj, dk, ba, bb):
    a, b = _f32(a), _f32(b)
    _check(a, b, di, dj, dk, ba, bb)
    y = np.empty(di * dk * max(ba, bb), dtype=np.float32)
    lib().ref_matmul_fw_f64(_p(a), _p(b), _p(y), di, dj, dk, ba, bb)
    return y


def matmul_bw_f64(a, b, gy, ga, gb, di, dj, dk, ba, bb):
    a, b, gy = _f32(a), _f32(b), _f32(gy)
    _check(a, b, di, dj, dk, ba, bb)
    ga, gb = _f32(ga).copy(), _f32(gb).copy()
    lib().ref_matmul_bw_f64(_p(a), _p(b), _p(gy), _p(ga), _p(gb), di, dj, dk, ba, bb)
    return ga, gb


def inplace_add(x, y, volume, bx, by):
    x, y = _f32(x), _f32(y).copy()
    assert x.size == volume * bx and y.size == volume * by
    lib().ref_inplace_add(_p(x), _p(y), volume, bx, by)
    return y


def batch_sum(x, volume, bs):
    x = _f32(x)
    assert x.size == volume * bs
    y = np.empty(volume, dtype=np.float32)
    lib().ref_batch_sum(_p(x), _p(y), volume, bs)
    return y


def pool_block_size(size, minimum=1):
    return int(lib().ref_pool_block_size(size, minimum))


def num_threads_available():
    return int(lib().ref_num_threads_available())
