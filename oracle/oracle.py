"""ctypes front of ``libref_primitiv.so`` (see ``ref_primitiv.c``, ``ref_pointwise.c``).

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
    "UNARY_OPS", "CONST_OPS", "BINARY_OPS", "unary_fw", "unary_bw", "const_fw",
    "const_bw", "pown_fw", "pown_bw", "scalar_fw", "binary_fw", "binary_bw",
    "inplace_subtract", "inplace_multiply_const", "identity",
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
        _I, _Z = ctypes.c_int, ctypes.c_size_t
        l.ref_unary_fw.argtypes = [_I, _F, _F, _Z]
        l.ref_unary_bw.argtypes = [_I, _F, _F, _F, _F, _Z]
        l.ref_const_fw.argtypes = [_I, _F, ctypes.c_float, _F, _Z]
        l.ref_const_bw.argtypes = [_I, _F, _F, _F, ctypes.c_float, _F, _Z]
        l.ref_pown_fw.argtypes = [_F, ctypes.c_int32, _F, _Z]
        l.ref_pown_fw.restype = None
        l.ref_pown_bw.argtypes = [_F, _F, _F, ctypes.c_int32, _F, _Z]
        l.ref_pown_bw.restype = None
        l.ref_scalar_fw.argtypes = [_I, _I, _F, _F, _F, _U, _U, _U]
        l.ref_binary_fw.argtypes = [_I, _F, _F, _F, _U, _U, _U]
        l.ref_binary_bw.argtypes = [_I, _F, _F, _F, _F, _F, _F, _U, _U, _U]
        l.ref_inplace_subtract.argtypes = [_F, _F, _U, _U, _U]
        l.ref_inplace_subtract.restype = None
        l.ref_inplace_multiply_const.argtypes = [ctypes.c_float, _F, _Z]
        l.ref_inplace_multiply_const.restype = None
        l.ref_identity.argtypes = [_F, _U]
        l.ref_identity.restype = None
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


# ---- elementwise operations (ref_pointwise.c) --------------------------------
# Operation names in the order of the oracle's own codes.
UNARY_OPS = ["negate", "abs", "sqrt", "exp", "log", "tanh", "sigmoid", "softplus",
             "sin", "cos", "tan"]
CONST_OPS = ["add_const", "subtract_const_r", "subtract_const_l", "multiply_const",
             "divide_const_r", "divide_const_l", "pow_const_r", "pow_const_l",
             "prelu", "elu"]
BINARY_OPS = ["add", "subtract", "multiply", "divide", "pow"]


def _ok(rc, what):
    if rc != 0:
        raise ValueError("the oracle has no operation %r" % (what,))


def unary_fw(op, x):
    x = _f32(x)
    y = np.empty_like(x)
    _ok(lib().ref_unary_fw(UNARY_OPS.index(op), _p(x), _p(y), x.size), op)
    return y


def unary_bw(op, x, y, gy, gx):
    """Returns gx + f'(x, y) * gy."""
    x, y, gy, gx = _f32(x), _f32(y), _f32(gy), _f32(gx).copy()
    assert x.size == y.size == gy.size == gx.size
    _ok(lib().ref_unary_bw(UNARY_OPS.index(op), _p(x), _p(y), _p(gy), _p(gx), x.size), op)
    return gx


def const_fw(op, x, k):
    x = _f32(x)
    y = np.empty_like(x)
    _ok(lib().ref_const_fw(CONST_OPS.index(op), _p(x), k, _p(y), x.size), op)
    return y


def const_bw(op, x, y, gy, k, gx):
    x, y, gy, gx = _f32(x), _f32(y), _f32(gy), _f32(gx).copy()
    assert x.size == y.size == gy.size == gx.size
    _ok(lib().ref_const_bw(CONST_OPS.index(op), _p(x), _p(y), _p(gy), k, _p(gx), x.size), op)
    return gx


def pown_fw(x, k):
    x = _f32(x)
    y = np.empty_like(x)
    lib().ref_pown_fw(_p(x), k, _p(y), x.size)
    return y


def pown_bw(x, y, gy, k, gx):
    x, y, gy, gx = _f32(x), _f32(y), _f32(gy), _f32(gx).copy()
    lib().ref_pown_bw(_p(x), _p(y), _p(gy), k, _p(gx), x.size)
    return gx


def scalar_fw(op, k_on_left, x, k, volume, bx, bk):
    x, k = _f32(x), _f32(k)
    assert x.size == volume * bx and k.size == bk
    y = np.empty(volume * max(bx, bk), dtype=np.float32)
    _ok(lib().ref_scalar_fw(BINARY_OPS.index(op), int(bool(k_on_left)), _p(x), _p(k), _p(y),
                            volume, bx, bk), op)
    return y


def binary_fw(op, a, b, volume, ba, bb):
    a, b = _f32(a), _f32(b)
    assert a.size == volume * ba and b.size == volume * bb
    y = np.empty(volume * max(ba, bb), dtype=np.float32)
    _ok(lib().ref_binary_fw(BINARY_OPS.index(op), _p(a), _p(b), _p(y), volume, ba, bb), op)
    return y


def binary_bw(op, a, b, y, gy, ga, gb, volume, ba, bb):
    """Returns new (ga, gb) = inputs plus the accumulated gradients."""
    a, b, y, gy = _f32(a), _f32(b), _f32(y), _f32(gy)
    ga, gb = _f32(ga).copy(), _f32(gb).copy()
    assert a.size == ga.size == volume * ba and b.size == gb.size == volume * bb
    assert y.size == gy.size == volume * max(ba, bb)
    _ok(lib().ref_binary_bw(BINARY_OPS.index(op), _p(a), _p(b), _p(y), _p(gy), _p(ga), _p(gb),
                            volume, ba, bb), op)
    return ga, gb


def inplace_subtract(x, y, volume, bx, by):
    x, y = _f32(x), _f32(y).copy()
    assert x.size == volume * bx and y.size == volume * by
    lib().ref_inplace_subtract(_p(x), _p(y), volume, bx, by)
    return y


def inplace_multiply_const(k, x):
    x = _f32(x).copy()
    lib().ref_inplace_multiply_const(k, _p(x), x.size)
    return x


def identity(rows):
    y = np.empty(rows * rows, dtype=np.float32)
    lib().ref_identity(_p(y), rows)
    return y
