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
    "REDUCE_OPS", "slice_fw", "slice_bw", "concat_fw", "pick_fw", "pick_bw", "batch_pick_fw",
    "batch_pick_bw", "batch_slice_fw", "batch_slice_bw", "batch_concat_fw", "transpose_fw",
    "transpose_bw", "permute_dims_fw", "permute_dims_bw", "flip_fw", "flip_bw", "reduce_fw",
    "extremum_bw", "arg_extremum", "broadcast_fw",
    "RANDOM_KINDS", "philox4x32_10", "random",
    "shape_conv2d", "shape_pool2d", "conv2d_fw", "conv2d_bw", "max_pool2d_fw", "max_pool2d_bw",
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
        _D = ctypes.POINTER(_U)
        for name, args in (
                ("ref_slice_fw", [_F, _D, _U, _U, _U, _U, _U, _F]),
                ("ref_slice_bw", [_F, _U, _U, _D, _U, _U, _U, _U, _F]),
                ("ref_concat_fw_one", [_F, _U, _U, _D, _U, _U, _U, _U, _F]),
                ("ref_pick_fw", [_F, _D, _U, _U, _D, _U, _U, _F]),
                ("ref_pick_bw", [_F, _D, _U, _U, _D, _U, _U, _F]),
                ("ref_batch_pick_fw", [_F, _U, _D, _U, _F]),
                ("ref_batch_pick_bw", [_F, _U, _D, _U, _F]),
                ("ref_batch_slice_fw", [_F, _U, _U, _U, _F]),
                ("ref_batch_slice_bw", [_F, _U, _U, _U, _F]),
                ("ref_transpose_fw", [_F, _U, _U, _U, _F]),
                ("ref_transpose_bw", [_F, _U, _U, _U, _F]),
                ("ref_permute_dims_fw", [_F, _D, _U, _D, _U, _F]),
                ("ref_permute_dims_bw", [_F, _D, _U, _D, _U, _F]),
                ("ref_flip", [_F, _D, _U, _U, _U, _I, _F]),
                ("ref_extremum_bw", [_F, _F, _F, _D, _U, _U, _U, _F]),
                ("ref_arg_extremum", [_I, _F, _D, _U, _U, _U, _D]),
                ("ref_broadcast_fw", [_F, _D, _U, _U, _U, _U, _F])):
            getattr(l, name).argtypes = args
            getattr(l, name).restype = None
        l.ref_reduce_fw.argtypes = [_I, _F, _D, _U, _U, _U, _F]
        l.ref_philox4x32_10.argtypes = [_D, _D, _D]
        l.ref_philox4x32_10.restype = None
        l.ref_random.argtypes = [_I, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_float, ctypes.c_float, _F, _Z]
        l.ref_shape_conv2d.argtypes = [_U] * 15 + [_D, _D]
        l.ref_shape_conv2d.restype = ctypes.c_int
        l.ref_shape_pool2d.argtypes = [_U] * 8 + [_D]
        l.ref_shape_pool2d.restype = ctypes.c_int
        l.ref_conv2d_fw.argtypes = [_F, _F, _F] + [_U] * 14
        l.ref_conv2d_fw.restype = None
        l.ref_conv2d_bw.argtypes = [_F, _F, _F, _F, _F] + [_U] * 14
        l.ref_conv2d_bw.restype = None
        l.ref_max_pool2d_fw.argtypes = [_F, _F] + [_U] * 9
        l.ref_max_pool2d_fw.restype = None
        l.ref_max_pool2d_bw.argtypes = [_F, _F, _F, _F] + [_U] * 9
        l.ref_max_pool2d_bw.restype = None
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


# ---- data movement and reductions (ref_indexing.c) -----------------------------
# Tensors are (flat float32 array, dims, batch); dims is the list of extents,
# dimension 0 first, as primitiv's Shape holds them.
REDUCE_OPS = ["sum", "logsumexp", "max", "min"]


def _dims(dims):
    dims = [int(d) for d in dims]
    return (_U * max(1, len(dims)))(*dims), len(dims)


def _ids(ids):
    ids = [int(i) for i in ids]
    return (_U * max(1, len(ids)))(*ids), len(ids)


def _vol(dims):
    v = 1
    for d in dims:
        v *= int(d)
    return v


def _dim(dims, i):
    return int(dims[i]) if i < len(dims) else 1


def slice_fw(x, dims, batch, dim, lower, upper):
    x = _f32(x)
    assert x.size == _vol(dims) * batch
    d, depth = _dims(dims)
    y = np.empty(x.size // _dim(dims, dim) * (upper - lower), dtype=np.float32)
    lib().ref_slice_fw(_p(x), d, depth, batch, dim, lower, upper - lower, _p(y))
    return y


def slice_bw(gy, by, ny, gx, dims, bx, dim, offset):
    """Returns gx plus gy placed at `offset` along dim (gx has dims x bx, gy extent ny along dim, batch by)."""
    gy, gx = _f32(gy), _f32(gx).copy()
    assert gx.size == _vol(dims) * bx and gy.size == _vol(dims) // _dim(dims, dim) * ny * by
    d, depth = _dims(dims)
    lib().ref_slice_bw(_p(gy), by, ny, d, depth, bx, dim, offset, _p(gx))
    return gx


def concat_fw(xs, dim):
    """xs: list of (array, dims, batch); returns (array, dims, batch) of the concatenation along dim."""
    dims0 = list(xs[0][1]) + [1] * max(0, dim + 1 - len(xs[0][1]))
    ydims = list(dims0)
    ydims[dim] = sum(_dim(x[1], dim) for x in xs)
    by = max(x[2] for x in xs)
    y = np.empty(_vol(ydims) * by, dtype=np.float32)
    d, depth = _dims(ydims)
    offset = 0
    for arr, dims, batch in xs:
        arr = _f32(arr)
        assert arr.size == _vol(dims) * batch
        lib().ref_concat_fw_one(_p(arr), _dim(dims, dim), batch, d, depth, by, dim, offset, _p(y))
        offset += _dim(dims, dim)
    return y, ydims, by


def pick_fw(x, dims, bx, ids, dim):
    x = _f32(x)
    assert x.size == _vol(dims) * bx
    d, depth = _dims(dims)
    i, n = _ids(ids)
    y = np.empty(_vol(dims) // _dim(dims, dim) * max(bx, n), dtype=np.float32)
    lib().ref_pick_fw(_p(x), d, depth, bx, i, n, dim, _p(y))
    return y


def pick_bw(gy, gx, dims, bx, ids, dim):
    gy, gx = _f32(gy), _f32(gx).copy()
    d, depth = _dims(dims)
    i, n = _ids(ids)
    assert gx.size == _vol(dims) * bx and gy.size == _vol(dims) // _dim(dims, dim) * max(bx, n)
    lib().ref_pick_bw(_p(gy), d, depth, bx, i, n, dim, _p(gx))
    return gx


def batch_pick_fw(x, volume, ids):
    x = _f32(x)
    i, n = _ids(ids)
    y = np.empty(volume * n, dtype=np.float32)
    lib().ref_batch_pick_fw(_p(x), volume, i, n, _p(y))
    return y


def batch_pick_bw(gy, gx, volume, ids):
    gy, gx = _f32(gy), _f32(gx).copy()
    i, n = _ids(ids)
    assert gy.size == volume * n
    lib().ref_batch_pick_bw(_p(gy), volume, i, n, _p(gx))
    return gx


def batch_slice_fw(x, volume, lower, upper):
    x = _f32(x)
    y = np.empty(volume * (upper - lower), dtype=np.float32)
    lib().ref_batch_slice_fw(_p(x), volume, lower, upper - lower, _p(y))
    return y


def batch_slice_bw(gy, gx, volume, offset):
    gy, gx = _f32(gy), _f32(gx).copy()
    lib().ref_batch_slice_bw(_p(gy), volume, offset, gy.size // volume, _p(gx))
    return gx


def batch_concat_fw(xs):
    # naive/ops/batch_concat.cc:11-22: the inputs one after the other
    return np.concatenate([_f32(x) for x in xs])


def transpose_fw(x, d1, d2, bs):
    x = _f32(x)
    assert x.size == d1 * d2 * bs
    y = np.empty_like(x)
    lib().ref_transpose_fw(_p(x), d1, d2, bs, _p(y))
    return y


def transpose_bw(gy, gx, d1, d2, bs):
    """gx (d1 x d2 per sample) plus the transpose of gy (d2 x d1)."""
    gy, gx = _f32(gy), _f32(gx).copy()
    lib().ref_transpose_bw(_p(gy), d1, d2, bs, _p(gx))
    return gx


def permute_dims_fw(x, dims, perm, bs):
    x = _f32(x)
    dims = list(dims) + [1] * (len(perm) - len(dims))
    d, nd = _dims(dims)
    pm, _ = _ids(perm)
    y = np.empty_like(x)
    lib().ref_permute_dims_fw(_p(x), d, nd, pm, bs, _p(y))
    return y


def permute_dims_bw(gy, gx, dims, perm, bs):
    gy, gx = _f32(gy), _f32(gx).copy()
    dims = list(dims) + [1] * (len(perm) - len(dims))
    d, nd = _dims(dims)
    pm, _ = _ids(perm)
    lib().ref_permute_dims_bw(_p(gy), d, nd, pm, bs, _p(gx))
    return gx


def flip_fw(x, dims, batch, dim):
    x = _f32(x)
    d, depth = _dims(dims)
    y = np.empty_like(x)
    lib().ref_flip(_p(x), d, depth, batch, dim, 0, _p(y))
    return y


def flip_bw(gy, gx, dims, batch, dim):
    gy, gx = _f32(gy), _f32(gx).copy()
    d, depth = _dims(dims)
    lib().ref_flip(_p(gy), d, depth, batch, dim, 1, _p(gx))
    return gx


def reduce_fw(op, x, dims, batch, dim):
    x = _f32(x)
    assert x.size == _vol(dims) * batch
    d, depth = _dims(dims)
    y = np.empty(x.size // _dim(dims, dim), dtype=np.float32)
    _ok(lib().ref_reduce_fw(REDUCE_OPS.index(op), _p(x), d, depth, batch, dim, _p(y)), op)
    return y


def extremum_bw(x, y, gy, gx, dims, batch, dim):
    x, y, gy, gx = _f32(x), _f32(y), _f32(gy), _f32(gx).copy()
    d, depth = _dims(dims)
    lib().ref_extremum_bw(_p(x), _p(y), _p(gy), d, depth, batch, dim, _p(gx))
    return gx


def arg_extremum(op, x, dims, batch, dim):
    x = _f32(x)
    d, depth = _dims(dims)
    n = x.size // _dim(dims, dim)
    out = (_U * max(1, n))()
    lib().ref_arg_extremum(1 if op == "max" else 0, _p(x), d, depth, batch, dim, out)
    return np.array(out[:n], dtype=np.uint32)


def broadcast_fw(x, dims, batch, dim, size):
    x = _f32(x)
    d, depth = _dims(dims)
    y = np.empty(x.size * size, dtype=np.float32)
    lib().ref_broadcast_fw(_p(x), d, depth, batch, dim, size, _p(y))
    return y


# ---- random tensors (ref_random.c) ---------------------------------------------
RANDOM_KINDS = ["uniform", "bernoulli", "normal", "log_normal"]


def philox4x32_10(counter, key):
    """One Philox4x32-10 block: 4 counter words, 2 key words -> 4 output words."""
    c = (_U * 4)(*[int(v) for v in counter])
    k = (_U * 2)(*[int(v) for v in key])
    out = (_U * 4)()
    lib().ref_philox4x32_10(c, k, out)
    return list(out)


def random(kind, seed, offset, p0, p1, n):
    """n draws: uniform (p0, p1], bernoulli(p0), normal / log_normal (mean p0, sd p1)."""
    y = np.empty(n, dtype=np.float32)
    _ok(lib().ref_random(RANDOM_KINDS.index(kind), seed, offset, p0, p1, _p(y), n), kind)
    return y


# ---- convolution and pooling (ref_conv_pool.c) ---------------------------------
def _pad(dims, n):
    dims = [int(d) for d in dims]
    return dims + [1] * (n - len(dims))


def shape_conv2d(x_dims, bx, w_dims, bw, pad0, pad1, str0, str1, dil0, dil1):
    """(dims, batch) of conv2d's result; ValueError for arguments the reference rejects
    (shape_ops.cc:162-187)."""
    if len(x_dims) > 3 or len(w_dims) > 4:
        raise ValueError("Invalid arguments to calculate a convolution")
    x, w = _pad(x_dims, 3), _pad(w_dims, 4)
    dims, batch = (_U * 3)(), (_U * 1)()
    if lib().ref_shape_conv2d(x[0], x[1], x[2], bx, w[0], w[1], w[2], w[3], bw, pad0, pad1, str0, str1, dil0, dil1,
                              dims, batch):
        raise ValueError("Invalid arguments to calculate a convolution")
    return list(dims), int(batch[0])


def shape_pool2d(x_dims, win0, win1, pad0, pad1, str0, str1):
    """dims of max_pool2d's result (the minibatch is x's); ValueError as shape_ops.cc:189-213."""
    if len(x_dims) > 3:
        raise ValueError("Invalid arguments to calculate a pooling")
    x = _pad(x_dims, 3)
    dims = (_U * 2)()
    if lib().ref_shape_pool2d(x[0], x[1], win0, win1, pad0, pad1, str0, str1, dims):
        raise ValueError("Invalid arguments to calculate a pooling")
    return [int(dims[0]), int(dims[1]), x[2]]


def conv2d_fw(x, w, x_dims, bx, w_dims, bw, pad0, pad1, str0, str1, dil0, dil1):
    x, w = _f32(x), _f32(w)
    xd, wd = _pad(x_dims, 3), _pad(w_dims, 4)
    yd, bs = shape_conv2d(x_dims, bx, w_dims, bw, pad0, pad1, str0, str1, dil0, dil1)
    y = np.empty(int(np.prod(yd)) * bs, dtype=np.float32)
    lib().ref_conv2d_fw(_p(x), _p(w), _p(y), xd[0], xd[1], xd[2], wd[0], wd[1], wd[3], bx, bw, pad0, pad1, str0, str1,
                        dil0, dil1)
    return y


def conv2d_bw(x, w, gy, gx, gw, x_dims, bx, w_dims, bw, pad0, pad1, str0, str1, dil0, dil1):
    """(gx, gw) after the gradients have been added to copies of the given ones."""
    x, w, gy = _f32(x), _f32(w), _f32(gy)
    gx, gw = _f32(gx).copy(), _f32(gw).copy()
    xd, wd = _pad(x_dims, 3), _pad(w_dims, 4)
    lib().ref_conv2d_bw(_p(x), _p(w), _p(gy), _p(gx), _p(gw), xd[0], xd[1], xd[2], wd[0], wd[1], wd[3], bx, bw, pad0,
                        pad1, str0, str1, dil0, dil1)
    return gx, gw


def max_pool2d_fw(x, x_dims, bs, win0, win1, pad0, pad1, str0, str1):
    x = _f32(x)
    xd = _pad(x_dims, 3)
    yd = shape_pool2d(x_dims, win0, win1, pad0, pad1, str0, str1)
    y = np.empty(yd[0] * yd[1] * xd[2] * bs, dtype=np.float32)
    lib().ref_max_pool2d_fw(_p(x), _p(y), xd[0], xd[1], xd[2] * bs, win0, win1, pad0, pad1, str0, str1)
    return y


def max_pool2d_bw(x, y, gy, gx, x_dims, bs, win0, win1, pad0, pad1, str0, str1):
    x, y, gy = _f32(x), _f32(y), _f32(gy)
    gx = _f32(gx).copy()
    xd = _pad(x_dims, 3)
    lib().ref_max_pool2d_bw(_p(x), _p(y), _p(gy), _p(gx), xd[0], xd[1], xd[2] * bs, win0, win1, pad0, pad1, str0, str1)
    return gx
