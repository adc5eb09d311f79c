"""Comparison helpers shared by the tests.

`ulp_diff` / `vector_match` follow the reference's own test helpers
(test/test_utils.h:26-80: distance in units in the last place, 4 ULPs by
default).  `norm_rel_err` is the tolerance gate of the matmul path:
max|x - ref| / max|ref| over one output tensor.
"""
import numpy as np


def ulp_diff(a, b):
    a = np.asarray(a, dtype=np.float32).reshape(-1)
    b = np.asarray(b, dtype=np.float32).reshape(-1)
    ia = a.view(np.int32).astype(np.int64)
    ib = b.view(np.int32).astype(np.int64)
    ia = np.where(ia < 0, -(ia & 0x7FFFFFFF), ia)
    ib = np.where(ib < 0, -(ib & 0x7FFFFFFF), ib)
    return np.abs(ia - ib)


def round_to_storage(x, storage):
    """float32 values rounded once, to nearest even, to the 16-bit storage type ("f16" / "bf16"), as float32."""
    x = np.asarray(x, dtype=np.float32)
    if storage == "f16":
        with np.errstate(over="ignore"):
            return x.astype(np.float16).astype(np.float32)
    bits = x.view(np.uint32).astype(np.uint64)
    bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return bits.astype(np.uint32).view(np.float32)


def vector_match(expected, actual, ulps=4):
    expected = np.asarray(expected, dtype=np.float32).reshape(-1)
    actual = np.asarray(actual, dtype=np.float32).reshape(-1)
    return expected.shape == actual.shape and bool(np.all(ulp_diff(expected, actual) <= ulps))


def norm_rel_err(x, ref):
    x = np.asarray(x, dtype=np.float64).reshape(-1)
    ref = np.asarray(ref, dtype=np.float64).reshape(-1)
    assert x.shape == ref.shape
    denom = np.max(np.abs(ref))
    if denom == 0:
        return float(np.max(np.abs(x)))
    return float(np.max(np.abs(x - ref)) / denom)


def np_matmul_fw(a, b, di, dj, dk, ba, bb, dtype=np.float64):
    """Library float64 restatement: per-sample column-major products."""
    bs = max(ba, bb)
    A = np.asarray(a, dtype=dtype).reshape(ba, dj, di).transpose(0, 2, 1)
    B = np.asarray(b, dtype=dtype).reshape(bb, dk, dj).transpose(0, 2, 1)
    Y = np.matmul(np.broadcast_to(A, (bs, di, dj)), np.broadcast_to(B, (bs, dj, dk)))
    return Y.transpose(0, 2, 1).reshape(-1)


def np_matmul_bw(a, b, gy, di, dj, dk, ba, bb, dtype=np.float64):
    """Returns the increments (dga, dgb) in float64, flat column-major."""
    bs = max(ba, bb)
    A = np.broadcast_to(np.asarray(a, dtype=dtype).reshape(ba, dj, di).transpose(0, 2, 1), (bs, di, dj))
    B = np.broadcast_to(np.asarray(b, dtype=dtype).reshape(bb, dk, dj).transpose(0, 2, 1), (bs, dj, dk))
    GY = np.asarray(gy, dtype=dtype).reshape(bs, dk, di).transpose(0, 2, 1)
    GA = np.matmul(GY, B.transpose(0, 2, 1))
    GB = np.matmul(A.transpose(0, 2, 1), GY)
    if ba == 1:
        GA = GA.sum(axis=0, keepdims=True)
    if bb == 1:
        GB = GB.sum(axis=0, keepdims=True)
    return GA.transpose(0, 2, 1).reshape(-1), GB.transpose(0, 2, 1).reshape(-1)
