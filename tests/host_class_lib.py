"""Builds and binds `libhostclass.so`: the C++ class primitiv::devices::HIP and its
C-API constructors, linked with the real primitiv core, the real primitiv C
API and a host stand-in for libphip (tests/host_class/phip_host_stub.cc).

Test infrastructure for the build container only: it needs the primitiv source
tree (never present on a GPU box) and g++.  Nothing is copied from that tree:
its sources are compiled where they lie.  The one generated header primitiv
needs, primitiv/config.h, is produced from primitiv's own template
(primitiv/config.h.in) the way its build does, with every optional backend off.

`HostDevice` wraps a Device* in the method names of the Python mirror
(primitiv_amd/device.py), so the golden-vector cases written for the GPU run
unchanged through the C++ class.
"""
import concurrent.futures
import ctypes
import glob
import hashlib
import os
import re
import shutil
import subprocess

import numpy as np

import primitiv_amd as pa

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = os.environ.get("PRIMITIV_SOURCE_DIR", "/root/reference")
HERE = os.path.join(ROOT, "tests", "host_class")
BUILD = os.path.join(HERE, "build")


def available():
    return os.path.isdir(os.path.join(REF, "primitiv", "core")) and shutil.which("g++") is not None


REASON = "needs the primitiv source tree and g++"


def _own_sources():
    return [
        os.path.join(ROOT, "primitiv_amd", "primitiv", "devices", "hip", "device.cc"),
        os.path.join(ROOT, "primitiv_amd", "primitiv", "c", "devices", "hip", "device.cc"),
        os.path.join(HERE, "phip_host_stub.cc"),
        os.path.join(HERE, "front_shim.cc"),
    ]


def _reference_sources():
    pats = ["core/*.cc", "devices/naive/*.cc", "devices/naive/ops/*.cc", "c/*.cc", "c/internal/*.cc",
            "c/devices/naive/*.cc"]
    out = []
    for p in pats:
        out += sorted(glob.glob(os.path.join(REF, "primitiv", p)))
    return out


def _oracle_sources():
    return sorted(glob.glob(os.path.join(ROOT, "oracle", "ref_*.c")))


def _digest():
    h = hashlib.sha256()
    deps = _own_sources() + _oracle_sources() + [
        os.path.join(ROOT, "include", "phip.h"),
        os.path.join(ROOT, "primitiv_amd", "primitiv", "devices", "hip", "device.h"),
        os.path.join(ROOT, "primitiv_amd", "primitiv", "c", "devices", "hip", "device.h"),
        os.path.abspath(__file__),
    ]
    for path in deps:
        with open(path, "rb") as f:
            h.update(path.encode() + b"\0" + f.read())
    for path in _reference_sources():
        st = os.stat(path)
        h.update(("%s %d %d" % (path, st.st_size, int(st.st_mtime))).encode())
    return h.hexdigest()[:16]


def _write_config(gen):
    """primitiv/config.h from primitiv's template: `#cmakedefine X` becomes a comment when
    option X is off, which is what its build writes (primitiv/CMakeLists.txt:4-7)."""
    os.makedirs(os.path.join(gen, "primitiv"), exist_ok=True)
    with open(os.path.join(REF, "primitiv", "config.h.in")) as f:
        text = f.read()
    text = re.sub(r"#cmakedefine (\w+)", r"/* #undef \1 */", text)
    with open(os.path.join(gen, "primitiv", "config.h"), "w") as f:
        f.write(text)


def build():
    """Returns the path of libhostclass.so, compiling it when its sources changed."""
    tag = _digest()
    out_dir = os.path.join(BUILD, tag)
    lib = os.path.join(out_dir, "libhostclass.so")
    if os.path.exists(lib):
        return lib
    shutil.rmtree(BUILD, ignore_errors=True)
    os.makedirs(out_dir)
    gen = os.path.join(out_dir, "gen")
    _write_config(gen)
    inc = ["-I" + gen, "-I" + REF, "-I" + os.path.join(ROOT, "primitiv_amd"), "-I" + os.path.join(ROOT, "include")]
    jobs = []
    for i, src in enumerate(_reference_sources()):
        # the reference's own code: its warnings are not this build's business
        jobs.append((["g++", "-std=c++11", "-O1", "-fPIC", "-w"] + inc, src, "ref%03d.o" % i))
    for i, src in enumerate(_own_sources()):
        jobs.append((["g++", "-std=c++11", "-O1", "-fPIC", "-Wall", "-Wextra", "-Werror"] + inc, src, "own%d.o" % i))
    for i, src in enumerate(_oracle_sources()):
        jobs.append((["gcc", "-std=c11", "-O2", "-fPIC", "-mavx2", "-mfma", "-w"], src, "oracle%d.o" % i))

    def compile_one(job):
        cmd, src, obj = job
        obj = os.path.join(out_dir, obj)
        res = subprocess.run(cmd + ["-c", src, "-o", obj], capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError("compiling %s failed:\n%s" % (src, res.stderr[-4000:]))
        return obj

    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as ex:
        objs = list(ex.map(compile_one, jobs))
    res = subprocess.run(["g++", "-shared", "-o", lib] + objs + ["-lm"], capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("linking libhostclass.so failed:\n" + res.stderr[-4000:])
    return lib


_lib = None
_vp = ctypes.c_void_p
_u32 = ctypes.c_uint32
_pp = ctypes.POINTER(ctypes.c_void_p)


class HostError(RuntimeError):
    """A primitiv::Error that came out of the C++ front."""


def lib():
    global _lib
    if _lib is None:
        l = ctypes.CDLL(build())
        l.hc_last_error.restype = ctypes.c_char_p
        _lib = l
    return _lib


def call(name, *args):
    rc = getattr(lib(), name)(*args)
    if rc != 0:
        raise HostError(lib().hc_last_error().decode("utf-8", "replace"))


def c_api(name, *args):
    """A function of primitiv's C API; raises with primitivGetMessage on a non-zero status."""
    rc = getattr(lib(), name)(*args)
    if rc != 0:
        size = ctypes.c_size_t(0)
        lib().primitivGetMessage(None, ctypes.byref(size))
        buf = ctypes.create_string_buffer(size.value + 1)
        lib().primitivGetMessage(buf, ctypes.byref(size))
        lib().primitivResetStatus()
        raise HostError(buf.value.decode("utf-8", "replace"))


def stub_stats():
    vals = [ctypes.c_uint64(0) for _ in range(5)]
    ctxs = ctypes.c_int(0)
    lib().phip_stub_stats(*[ctypes.byref(v) for v in vals], ctypes.byref(ctxs))
    keys = ("live_bytes", "live_blocks", "malloc_calls", "failed_mallocs", "release_calls")
    out = {k: v.value for k, v in zip(keys, vals)}
    out["live_contexts"] = ctxs.value
    return out


def stub_set_memory_limit(nbytes):
    lib().phip_stub_set_memory_limit(ctypes.c_uint64(nbytes))


def _dims(dims):
    arr = (ctypes.c_uint32 * max(1, len(dims)))(*dims)
    return arr, len(dims)


def _f32(values):
    return np.ascontiguousarray(np.asarray(values, dtype=np.float32).reshape(-1))


def _ids(ids):
    ids = [int(i) for i in ids]
    return (ctypes.c_uint32 * max(1, len(ids)))(*ids), len(ids)


class HostTensor:
    """Owns one heap-allocated primitiv::Tensor."""

    def __init__(self, ptr, dev=None):
        self.ptr = ptr if isinstance(ptr, ctypes.c_void_p) else ctypes.c_void_p(ptr)
        self.dev = dev

    def __del__(self):
        try:
            if self.ptr:
                lib().hc_tensor_delete(self.ptr)
        except Exception:
            pass

    def valid(self):
        out = ctypes.c_int(0)
        call("hc_tensor_valid", self.ptr, ctypes.byref(out))
        return bool(out.value)

    def shape(self):
        dims = (ctypes.c_uint32 * 8)()
        depth, batch, size = _u32(0), _u32(0), _u32(0)
        call("hc_tensor_shape", self.ptr, dims, ctypes.byref(depth), ctypes.byref(batch), ctypes.byref(size))
        return pa.Shape(list(dims)[:depth.value], batch.value)

    def to_vector(self):
        out = np.empty(self.shape().size(), dtype=np.float32)
        call("hc_tensor_to_vector", self.ptr, out.ctypes.data_as(_vp))
        return out

    def to_float(self):
        out = ctypes.c_float(0)
        call("hc_tensor_to_float", self.ptr, ctypes.byref(out))
        return out.value

    def share(self):
        """Another Tensor object on the same memory (Tensor's copy constructor)."""
        out = _vp()
        call("hc_tensor_share", self.ptr, ctypes.byref(out))
        return HostTensor(out, self.dev)

    copy = share

    def reset(self, k):
        call("hc_tensor_reset", self.ptr, ctypes.c_float(k))

    def reset_by_array(self, values):
        v = _f32(values)
        call("hc_tensor_reset_by_array", self.ptr, v.ctypes.data_as(_vp))

    def inplace_add(self, x):
        call("hc_tensor_inplace_add", self.ptr, x.ptr)

    def inplace_subtract(self, x):
        call("hc_tensor_inplace_subtract", self.ptr, x.ptr)

    def inplace_multiply_const(self, k):
        call("hc_tensor_inplace_multiply_const", self.ptr, ctypes.c_float(k))

    def argmax(self, dim):
        s = self.shape()
        out = (ctypes.c_uint32 * max(1, s.size() // s[dim]))()
        call("hc_tensor_argmax", self.ptr, dim, out)
        return list(out)[:s.size() // s[dim]]

    def argmin(self, dim):
        s = self.shape()
        out = (ctypes.c_uint32 * max(1, s.size() // s[dim]))()
        call("hc_tensor_argmin", self.ptr, dim, out)
        return list(out)[:s.size() // s[dim]]


def _shape_args(shape):
    if hasattr(shape, "dims"):
        return list(shape.dims()), shape.batch()
    return list(shape), 1


class HostDevice:
    """A primitiv::devices::HIP object (or, with storage "naive", primitiv's own CPU device) behind
    the Python mirror's method names."""

    UNARY_OPS = ("negate", "abs", "sqrt", "exp", "log", "tanh", "sigmoid", "softplus", "sin", "cos", "tan")

    def __init__(self, storage="f32", seed=1, via_c_api=False, device_id=0):
        self.storage = storage
        self._SUFFIX = storage
        self.ptr = _vp()
        if storage == "naive":
            # primitiv's own CPU device behind the same wrapper
            call("hc_device_new_naive", _u32(seed), ctypes.byref(self.ptr))
        elif via_c_api:
            if storage == "f32":
                c_api("primitivCreateHipDeviceWithSeed", _u32(device_id), _u32(seed), ctypes.byref(self.ptr))
            else:
                c_api("primitivCreateHip16DeviceWithSeed", _u32(device_id), _u32(seed),
                      _u32(1 if storage == "bf16" else 0), ctypes.byref(self.ptr))
        else:
            call("hc_device_new", _u32(device_id), _u32(seed), _u32({"f32": 0, "f16": 1, "bf16": 2}[storage]),
                 ctypes.byref(self.ptr))

    def close(self):
        if self.ptr:
            call("hc_device_delete", self.ptr)
            self.ptr = _vp()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def type(self):
        out = _u32(0)
        call("hc_device_type", self.ptr, ctypes.byref(out))
        return out.value

    def _t(self, out):
        return HostTensor(out, self)

    # -- storage ----------------------------------------------------------
    def new_tensor_by_vector(self, shape, values):
        dims, batch = _shape_args(shape)
        arr, n = _dims(dims)
        v = _f32(values)
        out = _vp()
        call("hc_tensor_by_vector", self.ptr, arr, n, batch, v.ctypes.data_as(_vp), ctypes.c_size_t(v.size),
             ctypes.byref(out))
        return self._t(out)

    def new_tensor_by_constant(self, shape, k):
        dims, batch = _shape_args(shape)
        arr, n = _dims(dims)
        out = _vp()
        call("hc_tensor_by_constant", self.ptr, arr, n, batch, ctypes.c_float(k), ctypes.byref(out))
        return self._t(out)

    def copy_tensor(self, x):
        return self._fw_x("copy_tensor", x)

    # -- generic front calls ------------------------------------------------
    def _fw_x(self, name, x):
        out = _vp()
        call("hc_fw_x", self.ptr, name.encode(), x.ptr, ctypes.byref(out))
        return self._t(out)

    def _fw_ab(self, name, a, b):
        out = _vp()
        call("hc_fw_ab", self.ptr, name.encode(), a.ptr, b.ptr, ctypes.byref(out))
        return self._t(out)

    def matmul_fw(self, a, b):
        return self._fw_ab("matmul", a, b)

    def matmul_bw(self, a, b, y, gy, ga, gb):
        call("hc_bw_ab", self.ptr, b"matmul", a.ptr, b.ptr, y.ptr, gy.ptr, ga.ptr, gb.ptr)

    def inplace_add(self, x, y):
        call("hc_inplace_add", self.ptr, x.ptr, y.ptr)

    def inplace_subtract(self, x, y):
        call("hc_inplace_subtract", self.ptr, x.ptr, y.ptr)

    def inplace_multiply_const(self, k, x):
        call("hc_inplace_multiply_const", self.ptr, ctypes.c_float(k), x.ptr)

    def batch_sum_fw(self, x):
        return self._fw_x("batch_sum", x)

    def identity(self, size):
        out = _vp()
        call("hc_identity", self.ptr, _u32(size), ctypes.byref(out))
        return self._t(out)

    # -- elementwise families ---------------------------------------------
    def unary_fw(self, op, x):
        return self._fw_x(op, x)

    def unary_bw(self, op, x, y, gy, gx):
        call("hc_bw_x", self.ptr, op.encode(), x.ptr, y.ptr, gy.ptr, gx.ptr)

    def const_fw(self, op, x, k):
        out = _vp()
        call("hc_fw_xk", self.ptr, op.encode(), x.ptr, ctypes.c_float(k), ctypes.byref(out))
        return self._t(out)

    def const_bw(self, op, x, y, gy, k, gx):
        call("hc_bw_xk", self.ptr, op.encode(), x.ptr, y.ptr, gy.ptr, ctypes.c_float(k), gx.ptr)

    def pown_fw(self, x, k):
        out = _vp()
        call("hc_pown_fw", self.ptr, x.ptr, ctypes.c_int32(k), ctypes.byref(out))
        return self._t(out)

    def pown_bw(self, x, y, gy, k, gx):
        call("hc_pown_bw", self.ptr, x.ptr, y.ptr, gy.ptr, ctypes.c_int32(k), gx.ptr)

    def scalar_fw(self, name, x, k):
        return self._fw_ab(name, x, k)

    def binary_fw(self, op, a, b):
        return self._fw_ab(op, a, b)

    def binary_bw(self, op, a, b, y, gy, ga, gb):
        call("hc_bw_ab", self.ptr, op.encode(), a.ptr, b.ptr, y.ptr, gy.ptr, ga.ptr, gb.ptr)

    # -- moving and reducing along one dimension ----------------------------
    def slice_fw(self, x, dim, lower, upper):
        out = _vp()
        call("hc_slice_fw", self.ptr, x.ptr, _u32(dim), _u32(lower), _u32(upper), ctypes.byref(out))
        return self._t(out)

    def slice_bw(self, gy, dim, offset, gx):
        call("hc_slice_bw", self.ptr, gy.ptr, _u32(dim), _u32(offset), gx.ptr)

    def concat_fw(self, xs, dim):
        arr = (ctypes.c_void_p * len(xs))(*[x.ptr.value for x in xs])
        out = _vp()
        call("hc_concat_fw", self.ptr, arr, _u32(len(xs)), _u32(dim), ctypes.byref(out))
        return self._t(out)

    def pick_fw(self, x, ids, dim):
        arr, n = _ids(ids)
        out = _vp()
        call("hc_pick_fw", self.ptr, x.ptr, arr, _u32(n), _u32(dim), ctypes.byref(out))
        return self._t(out)

    def pick_bw(self, gy, ids, dim, gx):
        arr, n = _ids(ids)
        call("hc_pick_bw", self.ptr, gy.ptr, arr, _u32(n), _u32(dim), gx.ptr)

    def batch_pick_fw(self, x, ids):
        arr, n = _ids(ids)
        out = _vp()
        call("hc_batch_pick_fw", self.ptr, x.ptr, arr, _u32(n), ctypes.byref(out))
        return self._t(out)

    def batch_pick_bw(self, gy, ids, gx):
        arr, n = _ids(ids)
        call("hc_batch_pick_bw", self.ptr, gy.ptr, arr, _u32(n), gx.ptr)

    def batch_slice_fw(self, x, lower, upper):
        out = _vp()
        call("hc_batch_slice_fw", self.ptr, x.ptr, _u32(lower), _u32(upper), ctypes.byref(out))
        return self._t(out)

    def batch_slice_bw(self, gy, offset, gx):
        call("hc_batch_slice_bw", self.ptr, gy.ptr, _u32(offset), gx.ptr)

    def batch_concat_fw(self, xs):
        arr = (ctypes.c_void_p * len(xs))(*[x.ptr.value for x in xs])
        out = _vp()
        call("hc_batch_concat_fw", self.ptr, arr, _u32(len(xs)), ctypes.byref(out))
        return self._t(out)

    def transpose_fw(self, x):
        return self._fw_x("transpose", x)

    def transpose_bw(self, x, y, gy, gx):
        call("hc_bw_x", self.ptr, b"transpose", x.ptr, y.ptr, gy.ptr, gx.ptr)

    def permute_dims_fw(self, x, perm):
        arr, n = _ids(perm)
        out = _vp()
        call("hc_permute_dims_fw", self.ptr, x.ptr, arr, _u32(n), ctypes.byref(out))
        return self._t(out)

    def permute_dims_bw(self, x, y, gy, perm, gx):
        arr, n = _ids(perm)
        call("hc_permute_dims_bw", self.ptr, x.ptr, y.ptr, gy.ptr, arr, _u32(n), gx.ptr)

    def flip_fw(self, x, dim):
        return self._fw_xdim("flip", x, dim)

    def flip_bw(self, gy, dim, gx):
        call("hc_flip_bw", self.ptr, gy.ptr, _u32(dim), gx.ptr)

    def _fw_xdim(self, name, x, dim):
        out = _vp()
        call("hc_fw_xdim", self.ptr, name.encode(), x.ptr, _u32(dim), ctypes.byref(out))
        return self._t(out)

    def reduce_fw(self, op, x, dim):
        return self._fw_xdim(op, x, dim)

    def extremum_bw(self, op, x, y, gy, dim, gx):
        call("hc_bw_xdim", self.ptr, op.encode(), x.ptr, y.ptr, gy.ptr, _u32(dim), gx.ptr)

    def arg_extremum(self, op, x, dim):
        return x.argmax(dim) if op == "max" else x.argmin(dim)

    def broadcast_fw(self, x, dim, size):
        out = _vp()
        call("hc_broadcast_fw", self.ptr, x.ptr, _u32(dim), _u32(size), ctypes.byref(out))
        return self._t(out)

    # -- random tensors, convolution, pooling --------------------------------
    def _random(self, kind, shape, p0, p1=0.0):
        dims, batch = _shape_args(shape)
        arr, n = _dims(dims)
        out = _vp()
        call("hc_random", self.ptr, kind, arr, n, batch, ctypes.c_float(p0), ctypes.c_float(p1), ctypes.byref(out))
        return self._t(out)

    def random_uniform(self, shape, lower, upper):
        return self._random(0, shape, lower, upper)

    def random_bernoulli(self, shape, p):
        return self._random(1, shape, p)

    def random_normal(self, shape, mean, sd):
        return self._random(2, shape, mean, sd)

    def random_log_normal(self, shape, mean, sd):
        return self._random(3, shape, mean, sd)

    def conv2d_fw(self, x, w, *p):
        out = _vp()
        call("hc_conv2d_fw", self.ptr, x.ptr, w.ptr, (ctypes.c_uint32 * 6)(*p), ctypes.byref(out))
        return self._t(out)

    def conv2d_bw(self, x, w, y, gy, p0, p1, s0, s1, d0, d1, gx, gw):
        call("hc_conv2d_bw", self.ptr, x.ptr, w.ptr, y.ptr, gy.ptr, (ctypes.c_uint32 * 6)(p0, p1, s0, s1, d0, d1),
             gx.ptr, gw.ptr)

    def max_pool2d_fw(self, x, *p):
        out = _vp()
        call("hc_max_pool2d_fw", self.ptr, x.ptr, (ctypes.c_uint32 * 6)(*p), ctypes.byref(out))
        return self._t(out)

    def max_pool2d_bw(self, x, y, gy, w0, w1, p0, p1, s0, s1, gx):
        call("hc_max_pool2d_bw", self.ptr, x.ptr, y.ptr, gy.ptr, (ctypes.c_uint32 * 6)(w0, w1, p0, p1, s0, s1), gx.ptr)
