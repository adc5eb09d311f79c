"""Python mirror of primitiv's Device front for the matmul path.

This is the thin host side used by the tests and the benchmark: the same
method names, argument meaning and error behaviour as the reference's
`Device`, `Tensor` and `Shape` (primitiv/core/device.{h,cc},
primitiv/core/tensor.{h,cc}, primitiv/core/shape.{h,cc}), restricted to what
the matmul path touches.  All arithmetic happens in libphip.so on the GPU; this
file only checks shapes, owns handles and moves bytes.
"""
import ctypes
import os

import numpy as np

from . import _lib
from ._lib import Error


class Shape:
    """Up to 8 dimensions plus a minibatch size (primitiv/core/shape.h).

    Trailing dimensions of size 1 are not stored; `shape[i]` past the depth
    reads 1 (shape.h:55).
    """

    MAX_DEPTH = 8

    def __init__(self, dims=(), batch=1):
        dims = [int(d) for d in dims]
        if len(dims) > self.MAX_DEPTH:
            raise Error("Exceeds dimension depth limit at Shape.init: %d > %d" % (len(dims), self.MAX_DEPTH))
        while dims and dims[-1] == 1:
            dims.pop()
        if any(d <= 0 for d in dims) or batch <= 0:
            raise Error("Invalid shape: %s x %d" % (dims, batch))
        self._dims = tuple(dims)
        self._batch = int(batch)
        vol = 1
        for d in dims:
            vol *= d
        self._volume = vol

    def __getitem__(self, i):
        return self._dims[i] if i < len(self._dims) else 1

    def dims(self):
        return list(self._dims)

    def depth(self):
        return len(self._dims)

    def batch(self):
        return self._batch

    def volume(self):
        return self._volume

    def size(self):
        return self._batch * self._volume

    def has_batch(self):
        return self._batch > 1

    def has_compatible_batch(self, rhs):
        return self._batch == rhs._batch or self._batch == 1 or rhs._batch == 1

    def is_matrix(self):
        return len(self._dims) <= 2

    def has_same_dims(self, rhs):
        return self._dims == rhs._dims

    def resize_batch(self, batch):
        return Shape(self._dims, batch)

    def lower_volume(self, dim):
        # shape.h:100-104: product of the dimensions below `dim`
        v = 1
        for d in self._dims[:dim]:
            v *= d
        return v

    def resize_dim(self, dim, m):
        # shape.cc: the same shape with dimension `dim` set to m
        dims = list(self._dims) + [1] * max(0, dim + 1 - len(self._dims))
        dims[dim] = m
        return Shape(dims, self._batch)

    def has_same_loo_dims(self, rhs, dim):
        # shape.cc: equal in every dimension except `dim` ("leave one out")
        depth = max(len(self._dims), len(rhs._dims))
        return all(self[i] == rhs[i] for i in range(depth) if i != dim)

    def to_string(self):
        return "[%s]x%d" % (",".join(str(d) for d in self._dims), self._batch)

    __repr__ = to_string

    def __eq__(self, rhs):
        return isinstance(rhs, Shape) and self._dims == rhs._dims and self._batch == rhs._batch

    def __ne__(self, rhs):
        return not self.__eq__(rhs)

    def __hash__(self):
        return hash((self._dims, self._batch))


def _as_shape(s):
    return s if isinstance(s, Shape) else Shape(s)


class shape_ops:
    """Result-shape rules (primitiv/core/shape_ops.cc)."""

    @staticmethod
    def matmul(l, r):
        # shape_ops.cc:152-160
        if (not l.is_matrix() or not r.is_matrix() or l[1] != r[0]
                or not l.has_compatible_batch(r)):
            raise Error("Invalid shapes to calculate the matrix product: %s, %s"
                        % (l.to_string(), r.to_string()))
        return Shape([l[0], r[1]], max(l.batch(), r.batch()))

    @staticmethod
    def conv2d(x, w, padding0, padding1, stride0, stride1, dilation0, dilation1):
        # shape_ops.cc:162-187
        x0, x1 = x[0] + 2 * padding0, x[1] + 2 * padding1
        w0, w1 = (w[0] - 1) * dilation0 + 1, (w[1] - 1) * dilation1 + 1
        if (x.depth() > 3 or w.depth() > 4 or x0 < w0 or x1 < w1 or x[2] != w[2]
                or not x.has_compatible_batch(w) or stride0 == 0 or stride1 == 0
                or dilation0 == 0 or dilation1 == 0):
            raise Error("Invalid arguments to calculate a convolution: %s, %s, %d, %d, %d, %d, %d, %d"
                        % (x.to_string(), w.to_string(), padding0, padding1, stride0, stride1, dilation0, dilation1))
        return Shape([(x0 - w0) // stride0 + 1, (x1 - w1) // stride1 + 1, w[3]], max(x.batch(), w.batch()))

    @staticmethod
    def pool2d(x, window0, window1, padding0, padding1, stride0, stride1):
        # shape_ops.cc:189-213
        x0, x1 = x[0] + 2 * padding0, x[1] + 2 * padding1
        if (x.depth() > 3 or x0 < window0 or x1 < window1 or window0 == 0 or window1 == 0
                or stride0 == 0 or stride1 == 0):
            raise Error("Invalid arguments to calculate a pooling: %s, %d, %d, %d, %d, %d, %d"
                        % (x.to_string(), window0, window1, padding0, padding1, stride0, stride1))
        return Shape([(x0 - window0) // stride0 + 1, (x1 - window1) // stride1 + 1, x[2]], x.batch())

    @staticmethod
    def batch_sum(x):
        return x.resize_batch(1)

    @staticmethod
    def slice(x, dim, lower, upper):
        # shape_ops.cc:43-53
        if lower >= upper or upper > x[dim]:
            raise Error("Invalid slice operation. shape: %s, dim: %d, lower: %d, upper: %d"
                        % (x.to_string(), dim, lower, upper))
        return x if dim >= x.depth() else x.resize_dim(dim, upper - lower)

    @staticmethod
    def concat(xs, dim):
        # shape_ops.cc:62-87
        if not xs:
            raise Error("No tensors to be concatenated.")
        s0, total = xs[0], xs[0][dim]
        for s in xs[1:]:
            if not s0.has_same_loo_dims(s, dim) or not s0.has_compatible_batch(s):
                raise Error("Invalid shapes to concatenate: " + ", ".join(x.to_string() for x in xs))
            if not s0.has_batch():
                s0 = s0.resize_batch(s.batch())
            total += s[dim]
        return s0.resize_dim(dim, total)

    @staticmethod
    def broadcast(x, dim, size):
        # shape_ops.cc:89-96
        if x[dim] != 1 or size == 0:
            raise Error("Invalid broadcasting. x: %s, dim: %d, size: %d" % (x.to_string(), dim, size))
        return x.resize_dim(dim, size)

    @staticmethod
    def pick(x, ids, dim):
        # shape_ops.cc:98-118
        n, bi = x[dim], len(ids)
        if bi == 0 or (x.batch() != bi and x.has_batch() and bi > 1):
            raise Error("Invalid IDs to pick. shape: %s, ids.size(): %d" % (x.to_string(), bi))
        for i, v in enumerate(ids):
            if v >= n:
                raise Error("Invalid IDs to pick. shape: %s, ids[%d]: %d" % (x.to_string(), i, v))
        return x.resize_dim(dim, 1).resize_batch(max(x.batch(), bi))

    @staticmethod
    def transpose(x):
        # shape_ops.cc:120-125
        if not x.is_matrix():
            raise Error("Invalid shape to transpose: " + x.to_string())
        return Shape([x[1], x[0]], x.batch())

    @staticmethod
    def permute_dims(x, perm):
        # shape_ops.cc:127-152
        if len(perm) < x.depth():
            raise Error("Invalid perm to permute. shape: %s, perm.size(): %d" % (x.to_string(), len(perm)))
        if sorted(perm) != list(range(len(perm))):
            raise Error("Invalid perm to permute. shape: %s, perm: %s" % (x.to_string(), list(perm)))
        return Shape([x[p] for p in perm], x.batch())

    @staticmethod
    def batch_pick(x, ids):
        # shape_ops.cc:216-233
        if len(ids) == 0:
            raise Error("Invalid IDs to pick. shape: %s, ids.size(): 0" % x.to_string())
        for i, v in enumerate(ids):
            if v >= x.batch():
                raise Error("Invalid IDs to pick. shape: %s, ids[%d]: %d" % (x.to_string(), i, v))
        return x.resize_batch(len(ids))

    @staticmethod
    def batch_slice(x, lower, upper):
        # shape_ops.cc:235-243
        if lower >= upper or upper > x.batch():
            raise Error("Invalid batch_slice operation. shape: %s, lower: %d, upper: %d"
                        % (x.to_string(), lower, upper))
        return x.resize_batch(upper - lower)

    @staticmethod
    def batch_concat(xs):
        # shape_ops.cc:252-274
        if not xs:
            raise Error("No tensors to be concatenated.")
        for s in xs[1:]:
            if not xs[0].has_same_dims(s):
                raise Error("Invalid shapes to concatenate minibatches: "
                            + ", ".join(x.to_string() for x in xs))
        return xs[0].resize_batch(sum(s.batch() for s in xs))

    @staticmethod
    def elementwise(a, b):
        # shape_ops.cc:34-41
        if not a.has_same_dims(b) or not a.has_compatible_batch(b):
            raise Error("Shape mismatched for the elementwise operation. a: %s != b: %s"
                        % (a.to_string(), b.to_string()))
        return a.resize_batch(max(a.batch(), b.batch()))

    @staticmethod
    def scalar_op(x, k):
        # shape_ops.cc:25-32
        if k.volume() != 1 or k.depth() != 0 or not x.has_compatible_batch(k):
            raise Error("Shape mismatched for the scalar operation. x: %s != k: %s"
                        % (x.to_string(), k.to_string()))
        return x.resize_batch(max(x.batch(), k.batch()))


class _Handle:
    """One pool block; returned to the pool of its context when dropped,
    silently if that context is already gone (primitiv/core/memory_pool.h:22-35)."""

    __slots__ = ("ptr", "ctx_id", "allocated", "sharers")

    def __init__(self, ptr, ctx_id, allocated):
        self.ptr, self.ctx_id, self.allocated = ptr, ctx_id, allocated
        self.sharers = 0  # tensors that currently refer to this block

    def __del__(self):
        try:
            if self.ptr:
                _lib.lib().phip_pool_free_by_id(self.ctx_id, self.ptr)
        except Exception:
            pass


class Tensor:
    """Value handle with copy-on-write sharing (primitiv/core/tensor.{h,cc})."""

    def __init__(self, shape=None, device=None, handle=None):
        self._shape = shape
        self._device = device
        self._handle = handle
        if handle is not None:
            handle.sharers += 1

    def __del__(self):
        if getattr(self, "_handle", None) is not None:
            self._handle.sharers -= 1

    def valid(self):
        return self._handle is not None

    def _check_valid(self):
        if not self.valid():
            raise Error("Invalid tensor.")

    def shape(self):
        self._check_valid()
        return self._shape

    def device(self):
        self._check_valid()
        return self._device

    def allocated_size(self):
        self._check_valid()
        return self._handle.allocated

    def handle(self):
        self._check_valid()
        return self._handle.ptr

    def mutable_handle(self):
        """Raw pointer for writing; clones the block first when it is shared
        (tensor.cc:33-41)."""
        self._check_valid()
        if self._handle.sharers > 1:
            clone = self._device.copy_tensor(self)
            self._handle.sharers -= 1
            self._handle = clone._handle
            self._handle.sharers += 1
        return self._handle.ptr

    def copy(self):
        """Copy construction: shares the handle until one side is written."""
        return Tensor(self._shape, self._device, self._handle)

    def to_vector(self):
        self._check_valid()
        return self._device.tensor_to_vector(self)

    def to_float(self):
        self._check_valid()
        if self._shape.size() != 1:
            raise Error("Tensor has more than 1 values. shape = " + self._shape.to_string())
        return float(self.to_vector()[0])

    def inplace_add(self, x):
        self._check_valid()
        self._device.inplace_add(x, self)
        return self

    __iadd__ = inplace_add


class DeviceType:
    # the reference's enum (primitiv/core/device.h:17-35) extended by one group
    GROUP_HIP = 0x00030000
    HIP = 0x00030000
    HIP16 = 0x00030001


class HIP:
    """fp32 device (mirrors primitiv::devices::CUDA's public face,
    primitiv/devices/cuda/device.h:27-62, for the calls on the matmul path)."""

    _SUFFIX = "f32"
    _ITEMSIZE = 4

    @staticmethod
    def num_devices():
        n = ctypes.c_int(0)
        _lib.call("phip_device_count", ctypes.byref(n))
        return n.value

    @staticmethod
    def assert_support(device_id):
        _lib.call("phip_check_support", int(device_id))

    @staticmethod
    def check_support(device_id):
        try:
            HIP.assert_support(device_id)
        except Error:
            return False
        return True

    def __init__(self, device_id, rng_seed=None):
        if device_id < 0:
            raise Error("Invalid device ID: %d" % device_id)
        self._ctx = ctypes.c_void_p()
        _lib.call("phip_ctx_create", int(device_id), ctypes.byref(self._ctx))
        self._ctx_id = _lib.lib().phip_ctx_id(self._ctx)
        self._device_id = int(device_id)
        # devices/cuda/device.cc: without a seed the generator is seeded from std::random_device
        self._rng_seed = int.from_bytes(os.urandom(8), "little") if rng_seed is None else int(rng_seed)
        self._rng_offset = 0   # position in the Philox stream, in blocks of four draws

    def close(self):
        if self._ctx:
            ctx, self._ctx = self._ctx, None
            _lib.call("phip_ctx_destroy", ctx)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- identity ---------------------------------------------------------
    def type(self):
        return DeviceType.HIP

    def ctx(self):
        return self._ctx

    def info(self):
        out = _lib.DeviceInfo()
        _lib.call("phip_device_info_get", self._ctx, ctypes.byref(out))
        return out

    def dump_description(self):
        buf = ctypes.create_string_buffer(2048)
        _lib.call("phip_describe", self._ctx, buf, len(buf))
        return buf.value.decode()

    def sync(self):
        _lib.call("phip_sync", self._ctx)

    def set_deterministic(self, on=True):
        """Gradients of split products are added in a fixed order (same bits on every run)."""
        _lib.call("phip_set_deterministic", self._ctx, 1 if on else 0)

    def set_overlap(self, on=True):
        """Matmul calls that do not touch each other's operands may run on two streams at once (the
        default); off: every launch on one stream."""
        _lib.call("phip_set_overlap", self._ctx, 1 if on else 0)

    def set_deferred_zero_fill(self, on=True):
        """Zero fills are noted and folded into the gradient operation that follows (the default);
        off: every fill is launched when it is asked for."""
        _lib.call("phip_set_deferred_zero_fill", self._ctx, 1 if on else 0)

    def gemm_trace(self, on=True):
        """Names of the GEMM kernels that this device's matmul calls went to since the previous call
        (a list, launch order per stream); `on` switches the note-taking on or off from here on."""
        buf = ctypes.create_string_buffer(1 << 16)
        _lib.call("phip_gemm_trace", self._ctx, 1 if on else 0, buf, len(buf))
        return buf.value.decode().split()

    # -- storage ----------------------------------------------------------
    def _elements_to_bytes(self, n):
        return self._ITEMSIZE * n

    def new_raw_tensor(self, shape):
        # device.cc:20-24 -> new_handle (devices/cuda/ops/new_handle.cu:10-12)
        shape = _as_shape(shape)
        ptr = ctypes.c_void_p()
        allocated = ctypes.c_size_t(0)
        _lib.call("phip_pool_alloc", self._ctx, self._elements_to_bytes(shape.size()),
                  ctypes.byref(ptr), ctypes.byref(allocated))
        return Tensor(shape, self, _Handle(ptr.value, self._ctx_id, allocated.value))

    def _check_device(self, x):
        # device.cc:11-16
        if x.device() is not self:
            raise Error("Device mismatched.")

    def _upload(self, ptr, host):
        _lib.call("phip_memcpy_h2d", self._ctx, ptr, host.ctypes.data, host.nbytes)

    def _download(self, ptr, n):
        out = np.empty(n, dtype=np.float32)
        _lib.call("phip_memcpy_d2h", self._ctx, out.ctypes.data, ptr, out.nbytes)
        return out

    def new_tensor_by_constant(self, shape, k):
        ret = self.new_raw_tensor(shape)
        self.reset_tensor(k, ret)
        return ret

    def new_tensor_by_array(self, shape, values):
        ret = self.new_raw_tensor(shape)
        self.reset_tensor_by_array(values, ret)
        return ret

    def new_tensor_by_vector(self, shape, values):
        # device.cc:42-49
        shape = _as_shape(shape)
        values = np.ascontiguousarray(np.asarray(values, dtype=np.float32).reshape(-1))
        if values.size != shape.size():
            raise Error("Data sizes mismatched. required: %d (%s) != actual: %d"
                        % (shape.size(), shape.to_string(), values.size))
        return self.new_tensor_by_array(shape, values)

    def reset_tensor(self, k, x):
        self._check_device(x)
        _lib.call("phip_fill_" + self._SUFFIX, self._ctx, x.mutable_handle(), float(k), x.shape().size())

    def reset_tensor_by_array(self, values, x):
        self._check_device(x)
        values = np.ascontiguousarray(np.asarray(values, dtype=np.float32).reshape(-1))
        n = x.shape().size()
        if values.size < n:
            raise Error("host array is shorter than the tensor")
        self._upload(x.mutable_handle(), values[:n])

    def tensor_to_vector(self, x):
        self._check_device(x)
        return self._download(x.handle(), x.shape().size())

    def copy_tensor(self, x):
        # devices/cuda/ops/copy_tensor.cu:10-30.  Within one device the copy is
        # ordered by the device's stream.  Between two devices on the same GPU
        # (each has a stream of its own) the source is drained first and the
        # copy, or the storage conversion, runs on the GPU; the destination is
        # drained afterwards so that the source may be released at once.
        # Anything else bounces through the host.
        ret = self.new_raw_tensor(x.shape())
        src = x.device()
        n = x.shape().size()
        if src is self:
            _lib.call("phip_memcpy_d2d", self._ctx, ret._handle.ptr, x.handle(), self._elements_to_bytes(n))
        elif isinstance(src, HIP) and src._device_id == self._device_id and (
                src._SUFFIX == self._SUFFIX or "f32" in (src._SUFFIX, self._SUFFIX)):
            src.sync()
            if src._SUFFIX == self._SUFFIX:
                _lib.call("phip_memcpy_d2d", self._ctx, ret._handle.ptr, x.handle(), self._elements_to_bytes(n))
            else:
                _lib.call("phip_cvt_%s_to_%s" % (src._SUFFIX, self._SUFFIX), self._ctx, x.handle(),
                          ret._handle.ptr, n)
            self.sync()
        else:
            self.reset_tensor_by_array(x.to_vector(), ret)
        return ret

    # -- the matmul path --------------------------------------------------
    def matmul_fw(self, a, b):
        # DEV_FW_AB, device.cc:268-275,418
        self._check_device(a)
        self._check_device(b)
        y = self.new_raw_tensor(shape_ops.matmul(a.shape(), b.shape()))
        sa, sb = a.shape(), b.shape()
        _lib.call("phip_matmul_fw_" + self._SUFFIX, self._ctx, a.handle(), b.handle(),
                  y.mutable_handle(), sa[0], sa[1], sb[1], sa.batch(), sb.batch())
        return y

    def matmul_bw(self, a, b, y, gy, ga, gb):
        # DEV_BW_AB, device.cc:277-301,453
        for t in (a, b, y, gy, ga, gb):
            self._check_device(t)
        if (a.shape() != ga.shape() or b.shape() != gb.shape() or y.shape() != gy.shape()
                or y.shape() != shape_ops.matmul(a.shape(), b.shape())):
            raise Error("Shape mismatched at matmul_bw. a: %s, b: %s, y: %s, gy: %s, ga: %s, gb: %s"
                        % tuple(t.shape().to_string() for t in (a, b, y, gy, ga, gb)))
        sa, sb = a.shape(), b.shape()
        # writable pointers first: taking them may clone a shared block
        pga, pgb = ga.mutable_handle(), gb.mutable_handle()
        _lib.call("phip_matmul_bw_" + self._SUFFIX, self._ctx, a.handle(), b.handle(),
                  gy.handle(), pga, pgb, sa[0], sa[1], sb[1], sa.batch(), sb.batch())

    # -- convolution and pooling -------------------------------------------
    def conv2d_fw(self, x, w, padding0, padding1, stride0, stride1, dilation0, dilation1):
        # device.cc:420-433
        self._check_device(x)
        self._check_device(w)
        args = (padding0, padding1, stride0, stride1, dilation0, dilation1)
        y = self.new_raw_tensor(shape_ops.conv2d(x.shape(), w.shape(), *args))
        sx, sw = x.shape(), w.shape()
        _lib.call("phip_conv2d_fw_" + self._SUFFIX, self._ctx, x.handle(), w.handle(), y.mutable_handle(),
                  sx[0], sx[1], sx[2], sw[0], sw[1], sw[3], sx.batch(), sw.batch(), *args)
        return y

    def conv2d_bw(self, x, w, y, gy, padding0, padding1, stride0, stride1, dilation0, dilation1, gx, gw):
        # device.cc:455-491
        for t in (x, w, y, gy, gx, gw):
            self._check_device(t)
        args = (padding0, padding1, stride0, stride1, dilation0, dilation1)
        if (x.shape() != gx.shape() or w.shape() != gw.shape() or y.shape() != gy.shape()
                or y.shape() != shape_ops.conv2d(x.shape(), w.shape(), *args)):
            raise Error("Shape mismatched at conv2d_bw. x.shape: %s, w.shape: %s, y.shape: %s, gy.shape: %s, "
                        "gx.shape: %s, gw.shape: %s, padding0: %d, padding1: %d, stride0: %d, stride1: %d, "
                        "dilation0: %d, dilation1: %d"
                        % (tuple(t.shape().to_string() for t in (x, w, y, gy, gx, gw)) + args))
        sx, sw = x.shape(), w.shape()
        pgx, pgw = gx.mutable_handle(), gw.mutable_handle()
        _lib.call("phip_conv2d_bw_" + self._SUFFIX, self._ctx, x.handle(), w.handle(), gy.handle(), pgx, pgw,
                  sx[0], sx[1], sx[2], sw[0], sw[1], sw[3], sx.batch(), sw.batch(), *args)

    def max_pool2d_fw(self, x, window0, window1, padding0, padding1, stride0, stride1):
        # device.cc:435-446
        self._check_device(x)
        args = (window0, window1, padding0, padding1, stride0, stride1)
        y = self.new_raw_tensor(shape_ops.pool2d(x.shape(), *args))
        sx = x.shape()
        _lib.call("phip_max_pool2d_fw_" + self._SUFFIX, self._ctx, x.handle(), y.mutable_handle(), sx[0], sx[1],
                  sx.size() // (sx[0] * sx[1]), *args)
        return y

    def max_pool2d_bw(self, x, y, gy, window0, window1, padding0, padding1, stride0, stride1, gx):
        # device.cc:493-522
        for t in (x, y, gy, gx):
            self._check_device(t)
        args = (window0, window1, padding0, padding1, stride0, stride1)
        if (x.shape() != gx.shape() or y.shape() != gy.shape()
                or y.shape() != shape_ops.pool2d(x.shape(), *args)):
            raise Error("Shape mismatched at max_pool2d_bw. x.shape: %s, y.shape: %s, gy.shape: %s, gx.shape: %s, "
                        "window0: %d, window1: %d, padding0: %d, padding1: %d, stride0: %d, stride1: %d"
                        % (tuple(t.shape().to_string() for t in (x, y, gy, gx)) + args))
        sx = x.shape()
        pgx = gx.mutable_handle()
        _lib.call("phip_max_pool2d_bw_" + self._SUFFIX, self._ctx, x.handle(), y.handle(), gy.handle(), pgx, sx[0],
                  sx[1], sx.size() // (sx[0] * sx[1]), *args)

    def inplace_add(self, x, y):
        # device.cc:692-703
        self._check_device(x)
        self._check_device(y)
        sx, sy = x.shape(), y.shape()
        if not sx.has_same_dims(sy) or not sx.has_compatible_batch(sy):
            raise Error("Attempted to add values of shape %s to shape %s"
                        % (sx.to_string(), sy.to_string()))
        _lib.call("phip_inplace_add_" + self._SUFFIX, self._ctx, x.handle(), y.mutable_handle(),
                  sy.volume(), sx.batch(), sy.batch())
        return y

    def batch_sum_fw(self, x):
        self._check_device(x)
        y = self.new_raw_tensor(shape_ops.batch_sum(x.shape()))
        _lib.call("phip_batch_sum_" + self._SUFFIX, self._ctx, x.handle(), y.mutable_handle(),
                  x.shape().volume(), x.shape().batch())
        return y

    # -- elementwise operations around the matmul ------------------------------
    # Operation codes of include/phip.h.
    UNARY_OPS = ("negate", "abs", "sqrt", "exp", "log", "tanh", "sigmoid", "softplus", "sin", "cos", "tan")
    CONST_OPS = ("add_const", "subtract_const_r", "subtract_const_l", "multiply_const", "divide_const_r",
                 "divide_const_l", "pow_const_r", "pow_const_l", "prelu", "elu")
    BINARY_OPS = ("add", "subtract", "multiply", "divide", "pow")
    # scalar operation -> (binary operation, scalar on the left)
    SCALAR_OPS = {"add_scalar": ("add", False), "subtract_scalar_r": ("subtract", False),
                  "subtract_scalar_l": ("subtract", True), "multiply_scalar": ("multiply", False),
                  "divide_scalar_r": ("divide", False), "divide_scalar_l": ("divide", True),
                  "pow_scalar_r": ("pow", False), "pow_scalar_l": ("pow", True)}

    def _bw_x_check(self, name, x, y, gy, gx):
        # DEV_BW_X / DEV_BW_X_CONST, device.cc:221-266
        for t in (x, y, gy, gx):
            self._check_device(t)
        s = x.shape()
        if y.shape() != s or gy.shape() != s or gx.shape() != s:
            raise Error("Shape mismatched at %s_bw. x.shape: %s, y.shape: %s, gy.shape: %s, gx.shape: %s"
                        % ((name,) + tuple(t.shape().to_string() for t in (x, y, gy, gx))))

    def unary_fw(self, op, x):
        """`op`_fw(x) for an op of UNARY_OPS (DEV_FW_X, device.cc:213-219,303-313)."""
        self._check_device(x)
        y = self.new_raw_tensor(x.shape())
        _lib.call("phip_unary_fw_" + self._SUFFIX, self._ctx, self.UNARY_OPS.index(op), x.handle(),
                  y.mutable_handle(), x.shape().size())
        return y

    def unary_bw(self, op, x, y, gy, gx):
        self._bw_x_check(op, x, y, gy, gx)
        pgx = gx.mutable_handle()
        _lib.call("phip_unary_bw_" + self._SUFFIX, self._ctx, self.UNARY_OPS.index(op), x.handle(), y.handle(),
                  gy.handle(), pgx, x.shape().size())

    def const_fw(self, op, x, k):
        """`op`_fw(x, k) for an op of CONST_OPS (DEV_FW_X_CONST, device.cc:241-247)."""
        self._check_device(x)
        y = self.new_raw_tensor(x.shape())
        _lib.call("phip_const_fw_" + self._SUFFIX, self._ctx, self.CONST_OPS.index(op), x.handle(), float(k),
                  y.mutable_handle(), x.shape().size())
        return y

    def const_bw(self, op, x, y, gy, k, gx):
        self._bw_x_check(op, x, y, gy, gx)
        pgx = gx.mutable_handle()
        _lib.call("phip_const_bw_" + self._SUFFIX, self._ctx, self.CONST_OPS.index(op), x.handle(), y.handle(),
                  gy.handle(), float(k), pgx, x.shape().size())

    def pown_fw(self, x, k):
        self._check_device(x)
        y = self.new_raw_tensor(x.shape())
        _lib.call("phip_pown_fw_" + self._SUFFIX, self._ctx, x.handle(), int(k), y.mutable_handle(),
                  x.shape().size())
        return y

    def pown_bw(self, x, y, gy, k, gx):
        self._bw_x_check("pown", x, y, gy, gx)
        pgx = gx.mutable_handle()
        _lib.call("phip_pown_bw_" + self._SUFFIX, self._ctx, x.handle(), y.handle(), gy.handle(), int(k), pgx,
                  x.shape().size())

    def scalar_fw(self, op, x, k):
        """`op`_fw(x, k) for an op of SCALAR_OPS; k holds one scalar per sample
        (DEV_FW_AB with shape_ops::scalar_op, device.cc:404-411)."""
        self._check_device(x)
        self._check_device(k)
        y = self.new_raw_tensor(shape_ops.scalar_op(x.shape(), k.shape()))
        binary, left = self.SCALAR_OPS[op]
        _lib.call("phip_scalar_fw_" + self._SUFFIX, self._ctx, self.BINARY_OPS.index(binary), int(left),
                  x.handle(), k.handle(), y.mutable_handle(), x.shape().volume(), x.shape().batch(),
                  k.shape().batch())
        return y

    def binary_fw(self, op, a, b):
        """`op`_fw(a, b) for an op of BINARY_OPS (DEV_FW_AB, device.cc:268-275,413-417)."""
        self._check_device(a)
        self._check_device(b)
        y = self.new_raw_tensor(shape_ops.elementwise(a.shape(), b.shape()))
        _lib.call("phip_binary_fw_" + self._SUFFIX, self._ctx, self.BINARY_OPS.index(op), a.handle(), b.handle(),
                  y.mutable_handle(), y.shape().volume(), a.shape().batch(), b.shape().batch())
        return y

    def binary_bw(self, op, a, b, y, gy, ga, gb):
        # DEV_BW_AB, device.cc:277-301,448-452
        for t in (a, b, y, gy, ga, gb):
            self._check_device(t)
        if (a.shape() != ga.shape() or b.shape() != gb.shape() or y.shape() != gy.shape()
                or y.shape() != shape_ops.elementwise(a.shape(), b.shape())):
            raise Error("Shape mismatched at %s_bw. a: %s, b: %s, y: %s, gy: %s, ga: %s, gb: %s"
                        % ((op,) + tuple(t.shape().to_string() for t in (a, b, y, gy, ga, gb))))
        pga, pgb = ga.mutable_handle(), gb.mutable_handle()
        _lib.call("phip_binary_bw_" + self._SUFFIX, self._ctx, self.BINARY_OPS.index(op), a.handle(), b.handle(),
                  y.handle(), gy.handle(), pga, pgb, y.shape().volume(), a.shape().batch(), b.shape().batch())

    def inplace_multiply_const(self, k, x):
        # device.cc:687-690
        self._check_device(x)
        _lib.call("phip_inplace_multiply_const_" + self._SUFFIX, self._ctx, float(k), x.mutable_handle(),
                  x.shape().size())
        return x

    def inplace_subtract(self, x, y):
        # device.cc:705-716
        self._check_device(x)
        self._check_device(y)
        sx, sy = x.shape(), y.shape()
        if not sx.has_same_dims(sy) or not sx.has_compatible_batch(sy):
            raise Error("Attempted to subtract values of shape %s from shape %s"
                        % (sx.to_string(), sy.to_string()))
        _lib.call("phip_inplace_subtract_" + self._SUFFIX, self._ctx, x.handle(), y.mutable_handle(),
                  sy.volume(), sx.batch(), sy.batch())
        return y

    def identity(self, size):
        # device.cc:98-105
        if size == 0:
            raise Error("Invalid size of the identity matrix. size: 0")
        y = self.new_raw_tensor(Shape([size, size]))
        _lib.call("phip_identity_" + self._SUFFIX, self._ctx, y.mutable_handle(), size)
        return y

    # -- moving and reducing along one dimension --------------------------------
    REDUCE_OPS = ("sum", "logsumexp", "max", "min")

    @staticmethod
    def _u32(values):
        values = [int(v) for v in values]
        return (ctypes.c_uint32 * max(1, len(values)))(*values), len(values)

    def _copy_rows(self, src, dst, span, rows, ss, ds, bs, sbs, dbs, accumulate):
        _lib.call("phip_copy_rows_" + self._SUFFIX, self._ctx, src, dst, span, rows, ss, ds, bs, sbs, dbs,
                  int(accumulate))

    def _at(self, ptr, elements):
        """Device address `elements` elements past ptr."""
        return ptr + elements * self._ITEMSIZE

    def slice_fw(self, x, dim, lower, upper):
        # device.cc:157-164; devices/cuda/ops/slice.cu:26-37
        self._check_device(x)
        y = self.new_raw_tensor(shape_ops.slice(x.shape(), dim, lower, upper))
        sx, sy = x.shape(), y.shape()
        base = sy.lower_volume(dim)
        span, skip = base * sy[dim], base * sx[dim]
        self._copy_rows(self._at(x.handle(), base * lower), y.mutable_handle(), span, sy.size() // span,
                        skip, span, 1, 0, 0, False)
        return y

    def slice_bw(self, gy, dim, offset, gx):
        # device.cc:195-211; devices/cuda/ops/slice.cu:39-55
        self._check_device(gy)
        self._check_device(gx)
        sy, sx = gy.shape(), gx.shape()
        if (not sy.has_same_loo_dims(sx, dim) or not sy.has_compatible_batch(sx)
                or offset + sy[dim] > sx[dim]):
            raise Error("Attempted to add gradients with shape %s, dim %d, offset %d to shape%s."
                        % (sy.to_string(), dim, offset, sx.to_string()))
        if dim >= sx.depth():
            return self.inplace_add(gy, gx)
        base = sx.lower_volume(dim)
        span, skip = base * sy[dim], base * sx[dim]
        pgx = gx.mutable_handle()
        self._copy_rows(gy.handle(), self._at(pgx, base * offset), span, sx.volume() // skip, span, skip,
                        max(sx.batch(), sy.batch()), sy.volume() if sy.has_batch() else 0,
                        sx.volume() if sx.has_batch() else 0, True)

    def concat_fw(self, xs, dim):
        # device.cc:166-179; devices/cuda/ops/concat.cu:20-40
        if not xs:
            raise Error("No tensors to concat.")
        for x in xs:
            self._check_device(x)
        y = self.new_raw_tensor(shape_ops.concat([x.shape() for x in xs], dim))
        sy = y.shape()
        base = sy.lower_volume(dim)
        skip = base * sy[dim]
        repeat = sy.volume() // skip
        py, offset = y.mutable_handle(), 0
        for x in xs:
            span = base * x.shape()[dim]
            self._copy_rows(x.handle(), self._at(py, offset), span, repeat, span, skip, sy.batch(),
                            x.shape().volume() if x.shape().has_batch() else 0, sy.volume(), False)
            offset += span
        return y

    def pick_fw(self, x, ids, dim):
        # device.cc:150-155
        self._check_device(x)
        y = self.new_raw_tensor(shape_ops.pick(x.shape(), ids, dim))
        sx = x.shape()
        base = sx.lower_volume(dim)
        arr, n = self._u32(ids)
        _lib.call("phip_pick_fw_" + self._SUFFIX, self._ctx, x.handle(), arr, n, y.mutable_handle(), base,
                  sx[dim], sx.volume() // (base * sx[dim]), sx.batch(), y.shape().batch())
        return y

    def pick_bw(self, gy, ids, dim, gx):
        # device.cc:181-193
        self._check_device(gy)
        self._check_device(gx)
        sx = gx.shape()
        sy = shape_ops.pick(sx, ids, dim)
        if gy.shape() != sy:
            raise Error("Shape mismatched. gy.shape(): %s != expected shape: %s"
                        % (gy.shape().to_string(), sy.to_string()))
        base = sx.lower_volume(dim)
        arr, n = self._u32(ids)
        pgx = gx.mutable_handle()
        _lib.call("phip_pick_bw_" + self._SUFFIX, self._ctx, gy.handle(), arr, n, pgx, base, sx[dim],
                  sx.volume() // (base * sx[dim]), sx.batch(), sy.batch())

    def batch_pick_fw(self, x, ids):
        # device.cc:616-622
        self._check_device(x)
        y = self.new_raw_tensor(shape_ops.batch_pick(x.shape(), ids))
        arr, n = self._u32(ids)
        _lib.call("phip_batch_pick_fw_" + self._SUFFIX, self._ctx, x.handle(), arr, n, y.mutable_handle(),
                  x.shape().volume(), x.shape().batch())
        return y

    def batch_pick_bw(self, gy, ids, gx):
        # device.cc:653-664
        self._check_device(gy)
        self._check_device(gx)
        sy = shape_ops.batch_pick(gx.shape(), ids)
        if gy.shape() != sy:
            raise Error("Shape mismatched. gy.shape(): %s != expected shape: %s"
                        % (gy.shape().to_string(), sy.to_string()))
        arr, n = self._u32(ids)
        pgx = gx.mutable_handle()
        _lib.call("phip_batch_pick_bw_" + self._SUFFIX, self._ctx, gy.handle(), arr, n, pgx,
                  gx.shape().volume(), gx.shape().batch())

    def batch_slice_fw(self, x, lower, upper):
        # device.cc:624-630
        self._check_device(x)
        y = self.new_raw_tensor(shape_ops.batch_slice(x.shape(), lower, upper))
        vol = y.shape().volume()
        self._copy_rows(self._at(x.handle(), vol * lower), y.mutable_handle(), vol, y.shape().batch(), vol, vol,
                        1, 0, 0, False)
        return y

    def batch_slice_bw(self, gy, offset, gx):
        # device.cc:666-679
        self._check_device(gy)
        self._check_device(gx)
        sy, sx = gy.shape(), gx.shape()
        if not sy.has_same_dims(sx) or offset + sy.batch() > sx.batch():
            raise Error("Attempted to add gradients with shape %s, batch offset %d to shape%s."
                        % (sy.to_string(), offset, sx.to_string()))
        vol = sy.volume()
        pgx = gx.mutable_handle()
        self._copy_rows(gy.handle(), self._at(pgx, vol * offset), vol, sy.batch(), vol, vol, 1, 0, 0, True)

    def batch_concat_fw(self, xs):
        # device.cc:632-644
        if not xs:
            raise Error("No tensors to concat.")
        for x in xs:
            self._check_device(x)
        y = self.new_raw_tensor(shape_ops.batch_concat([x.shape() for x in xs]))
        vol = y.shape().volume()
        py, offset = y.mutable_handle(), 0
        for x in xs:
            self._copy_rows(x.handle(), self._at(py, offset), vol, x.shape().batch(), vol, vol, 1, 0, 0, False)
            offset += x.shape().size()
        return y

    def transpose_fw(self, x):
        # DEV_FW_X(transpose, shape_ops::transpose), device.cc:314
        self._check_device(x)
        y = self.new_raw_tensor(shape_ops.transpose(x.shape()))
        _lib.call("phip_transpose_fw_" + self._SUFFIX, self._ctx, x.handle(), y.mutable_handle(), x.shape()[0],
                  x.shape()[1], x.shape().batch())
        return y

    def transpose_bw(self, x, y, gy, gx):
        # DEV_BW_X(transpose, shape_ops::transpose), device.cc:334
        for t in (x, y, gy, gx):
            self._check_device(t)
        if (x.shape() != gx.shape() or y.shape() != gy.shape()
                or y.shape() != shape_ops.transpose(x.shape())):
            raise Error("Shape mismatched at transpose_bw. x.shape: %s, y.shape: %s, gy.shape: %s, gx.shape: %s"
                        % tuple(t.shape().to_string() for t in (x, y, gy, gx)))
        pgx = gx.mutable_handle()
        _lib.call("phip_transpose_bw_" + self._SUFFIX, self._ctx, gy.handle(), pgx, gx.shape()[0],
                  gx.shape()[1], gx.shape().batch())

    def permute_dims_fw(self, x, perm):
        # device.cc:316-322
        self._check_device(x)
        y = self.new_raw_tensor(shape_ops.permute_dims(x.shape(), perm))
        dims, n = self._u32([x.shape()[i] for i in range(len(perm))])
        pm, _ = self._u32(perm)
        _lib.call("phip_permute_dims_fw_" + self._SUFFIX, self._ctx, x.handle(), y.mutable_handle(), n, dims, pm,
                  x.shape().batch())
        return y

    def permute_dims_bw(self, x, y, gy, perm, gx):
        # device.cc:336-354
        for t in (x, y, gy, gx):
            self._check_device(t)
        sy = shape_ops.permute_dims(x.shape(), perm)
        if y.shape() != sy or gy.shape() != sy or gx.shape() != x.shape():
            raise Error("Shape mismatched at permute_dims_bw. x.shape: %s, y.shape: %s, gy.shape: %s, gx.shape: %s"
                        % tuple(t.shape().to_string() for t in (x, y, gy, gx)))
        dims, n = self._u32([x.shape()[i] for i in range(len(perm))])
        pm, _ = self._u32(perm)
        pgx = gx.mutable_handle()
        _lib.call("phip_permute_dims_bw_" + self._SUFFIX, self._ctx, gy.handle(), pgx, n, dims, pm,
                  x.shape().batch())

    def _around(self, s, dim):
        """(base, n, outer) of shape s seen around dimension dim."""
        base = s.lower_volume(dim)
        return base, s[dim], s.size() // (base * s[dim])

    def flip_fw(self, x, dim):
        # device.cc:530-535
        self._check_device(x)
        y = self.new_raw_tensor(x.shape())
        _lib.call("phip_flip_fw_" + self._SUFFIX, self._ctx, x.handle(), y.mutable_handle(),
                  *self._around(x.shape(), dim))
        return y

    def flip_bw(self, gy, dim, gx):
        # device.cc:537-547
        self._check_device(gy)
        self._check_device(gx)
        if gy.shape() != gx.shape():
            raise Error("Shape mismatched. gy.shape(): %s != expected shape: %s"
                        % (gy.shape().to_string(), gx.shape().to_string()))
        pgx = gx.mutable_handle()
        _lib.call("phip_flip_bw_" + self._SUFFIX, self._ctx, gy.handle(), pgx, *self._around(gx.shape(), dim))

    def reduce_fw(self, op, x, dim):
        """sum_fw / logsumexp_fw / max_fw / min_fw along dim (device.cc:549-561,597-609)."""
        self._check_device(x)
        y = self.new_raw_tensor(x.shape().resize_dim(dim, 1))
        _lib.call("phip_reduce_fw_" + self._SUFFIX, self._ctx, self.REDUCE_OPS.index(op), x.handle(),
                  y.mutable_handle(), *self._around(x.shape(), dim))
        return y

    def extremum_bw(self, op, x, y, gy, dim, gx):
        """max_bw / min_bw (device.cc:563-595)."""
        for t in (x, y, gy, gx):
            self._check_device(t)
        r = x.shape()
        s = r.resize_dim(dim, 1)
        if gx.shape() != r or y.shape() != s or gy.shape() != s:
            raise Error("Shape mismatched at %s_bw(dim=%d). x.shape: %s, y.shape: %s, gy.shape: %s, gx.shape: %s"
                        % ((op, dim) + tuple(t.shape().to_string() for t in (x, y, gy, gx))))
        pgx = gx.mutable_handle()
        _lib.call("phip_extremum_bw_" + self._SUFFIX, self._ctx, self.REDUCE_OPS.index(op), x.handle(),
                  y.handle(), gy.handle(), pgx, *self._around(r, dim))

    def arg_extremum(self, op, x, dim):
        """argmax / argmin along dim as a list of indices (device.cc:56-64)."""
        self._check_device(x)
        base, n, outer = self._around(x.shape(), dim)
        out = (ctypes.c_uint32 * max(1, base * outer))()
        _lib.call("phip_arg_extremum_" + self._SUFFIX, self._ctx, self.REDUCE_OPS.index(op), x.handle(), out,
                  base, n, outer)
        return list(out[:base * outer])

    def broadcast_fw(self, x, dim, size):
        # device.cc:611-616
        self._check_device(x)
        y = self.new_raw_tensor(shape_ops.broadcast(x.shape(), dim, size))
        base = y.shape().lower_volume(dim)
        _lib.call("phip_broadcast_fw_" + self._SUFFIX, self._ctx, x.handle(), y.mutable_handle(), base, size,
                  x.shape().size() // base)
        return y

    # -- random tensors ---------------------------------------------------------
    def _random(self, kind, shape, *params):
        y = self.new_raw_tensor(shape)
        n = y.shape().size()
        _lib.call("phip_random_%s_%s" % (kind, self._SUFFIX), self._ctx, self._rng_seed & (2 ** 64 - 1),
                  self._rng_offset, *params, y.mutable_handle(), n)
        self._rng_offset += (n + 3) // 4
        return y

    def random_bernoulli(self, shape, p):
        # device.cc:107-114
        if p < 0 or p > 1:
            raise Error("Invalid Bernoulli probability: %g" % p)
        return self._random("bernoulli", shape, float(p))

    def random_uniform(self, shape, lower, upper):
        # device.cc:116-126
        if upper < lower:
            raise Error("Invalid parameter of the uniform distribution. lower: %g, upper: %g" % (lower, upper))
        return self._random("uniform", shape, float(lower), float(upper))

    def random_normal(self, shape, mean, sd):
        # device.cc:128-137
        if sd <= 0:
            raise Error("Invalid parameter of the normal distribution. mean: %g, SD: %g" % (mean, sd))
        return self._random("normal", shape, float(mean), float(sd))

    def random_log_normal(self, shape, mean, sd):
        # device.cc:139-148
        if sd <= 0:
            raise Error("Invalid parameter of the log-normal distribution. mean: %g, SD: %g" % (mean, sd))
        return self._random("log_normal", shape, float(mean), float(sd))


class HIP16(HIP):
    """Half-storage device: 16-bit tensors on the GPU, float at the API edge,
    fp32 accumulation (the counterpart of primitiv::devices::CUDA16,
    primitiv/devices/cuda16/).  `storage` is "f16" or "bf16"."""

    _ITEMSIZE = 2

    def __init__(self, device_id, rng_seed=None, storage="f16"):
        if storage not in ("f16", "bf16"):
            raise Error("unknown storage type: %r" % (storage,))
        super().__init__(device_id, rng_seed)
        self._SUFFIX = storage

    def type(self):
        return DeviceType.HIP16

    def _elements_to_bytes(self, n):
        # element count rounded up to even (devices/cuda16/ops/new_handle.cu:10-16)
        return 2 * (n + (n & 1))

    def _staging(self, n):
        ptr = ctypes.c_void_p()
        _lib.call("phip_pool_alloc", self._ctx, 4 * n, ctypes.byref(ptr), None)
        return _Handle(ptr.value, self._ctx_id, 0)

    def _upload(self, ptr, host):
        # host floats -> pooled fp32 staging block -> 16-bit storage
        # (devices/cuda16/ops/reset_tensor_by_array.cu:19-30)
        tmp = self._staging(host.size)
        _lib.call("phip_memcpy_h2d", self._ctx, tmp.ptr, host.ctypes.data, host.nbytes)
        _lib.call("phip_cvt_f32_to_" + self._SUFFIX, self._ctx, tmp.ptr, ptr, host.size)

    def _download(self, ptr, n):
        # (devices/cuda16/ops/tensor_to_vector.cu:19-32)
        tmp = self._staging(n)
        _lib.call("phip_cvt_%s_to_f32" % self._SUFFIX, self._ctx, ptr, tmp.ptr, n)
        out = np.empty(n, dtype=np.float32)
        _lib.call("phip_memcpy_d2h", self._ctx, out.ctypes.data, tmp.ptr, out.nbytes)
        return out
