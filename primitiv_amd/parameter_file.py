"""primitiv's parameter file (a checkpoint of one trainable tensor and its
optimizer statistics) read and written through a device of this package.

The format is the reference's (primitiv/core/parameter.cc:26-57,131-213 over
primitiv/msgpack/writer.h and reader.h): a MessagePack stream of

    uint32 major (0), uint32 minor (1), uint32 datatype (0x200 = parameter),
    tensor value, uint32 number of statistics, then per statistic: str name, tensor

where a tensor is: array of uint32 dims, uint32 batch, bin of float32 values in
the host's byte order.  Integers always use the 5-byte 0xce form and the
reader accepts nothing else (reader.h:125-129), so a file written here loads
in the reference and the other way round.  Values are float32 on disk whatever
the device stores: a 16-bit device rounds on load and widens exactly on save.
"""
import struct

import numpy as np

from .device import Error, Shape

MAJOR, MINOR = 0, 1                  # primitiv/core/file_format.h:12-16
DATATYPE_PARAMETER = 0x200           # primitiv/core/file_format.h:18-24


def _u32(x):
    return b"\xce" + struct.pack(">I", x)                       # writer.h:117-125


def _str(s):
    raw = s.encode("utf-8")
    n = len(raw)                                                  # writer.h:30-55
    if n < 32:
        head = bytes([0xa0 | n])
    elif n < 1 << 8:
        head = b"\xd9" + bytes([n])
    elif n < 1 << 16:
        head = b"\xda" + struct.pack(">H", n)
    else:
        head = b"\xdb" + struct.pack(">I", n)
    return head + raw


def _bin(raw):
    n = len(raw)                                                  # writer.h:211-234
    if n < 1 << 8:
        head = b"\xc4" + bytes([n])
    elif n < 1 << 16:
        head = b"\xc5" + struct.pack(">H", n)
    elif n < 1 << 32:
        head = b"\xc6" + struct.pack(">I", n)
    else:
        raise Error("MessagePack: Can't store more than 2^32 - 1 bytes in one bin message.")
    return head + raw


def _array_head(n):
    if n < 16:                                                    # writer.h:392-411
        return bytes([0x90 | n])
    if n < 1 << 16:
        return b"\xdc" + struct.pack(">H", n)
    return b"\xdd" + struct.pack(">I", n)


def _tensor(t):
    shape = t.shape()
    dims = shape.dims()
    values = np.ascontiguousarray(t.to_vector(), dtype=np.float32)
    return (_array_head(len(dims)) + b"".join(_u32(d) for d in dims) + _u32(shape.batch())
            + _bin(values.tobytes()))


def dumps(value, stats=None):
    """The bytes of a parameter file holding `value` and the `stats` mapping."""
    stats = stats or {}
    if value.shape().has_batch():
        raise Error("The batch size of the parameter should be 1. shape: %s" % value.shape())
    out = [_u32(MAJOR), _u32(MINOR), _u32(DATATYPE_PARAMETER), _tensor(value), _u32(len(stats))]
    for name, t in stats.items():
        out.append(_str(name))
        out.append(_tensor(t))
    return b"".join(out)


def save(path, value, stats=None, with_stats=True):
    """Parameter::save (primitiv/core/parameter.cc:199-213)."""
    data = dumps(value, stats if with_stats else None)
    try:
        f = open(path, "wb")
    except OSError:
        raise Error("Could not open file: %s" % path)
    with f:
        f.write(data)


class _Reader:
    def __init__(self, data):
        self.data, self.pos = data, 0

    def take(self, n):
        if self.pos + n > len(self.data):
            raise Error("MessagePack: the stream ended inside an object.")
        out = self.data[self.pos:self.pos + n]
        self.pos += n
        return out

    def expect(self, tag):
        got = self.take(1)[0]                                     # reader.h:78-86
        if got != tag:
            raise Error("MessagePack: Next object does not have a correct type. expected: %x, observed: %x"
                        % (tag, got))

    def u32(self):
        self.expect(0xce)
        return struct.unpack(">I", self.take(4))[0]

    def sized(self, fix_mask, fix_tag, tags, what):
        tag = self.take(1)[0]
        if fix_mask and (tag & fix_mask) == fix_tag:
            return tag & ~fix_mask & 0xff
        for t, width, fmt in tags:
            if tag == t:
                return struct.unpack(fmt, self.take(width))[0]
        raise Error("MessagePack: Next object does not have the '%s' type. observed: %x" % (what, tag))

    def string(self):
        n = self.sized(0xe0, 0xa0, ((0xd9, 1, ">B"), (0xda, 2, ">H"), (0xdb, 4, ">I")), "str")
        return self.take(n).decode("utf-8")

    def binary(self):
        n = self.sized(0, 0, ((0xc4, 1, ">B"), (0xc5, 2, ">H"), (0xc6, 4, ">I")), "bin")
        return self.take(n)

    def array(self):
        return self.sized(0xf0, 0x90, ((0xdc, 2, ">H"), (0xdd, 4, ">I")), "array")

    def tensor(self, device):
        dims = [self.u32() for _ in range(self.array())]
        shape = Shape(dims, self.u32())
        raw = self.binary()
        if len(raw) != shape.size() * 4:                          # parameter.cc:33-38
            raise Error("Shape and data length mismatched. shape.size() * sizeof(float): %d != data.size(): %d"
                        % (shape.size() * 4, len(raw)))
        return device.new_tensor_by_vector(shape, np.frombuffer(raw, dtype=np.float32))


def loads(data, device, with_stats=True):
    """(value, stats) of the parameter file `data`, as tensors on `device`."""
    r = _Reader(data)
    major, minor = r.u32(), r.u32()
    if (major, minor) != (MAJOR, MINOR):                          # file_format.h:26-34
        raise Error("File version mismatched. required: %d.%d, observed: %d.%d" % (MAJOR, MINOR, major, minor))
    datatype = r.u32()
    if datatype != DATATYPE_PARAMETER:                            # file_format.h:36-44
        raise Error("Data type mismatched. required: %x, observed: %x" % (DATATYPE_PARAMETER, datatype))
    value = r.tensor(device)
    stats = {}
    for _ in range(r.u32()):                                      # parameter.cc:131-147
        name = r.string()
        t = r.tensor(device)
        if with_stats:
            stats[name] = t
    if value.shape().has_batch():
        raise Error("The batch size of the parameter should be 1. shape: %s" % value.shape())
    return value, stats


def load(path, device, with_stats=True):
    """Parameter::load (primitiv/core/parameter.cc:182-197)."""
    try:
        f = open(path, "rb")
    except OSError:
        raise Error("Could not open file: %s" % path)
    with f:
        return loads(f.read(), device, with_stats)
