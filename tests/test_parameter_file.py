"""The parameter file (checkpoint) format, host side: the bytes against the
reference writer's known answers (test/msgpack_writer_test.cc) and against an
independent MessagePack decoder, and the loader's error behaviour
(primitiv/core/parameter.cc, file_format.h, msgpack/reader.h)."""
import struct

import msgpack
import numpy as np
import pytest

import primitiv_amd as pa
from primitiv_amd import parameter_file as pf

S = pa.Shape


class HostTensor:
    def __init__(self, shape, values):
        self._shape, self._values = shape, np.asarray(values, dtype=np.float32)

    def shape(self):
        return self._shape

    def to_vector(self):
        return self._values


class HostDevice:
    """Stands in for a device: the file code only creates and reads tensors."""

    def new_tensor_by_vector(self, shape, values):
        return HostTensor(shape, np.array(values, dtype=np.float32))


def test_headers_match_the_reference_writer():
    assert pf._u32(0x12345678) == bytes([0xce, 0x12, 0x34, 0x56, 0x78])      # msgpack_writer_test.cc:71-74
    assert pf._str("") == bytes([0xa0])                                       # :111-114
    assert pf._str("1" * 31)[:1] == bytes([0xbf])                             # :121-125
    assert pf._str("1" * 32)[:2] == bytes([0xd9, 0x20])                       # :127-131
    assert pf._str("1" * 0x100)[:3] == bytes([0xda, 0x01, 0x00])              # :139-143
    assert pf._str("1" * 0x10000)[:5] == bytes([0xdb, 0, 1, 0, 0])            # :151-155
    assert pf._bin(b"") == bytes([0xc4, 0x00])                                # :157-160
    assert pf._bin(b"a" * 0xff)[:2] == bytes([0xc4, 0xff])                    # :167-171
    assert pf._bin(b"b" * 0x100)[:3] == bytes([0xc5, 0x01, 0x00])             # :173-177
    assert pf._bin(b"c" * 0xffff)[:3] == bytes([0xc5, 0xff, 0xff])            # :179-183
    assert pf._bin(b"d" * 0x10000)[:5] == bytes([0xc6, 0, 1, 0, 0])           # :185-189
    assert pf._array_head(0) == bytes([0x90]) and pf._array_head(15) == bytes([0x9f])
    assert pf._array_head(16) == bytes([0xdc, 0x00, 0x10])
    assert pf._array_head(0x10000) == bytes([0xdd, 0, 1, 0, 0])


def test_file_bytes_spelled_out():
    value = HostTensor(S([2, 2]), [1, 2, 3, 4])
    want = (bytes([0xce, 0, 0, 0, 0, 0xce, 0, 0, 0, 1, 0xce, 0, 0, 2, 0])       # version 0.1, parameter
            + bytes([0x92, 0xce, 0, 0, 0, 2, 0xce, 0, 0, 0, 2, 0xce, 0, 0, 0, 1])  # dims {2,2}, batch 1
            + bytes([0xc4, 16]) + struct.pack("<4f", 1, 2, 3, 4)
            + bytes([0xce, 0, 0, 0, 0]))                                             # no statistics
    assert pf.dumps(value) == want


def test_an_independent_decoder_reads_the_same_objects():
    rng = np.random.default_rng(0)
    value = HostTensor(S([3, 5]), rng.standard_normal(15))
    stats = {"adam-m1": HostTensor(S([3, 5]), rng.standard_normal(15)), "n": HostTensor(S([]), [7])}
    up = msgpack.Unpacker(raw=False)
    up.feed(pf.dumps(value, stats))
    objs = list(up)
    assert objs[:3] == [0, 1, 0x200]
    assert objs[3:5] == [[3, 5], 1]
    assert np.array_equal(np.frombuffer(objs[5], dtype=np.float32), value.to_vector())
    assert objs[6] == 2
    assert objs[7] == "adam-m1" and objs[8:10] == [[3, 5], 1]
    assert np.array_equal(np.frombuffer(objs[10], dtype=np.float32), stats["adam-m1"].to_vector())
    assert objs[11] == "n" and objs[12:14] == [[], 1] and len(objs) == 15


def test_round_trip_and_with_stats_flag(tmp_path):
    dev = HostDevice()
    rng = np.random.default_rng(1)
    value = HostTensor(S([4, 3, 2]), rng.standard_normal(24))
    stats = {"a": HostTensor(S([4, 3, 2]), rng.standard_normal(24)), "b" * 40: HostTensor(S([2]), [1, 2])}
    path = str(tmp_path / "p.data")
    pf.save(path, value, stats)
    v, st = pf.load(path, dev)
    assert v.shape() == S([4, 3, 2]) and np.array_equal(v.to_vector(), value.to_vector())
    assert sorted(st) == sorted(stats)
    for k in stats:
        assert st[k].shape() == stats[k].shape() and np.array_equal(st[k].to_vector(), stats[k].to_vector())
    v, st = pf.load(path, dev, with_stats=False)          # parameter_test.cc:345-364
    assert st == {} and np.array_equal(v.to_vector(), value.to_vector())
    pf.save(path, value, stats, with_stats=False)         # parameter_test.cc:324-343
    v, st = pf.load(path, dev)
    assert st == {}


def test_errors(tmp_path):
    dev = HostDevice()
    good = pf.dumps(HostTensor(S([2]), [1, 2]))
    with pytest.raises(pa.Error, match="version"):
        pf.loads(pf._u32(1) + good[5:], dev)
    with pytest.raises(pa.Error, match="Data type"):
        pf.loads(good[:10] + pf._u32(0x100) + good[15:], dev)
    with pytest.raises(pa.Error, match="correct type"):
        pf.loads(bytes([0xcc, 0]) + good[5:], dev)           # a shorter integer form is not accepted
    with pytest.raises(pa.Error, match="length mismatched"):
        pf.loads(good.replace(bytes([0xc4, 8]), bytes([0xc4, 4]), 1)[:-9] + pf._u32(0), dev)
    with pytest.raises(pa.Error, match="ended"):
        pf.loads(good[:-3], dev)
    with pytest.raises(pa.Error, match="Could not open"):
        pf.load(str(tmp_path / "missing" / "file"), dev)
    with pytest.raises(pa.Error, match="Could not open"):
        pf.save(str(tmp_path / "missing" / "file"), HostTensor(S([2]), [1, 2]))
    with pytest.raises(pa.Error, match="batch size"):
        pf.dumps(HostTensor(S([2], 3), np.zeros(6)))
