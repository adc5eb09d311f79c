"""Host-side checks that need no GPU: the C ABI loads and exports what the
header declares, the seeded-input generator reproduces the reference's golden
vectors, and the shape rules of the Python mirror follow the reference."""
import ctypes
import os
import re

import numpy as np
import pytest

import primitiv_amd as pa
from primitiv_amd import _lib
from primitiv_amd.configs import WORKLOADS, Randomizer
from util import vector_match

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "phip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(phip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert len(names) >= 45
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), "libphip.so does not export " + n
    # and the binding knows every one of them
    assert set(names) == set(_lib.SIGNATURES)


@pytest.mark.parametrize("compiler,std,lang", [("gcc", "-std=c99", "c"), ("g++", "-std=c++11", "c++")])
def test_header_is_plain_c_and_cxx(tmp_path, compiler, std, lang):
    """The boundary is a C ABI: the header must compile on its own as strict C99
    (what cgo / ctypes-style bindings parse) and as C++11 (what primitiv uses)."""
    import shutil
    import subprocess
    if not shutil.which(compiler):
        pytest.skip(compiler + " not installed")
    src = tmp_path / "include_only.c"
    src.write_text('#include "phip.h"\nint main(void) { return 0; }\n')
    cmd = [compiler, std, "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-x", lang,
           "-I" + os.path.join(ROOT, "include"), str(src)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr


def test_status_and_message_without_gpu():
    l = _lib.lib()
    assert l.phip_sync(None) == _lib.PHIP_ERR_INVALID_ARGUMENT
    assert b"null context" in l.phip_last_error()
    assert l.phip_pool_free_by_id(123456789, ctypes.c_void_p(16)) == _lib.PHIP_OK  # dead pool: silent
    with pytest.raises(pa.Error):
        pa.HIP(-1)
    n = ctypes.c_int(-1)
    assert l.phip_device_count(ctypes.byref(n)) == _lib.PHIP_OK and n.value >= 0


def test_randomizer_golden(golden):
    g = golden["randomizer_seed_12345"]
    u = Randomizer(12345).uniform(g["uniform"]["lower"], g["uniform"]["upper"], 8)
    assert vector_match(g["uniform"]["expected"], u)
    nrm = Randomizer(12345).normal(g["normal"]["mean"], g["normal"]["sd"], 8)
    assert vector_match(g["normal"]["expected"], nrm)
    # (lower, upper]: the open end is the lower one (primitiv/core/random.h:49-57)
    u = Randomizer(1).uniform(0.0, 1.0, 200000)
    assert u.min() > 0.0 and u.max() <= 1.0
    # one stream per generator: two fills continue it
    r = Randomizer(12345)
    first = r.uniform(-9, 9, 4)
    second = r.uniform(-9, 9, 4)
    assert vector_match(g["uniform"]["expected"], np.concatenate([first, second]))


def test_shape_rules_golden(golden):
    for c in golden["shape_matmul_valid"]["cases"]:
        for ba, bb in ((1, 1), (3, 1), (1, 3), (3, 3)):
            got = pa.shape_ops.matmul(pa.Shape(c["a"], ba), pa.Shape(c["b"], bb))
            assert got == pa.Shape(c["y"], max(ba, bb)), c
    for c in golden["shape_matmul_invalid"]["cases"]:
        with pytest.raises(pa.Error):
            pa.shape_ops.matmul(pa.Shape(c["a"], c["ba"]), pa.Shape(c["b"], c["bb"]))
    s = pa.Shape([3, 1, 1], 2)
    assert s.depth() == 1 and s[0] == 3 and s[5] == 1 and s.size() == 6 and s.to_string() == "[3]x2"


def test_workload_table_matches_published_work():
    # flops and bytes per fw+bw call, as tabulated for the five workloads
    expect = {"dense": (0.1541, 5.079), "rnn_gate": (0.4027, 18.35),
              "square_batched": (103.08, 671.1), "output_projection": (2.496, 109.8),
              "half_storage": (3298.5, 1744.8)}
    for name, (gf, mb) in expect.items():
        w = WORKLOADS[name]
        assert abs(w.flops_per_step() / 1e9 - gf) / gf < 1e-3
        assert abs(w.bytes_per_step() / 1e6 - mb) / mb < 1e-3
