"""The C++ devices::HIP class must compile, warning-free, against the real
primitiv headers.  Runs only where the reference tree and g++ are present (it
is never available on a GPU box); nothing is linked or executed."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = os.environ.get("PRIMITIV_SOURCE_DIR", "/root/reference")


@pytest.mark.skipif(not os.path.isdir(os.path.join(REF, "primitiv", "core")) or not shutil.which("g++"),
                    reason="needs the primitiv source tree and g++")
def test_hip_device_class_compiles_against_primitiv_headers():
    src = os.path.join(ROOT, "primitiv_amd", "primitiv", "devices", "hip", "device.cc")
    cmd = ["g++", "-std=c++11", "-Wall", "-Wextra", "-Werror", "-fsyntax-only",
           "-I" + REF, "-I" + os.path.join(ROOT, "primitiv_amd"), "-I" + os.path.join(ROOT, "include"), src]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr


def test_every_pure_virtual_is_overridden():
    """Counts the pure virtuals of Device in the reference header (when it is
    there) and checks that the class names each of them."""
    hdr = os.path.join(REF, "primitiv", "core", "device.h")
    if not os.path.exists(hdr):
        pytest.skip("primitiv source tree not present")
    import re
    text = open(hdr).read()
    names = re.findall(r"virtual\s+[\w:<>\s\*&]+?\b(\w+)\s*\([^;]*?\)\s*(?:const\s*)?=\s*0\s*;", text, flags=re.S)
    assert len(names) >= 100
    mine = open(os.path.join(ROOT, "primitiv_amd", "primitiv", "devices", "hip", "device.h")).read()
    # macro-generated overrides are spelled NAME(stem[, ...]) -> stem_fw_impl / stem_bw_impl / stem_impl
    expanded = set(re.findall(r"\b(\w+_impl|new_handle|dump_description|type)\s*\(", mine))
    for macro, forms in (("PHIP_NI_X", ["%s_impl"]), ("PHIP_NI_X_BW", ["%s_impl"]),
                         ("PHIP_NI_CONST", ["%s_fw_impl", "%s_bw_impl"]), ("PHIP_NI_SCALAR", ["%s_fw_impl"]),
                         ("PHIP_NI_AB", ["%s_fw_impl", "%s_bw_impl"]), ("PHIP_NI_DIM", ["%s_fw_impl"]),
                         ("PHIP_NI_DIM_BW", ["%s_bw_impl"]), ("PHIP_NI_RANDOM", ["random_%s_impl"])):
        for stem in re.findall(r"\b%s\((\w+)" % macro, mine):
            for f in forms:
                expanded.add(f % stem)
    missing = [n for n in names if n not in expanded]
    assert not missing, missing
