"""Every pure virtual of primitiv::Device must be overridden by the C++ classes.
Runs only where the reference tree and g++ are present (never on a GPU box).
The class itself is compiled with -Wall -Wextra -Werror, linked and run by
test_host_class_runs.py."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = os.environ.get("PRIMITIV_SOURCE_DIR", "/root/reference")


@pytest.mark.skipif(not os.path.isdir(os.path.join(REF, "primitiv", "core")) or not shutil.which("g++"),
                    reason="needs the primitiv source tree and g++")
def test_every_pure_virtual_is_overridden(tmp_path):
    """Constructing the classes only compiles if none of Device's pure virtuals
    (primitiv/core/device.h:368-534) is left without an override."""
    src = tmp_path / "instantiate.cc"
    src.write_text("#include <primitiv/devices/hip/device.h>\n"
                   "void make() { primitiv::devices::HIP a(0); primitiv::devices::HIP16 b(0, 1); }\n")
    cmd = ["g++", "-std=c++11", "-Wall", "-Wextra", "-Werror", "-fsyntax-only",
           "-I" + REF, "-I" + os.path.join(ROOT, "primitiv_amd"), "-I" + os.path.join(ROOT, "include"), str(src)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
