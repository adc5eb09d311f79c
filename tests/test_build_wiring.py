"""The PRIMITIV_USE_HIP build wiring: the edits a maintainer makes to primitiv's tree to add the backend
(sources copied in, the CMake option, the two CMake fragments included, the config macro, the umbrella headers)
are applied to a scratch copy of primitiv, the copy is configured with the option on and built
(hipcc cross-compiles gfx950 without a GPU), and a C program against the three libraries asks the C
API for a HIP device.  Skipped where the primitiv source tree is absent (any GPU box)."""
import os
import re
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFERENCE = os.environ.get("PRIMITIV_SOURCE_DIR", "/root/reference")
BACKEND = os.path.join(ROOT, "primitiv_amd")

sys.path.insert(0, ROOT)


def test_cmake_fragment_lists_the_sources_that_build_py_compiles():
    from primitiv_amd import build
    text = open(os.path.join(BACKEND, "primitiv", "cmake", "hip_backend.cmake")).read()
    block = text[text.index("set(phip_SRCS"):]
    listed = re.findall(r"csrc/(\w+\.hip)", block[:block.index(")")])
    assert sorted(listed) == sorted(build.SOURCES)
    assert len(set(listed)) == len(listed)
    # the flags too: same target, same optimisation level, packed-fp32 selection off in both
    for flag in ("--offload-arch=gfx950", "-O3", "-std=c++17", "-packed-fp32-ops"):
        assert flag in " ".join(build.HIPCC_FLAGS) and flag in text


def _insert(path, anchor, text, before=False, occurrence=1):
    s = open(path).read()
    at = -1
    for _ in range(occurrence):
        at = s.index(anchor, at + 1)
    at = at if before else at + len(anchor)
    with open(path, "w") as f:
        f.write(s[:at] + text + s[at:])


def apply_integration_edits(tree):
    """The six edits that add the backend to a copy of primitiv's tree (a seventh, adding the backend to its gtest suite, is not needed here)."""
    # 1. the host side next to the other backends
    shutil.copytree(os.path.join(BACKEND, "primitiv", "devices", "hip"), os.path.join(tree, "primitiv", "devices", "hip"))
    shutil.copytree(os.path.join(BACKEND, "primitiv", "c", "devices", "hip"),
                    os.path.join(tree, "primitiv", "c", "devices", "hip"))
    # 2. the option, with the other backend options
    _insert(os.path.join(tree, "CMakeLists.txt"), 'option(PRIMITIV_USE_OPENCL "Enables the OpenCL backend." OFF)\n',
            'option(PRIMITIV_USE_HIP "Enable the AMD MI355X (gfx950) HIP backend." OFF)\n')
    # 3a. the backend block, before libprimitiv is assembled
    cm = os.path.join(tree, "primitiv", "CMakeLists.txt")
    _insert(cm, "# Builds the integrated binary.\n",
            "if(PRIMITIV_USE_HIP)\n  set(PRIMITIV_HIP_BACKEND_DIR %s)\n"
            "  include(${PRIMITIV_HIP_BACKEND_DIR}/primitiv/cmake/hip_backend.cmake)\nendif()\n\n" % BACKEND, before=True)
    # 3b. the C-API constructors, before libprimitiv_c is assembled
    _insert(cm, "  if(PRIMITIV_BUILD_STATIC_LIBRARY)\n    add_library(primitiv_c STATIC",
            "  if(PRIMITIV_USE_HIP)\n    include(${PRIMITIV_HIP_BACKEND_DIR}/primitiv/cmake/hip_backend_c_api.cmake)\n  endif()\n\n",
            before=True)
    # 4. config.h.in
    _insert(os.path.join(tree, "primitiv", "config.h.in"), "#cmakedefine PRIMITIV_USE_OPENCL\n",
            "#cmakedefine PRIMITIV_USE_HIP\n")
    # 5. the device type group
    _insert(os.path.join(tree, "primitiv", "core", "device.h"), "  OPENCL = 0x00020000,\n",
            "\n  GROUP_HIP = 0x00030000,\n  HIP = 0x00030000,\n  HIP16 = 0x00030001,\n")
    # 6. umbrella headers
    _insert(os.path.join(tree, "primitiv", "primitiv.h"), "#endif  // PRIMITIV_USE_OPENCL\n",
            "#ifdef PRIMITIV_USE_HIP\n#include <primitiv/devices/hip/device.h>\n#endif  // PRIMITIV_USE_HIP\n")
    _insert(os.path.join(tree, "primitiv", "c", "api.h"), "#endif  // PRIMITIV_USE_OPENCL\n",
            "#ifdef PRIMITIV_USE_HIP\n#include <primitiv/c/devices/hip/device.h>\n#endif  // PRIMITIV_USE_HIP\n")


C_PROGRAM = r"""
#include <stdio.h>
#include <string.h>
#include <primitiv/c/api.h>
int main(void) {
  uint32_t n = 12345;
  if (primitivGetNumHipDevices(&n) != PRIMITIV_C_OK) return 10;
  printf("devices %u\n", n);
  primitivDevice_t *dev = NULL;
  PRIMITIV_C_STATUS st = primitivCreateHipDevice(0, &dev);
  if (st == PRIMITIV_C_OK) { primitivDeleteDevice(dev); printf("created\n"); return 0; }
  char msg[1024]; size_t len = sizeof(msg);
  primitivGetMessage(msg, &len);
  printf("error: %s\n", msg);
  st = primitivCreateHipDeviceWithSeed(0, 7, &dev);
  return st == PRIMITIV_C_OK ? 11 : 0;
}
"""


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "primitiv", "core")), reason="primitiv source tree not present")
@pytest.mark.skipif(shutil.which("cmake") is None or not os.path.exists("/opt/rocm/bin/hipcc"), reason="cmake or hipcc missing")
def test_primitiv_use_hip_configures_builds_and_links(tmp_path):
    tree = str(tmp_path / "primitiv")
    shutil.copytree(REFERENCE, tree, ignore=shutil.ignore_patterns(".git", "docs", "examples"))
    apply_integration_edits(tree)
    build = str(tmp_path / "build")
    run = lambda cmd, **kw: subprocess.run(cmd, check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, **kw)
    # -Wno-error for the reference's own sources under a current gcc (primitiv/msgpack/writer.h trips -Wrange-loop-construct);
    # this backend's two host files are held to -Wall -Wextra -Werror by tests/host_class_lib.py
    run(["cmake", "-S", tree, "-B", build, "-DPRIMITIV_USE_HIP=ON", "-DPRIMITIV_BUILD_C_API=ON",
         "-DCMAKE_POLICY_VERSION_MINIMUM=3.5", "-DCMAKE_CXX_FLAGS=-Wno-error", "-DCMAKE_BUILD_TYPE=Release"])
    try:
        run(["cmake", "--build", build, "--", "-j8"])
    except subprocess.CalledProcessError as e:
        pytest.fail("build failed:\n" + e.stdout[-4000:])
    libdir = os.path.join(build, "primitiv")
    libs = {name: os.path.join(libdir, name) for name in ("libphip.so", "libprimitiv.so", "libprimitiv_c.so")}
    for path in libs.values():
        assert os.path.exists(path), path
    config = open(os.path.join(libdir, "config.h")).read() if os.path.exists(os.path.join(libdir, "config.h")) else \
        open(os.path.join(build, "primitiv", "config.h")).read()
    assert "#define PRIMITIV_USE_HIP" in config
    symbols = lambda lib: run(["nm", "-D", "--defined-only", lib]).stdout
    # the constructors live in libprimitiv_c like the other backends', the class in libprimitiv
    assert "primitivCreateHipDevice" in symbols(libs["libprimitiv_c.so"])
    assert "primitivCreateHipDevice" not in symbols(libs["libprimitiv.so"])
    assert "primitiv7devices3HIP" in symbols(libs["libprimitiv.so"])
    assert "phip_matmul_fw_f32" in symbols(libs["libphip.so"])
    # a C program against the three libraries: no GPU here, so no device and a refusal by id
    src = tmp_path / "ask.c"
    src.write_text(C_PROGRAM)
    exe = str(tmp_path / "ask")
    run(["gcc", "-std=c99", "-DPRIMITIV_USE_HIP", str(src), "-o", exe, "-I" + tree, "-I" + build, "-I" + os.path.join(ROOT, "include"),
         "-L" + libdir, "-lprimitiv_c", "-lprimitiv", "-lphip", "-Wl,-rpath," + libdir])
    out = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert out.returncode == 0, out.stdout
    if "created" not in out.stdout:        # a GPU-less machine
        assert "devices 0" in out.stdout and "Invalid device ID" in out.stdout, out.stdout
