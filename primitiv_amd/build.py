"""Builds libphip.so (HIP, gfx950 only) in-tree with hipcc.

Usage:  python -m primitiv_amd.build [-j N]
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libphip.so")

SOURCES = [
    "phip_runtime.hip",
    "phip_lanes.hip",
    "phip_elementwise.hip",
    "phip_pointwise_unary.hip",
    "phip_pointwise_binary.hip",
    "phip_indexing.hip",
    "phip_reduce.hip",
    "phip_random.hip",
    "phip_gemm_f32.hip",
    "phip_gemm_f32_direct.hip",
    "phip_gemm_f32_tile16.hip",
    "phip_gemm_f32_lds.hip",
    "phip_gemm_f32_slab.hip",
    "phip_gemm_f32_rankk.hip",
    "phip_gemm_f32_pair.hip",
    "phip_gemm_f32_stream_pair.hip",
    "phip_conv_pool.hip",
    "phip_gemm_h16.hip",
    "phip_gemm_h16_skinny.hip",
    "phip_gemm_h16_big.hip",
    "phip_matmul.hip",
]

# Packed-fp32 instruction selection is switched off for all device code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _hipcc():
    return os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def _compile(src):
    obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc()] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    subprocess.check_call(cmd)
    return obj


def build(jobs=4, verbose=True):
    """Compiles every source and links libphip.so; always rebuilds."""
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    subprocess.check_call(cmd)
    if verbose:
        print("built", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    j = 4
    if "-j" in sys.argv:
        j = int(sys.argv[sys.argv.index("-j") + 1])
    build(jobs=j)
