"""Replays the golden elementwise cases (tests/golden/pointwise_vectors.json)
on a backend: the oracle on the CPU, the HIP devices on the GPU."""
import json
import os

import numpy as np

_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "pointwise_vectors.json")
with open(_PATH) as _f:
    CASES = json.load(_f)["cases"]


def case_id(case):
    name = case["source"].split()[-1]
    extra = case.get("op", "")
    if "k" in case and not isinstance(case["k"], list):
        extra += "_k%g" % case["k"]
    if case.get("k_on_left"):
        extra += "_left"
    return "%s-%s-%s" % (case["kind"], name, extra)


def f32(x):
    return np.asarray(x, dtype=np.float32)


def run_case_on(be, c):
    """Returns [(result, expected), ...] of case `c` computed by backend `be`.

    A backward case first computes y with the backend's own forward operation,
    as the reference's tests do."""
    kind = c["kind"]
    if kind == "unary_fw":
        return [(be.unary_fw(c["op"], f32(c["x"])), c["expected"])]
    if kind == "const_fw":
        return [(be.const_fw(c["op"], f32(c["x"]), c["k"]), c["expected"])]
    if kind == "pown_fw":
        return [(be.pown_fw(f32(c["x"]), c["k"]), c["expected"])]
    if kind == "scalar_fw":
        return [(be.scalar_fw(c["op"], c["k_on_left"], f32(c["x"]), f32(c["k"]), c["volume"], c["bx"], c["bk"]),
                 c["expected"])]
    if kind == "binary_fw":
        return [(be.binary_fw(c["op"], f32(c["a"]), f32(c["b"]), c["volume"], c["ba"], c["bb"]), c["expected"])]
    if kind == "unary_bw":
        x = f32(c["x"])
        y = be.unary_fw(c["op"], x)
        return [(be.unary_bw(c["op"], x, y, f32(c["gy"]), f32(c["gx0"])), c["expected"])]
    if kind == "const_bw":
        x = f32(c["x"])
        y = be.const_fw(c["op"], x, c["k"])
        return [(be.const_bw(c["op"], x, y, f32(c["gy"]), c["k"], f32(c["gx0"])), c["expected"])]
    if kind == "binary_bw":
        a, b = f32(c["a"]), f32(c["b"])
        y = be.binary_fw(c["op"], a, b, c["volume"], c["ba"], c["bb"])
        ga, gb = be.binary_bw(c["op"], a, b, y, f32(c["gy"]), np.zeros_like(a), np.zeros_like(b), c["volume"],
                              c["ba"], c["bb"])
        return [(ga, c["expected_ga"]), (gb, c["expected_gb"])]
    if kind == "inplace_subtract":
        return [(be.inplace_subtract(f32(c["x"]), f32(c["y"]), c["volume"], c["bx"], c["by"]), c["expected"])]
    if kind == "inplace_multiply_const":
        return [(be.inplace_multiply_const(c["k"], f32(c["x"])), c["expected"])]
    if kind == "identity":
        return [(be.identity(c["rows"]), c["expected"])]
    raise ValueError(kind)
