#!/usr/bin/env python3
"""Collects the golden vectors of the reference's convolution and pooling tests.

Reads the reference's test sources AS TEXT (nothing of the reference is
compiled, imported or run), pulls out the literal shapes, arguments, input and
expected-output vectors of the CheckConv2D_* and CheckMaxPool2D_* tests of
``test/tensor_forward_test.cc`` and ``test/tensor_backward_test.cc`` (all but
the VGG16-sized ones, whose expected values are closed forms that the tests
restate), and writes them to ``conv_pool_vectors.json`` next to this script.
Only needed to regenerate that fixture; the test-suite reads the JSON alone.

    python tests/golden/extract_conv_pool_vectors.py [/root/reference]

Forward cases hold x, w (convolution only) and the expected y.  Backward cases
hold the expected gx (and gw); their inputs are what the reference's macro
builds: x and w count up from 1, gy is all ones, gx and gw start at 1
(test/tensor_backward_test.cc:1920-1937, 2600-2612).
"""
import json
import os
import re
import sys

import numpy as np

from extract_pointwise_vectors import blocks, elements


def product(expr):
    return int(np.prod([int(t) for t in expr.split("*")]))


def vector(body, name):
    m = re.search(r"vector<float> %s = make_iota_vector\(([^,]*), (\d+)\);" % name, body)
    if m:
        return [float(int(m.group(2)) + i) for i in range(product(m.group(1)))]
    m = re.search(r"vector<float> %s\s*\{([^}]*)\}" % name, body)
    if m:
        return elements(re.sub(r"//[^\n]*", "", m.group(1)))
    return None


def shape(body, name):
    m = re.search(r"Shape %s\s*\{([^}]*)\};" % name, body)
    if m:
        return [int(d) for d in m.group(1).split(",") if d.strip()], 1
    m = re.search(r"Shape %s\(\{([^}]*)\}, (\d+)\);" % name, body)
    return [int(d) for d in m.group(1).split(",") if d.strip()], int(m.group(2))


def cases(path, fixture, prefix, macro, names):
    text = open(path).read()
    out = []
    for name, line, body in blocks(text, fixture):
        if not name.startswith(prefix) or "VGG16" in name:
            continue
        m = re.search(macro + r"\(([^)]*)\);", body)
        if not m:
            continue
        case = {"source": "%s:%d %s" % (os.path.relpath(path, root), line, name),
                "args": [int(a) for a in m.group(1).split(",")]}
        for key in names:
            if key.endswith("_shape"):
                case[key], case[key[:-6] + "_batch"] = shape(body, key)
            else:
                v = vector(body, key)
                if v is None:
                    raise ValueError("%s: no %s" % (name, key))
                case[key] = v
        out.append(case)
    return out


if __name__ == "__main__":
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    fw = os.path.join(root, "test", "tensor_forward_test.cc")
    bw = os.path.join(root, "test", "tensor_backward_test.cc")
    result = {
        "conv2d_fw": cases(fw, "TensorForwardTest", "CheckConv2D_", "TEST_CONV2D",
                           ["x_shape", "w_shape", "y_shape", "x_data", "w_data", "y_data"]),
        "conv2d_bw": cases(bw, "TensorBackwardTest", "CheckConv2D_", "TEST_CONV2D",
                           ["x_shape", "w_shape", "y_shape", "gx_data", "gw_data"]),
        "max_pool2d_fw": cases(fw, "TensorForwardTest", "CheckMaxPool2D_", "TEST_MAX_POOL2D",
                               ["x_shape", "y_shape", "x_data", "y_data"]),
        "max_pool2d_bw": cases(bw, "TensorBackwardTest", "CheckMaxPool2D_", "TEST_MAX_POOL2D",
                               ["x_shape", "y_shape", "gx_data"]),
    }
    target = os.path.join(os.path.dirname(os.path.abspath(__file__)), "conv_pool_vectors.json")
    with open(target, "w") as f:
        json.dump(result, f, indent=0, separators=(",", ":"))
        f.write("\n")
    print({k: len(v) for k, v in result.items()}, "->", target)
