#!/usr/bin/env python3
"""Collects the vectors of the reference's two LSTM graph tests.

Reads ``test/graph_test.cc`` AS TEXT (nothing of the reference is compiled,
imported or run) and pulls out of ``CheckLSTM`` and ``CheckConcatLSTM`` what
those tests hold as literals: the initial values of every parameter, the two
input nodes, the operator count the graph must have and the expected
per-element losses (``vector_near`` at 1e-6 there).  Written to
``graph_vectors.json`` next to this script.  Only needed to regenerate that
fixture; the test-suite reads the JSON alone.

    python tests/golden/extract_graph_vectors.py [/root/reference]
"""
import json
import os
import re
import sys

from extract_pointwise_vectors import blocks, elements


def floats(text):
    return elements(re.sub(r"//[^\n]*", "", text))


def lstm_case(name, line, body, path, root):
    case = {"source": "%s:%d %s" % (os.path.relpath(path, root), line, name), "parameters": {}, "inputs": {}}
    for m in re.finditer(r"Parameter (\w+)\(\{([^}]*)\}, \{([^}]*)\}\);", body):
        case["parameters"][m.group(1)] = {"shape": [int(d) for d in m.group(2).split(",")],
                                         "values": floats(m.group(3))}
    for m in re.finditer(r"Parameter (\w+)\(\{([^}]*)\}, initializers::Constant\(([^)]*)\)\);", body):
        shape = [int(d) for d in m.group(2).split(",")]
        n = 1
        for d in shape:
            n *= d
        case["parameters"][m.group(1)] = {"shape": shape, "values": [float(m.group(3))] * n}
    for m in re.finditer(r"const Node (\w+) = input<Node>\(Shape\(\{([^}]*)\}, (\d+)\), \{([^}]*)\}\);", body):
        case["inputs"][m.group(1)] = {"shape": [int(d) for d in m.group(2).split(",")], "batch": int(m.group(3)),
                                     "values": floats(m.group(4))}
    case["num_operators"] = int(re.search(r"EXPECT_EQ\((\d+)u, g\.num_operators\(\)\);", body).group(1))
    case["expected_losses"] = floats(re.search(r"expected_losses\s*\{([^}]*)\}", body).group(1))
    case["tolerance"] = float(re.search(r"vector_near\(expected_losses, loss_tensor\.to_vector\(\), ([^)]*)\)", body).group(1))
    return case


if __name__ == "__main__":
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    path = os.path.join(root, "test", "graph_test.cc")
    result = {"_comment": "literals of test/graph_test.cc CheckLSTM / CheckConcatLSTM, written by extract_graph_vectors.py"}
    for name, line, body in blocks(open(path).read(), "GraphTest"):
        if name in ("CheckLSTM", "CheckConcatLSTM"):
            result[name] = lstm_case(name, line, body, path, root)
    assert set(result) >= {"CheckLSTM", "CheckConcatLSTM"}
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "graph_vectors.json")
    with open(out, "w") as f:
        json.dump(result, f, indent=1)
        f.write("\n")
    print("wrote", out)
