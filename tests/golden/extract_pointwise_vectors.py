#!/usr/bin/env python3
"""Collects the golden vectors of the reference's elementwise-operation tests.

Reads the reference's test sources AS TEXT (nothing of the reference is
compiled, imported or run), pulls out the literal input and expected-output
vectors of the tests listed in FORWARD, BACKWARD and INPLACE, and writes them to
``pointwise_vectors.json`` next to this script.  Only needed to regenerate
that fixture; the test-suite reads the JSON alone.

    python tests/golden/extract_pointwise_vectors.py [/root/reference]

Every case records where it came from (``source``: file:line and test name),
what is computed (``kind`` + ``op``), the flat operand arrays with their batch
sizes, the expected arrays, and the ULP bounds the reference's test grants:
``ulps`` for 32-bit devices (the largest bound it gives any of them, 0 where
it demands exact equality) and ``ulps16`` for its half-precision device.
"""
import json
import os
import re
import sys

import numpy as np

F = np.float32
DEFAULT_ULPS, DEFAULT_ULPS16 = 4, 1 << 12   # test/test_utils.cc:42-55

UNARY = {"abs", "sqrt", "exp", "log", "tanh", "sigmoid", "softplus", "sin", "cos", "tan"}
ARITH = {"add": "add", "subtract": "subtract", "multiply": "multiply", "divide": "divide", "pow": "pow",
         "+": "add", "-": "subtract", "*": "multiply", "/": "divide"}


def blocks(text, fixture):
    """Yields (name, first_line, body) of every TEST_F(fixture, name)."""
    for m in re.finditer(r"TEST_F\(%s, (\w+)\) \{" % fixture, text):
        depth, i = 1, m.end()
        while depth:
            depth += {"{": 1, "}": -1}.get(text[i], 0)
            i += 1
        yield m.group(1), text.count("\n", 0, m.start()) + 1, text[m.end():i - 1]


def evaluate(expr, k=None):
    """Value of one C++ initializer element, in the arithmetic C++ would use."""
    e = expr.strip()
    e = re.sub(r"(?<![\w.])((?:\d+\.?\d*|\.\d+)(?:[eE][-+]?\d+)?)f\b", r"F(\1)", e)
    if not re.fullmatch(r"[-+*/() .\deExFk]*", e):
        raise ValueError("unexpected initializer element: %r" % expr)
    return F(eval(e, {"F": F, "k": None if k is None else F(k)}))


def elements(body, k=None):
    return [float(evaluate(x, k)) for x in body.split(",") if x.strip()]


def shape_of(text, tensors):
    """(volume, batch) of a shape expression; `x.shape()` refers to a tensor."""
    text = text.strip()
    m = re.fullmatch(r"(\w+)\.shape\(\)", text)
    if m:
        return tensors[m.group(1)]["shape"]
    m = re.fullmatch(r"Shape\(\{([^}]*)\}(?:,\s*(\d+))?\)", text) or re.fullmatch(r"\{([^}]*)\}()", text)
    if not m:
        raise ValueError("unexpected shape: %r" % text)
    dims = [int(d) for d in m.group(1).split(",") if d.strip()]
    return int(np.prod(dims)) if dims else 1, int(m.group(2) or 1)


def ulps_of(body):
    """(32-bit bound, half bound) granted by the test body."""
    if "vector_match_ulps" not in body and "vector_near" not in body:
        return 0, 0
    # of an `#ifdef PRIMITIV_MAYBE_FPMATH_X87 ... #else ... #endif` pair only the #else part applies here
    body = re.sub(r"#ifdef PRIMITIV_MAYBE_FPMATH_X87.*?#else", "", body, flags=re.S)
    m = re.search(r"ulps\s*=([^;]*);", body)
    if not m:
        return DEFAULT_ULPS, DEFAULT_ULPS16
    expr = re.sub(r"#\w+.*", "", m.group(1))
    half = re.search(r"CUDA16\s*\?\s*(\d+|get_default_ulps\(\*dev\))", expr)
    half = DEFAULT_ULPS16 if not half or not half.group(1).isdigit() else int(half.group(1))
    rest = re.sub(r"dev_type == DeviceType::CUDA16\s*\?\s*(\d+|get_default_ulps\(\*dev\))", "", expr)
    nums = [int(n) for n in re.findall(r"[?:]\s*(\d+)", rest)]
    if "get_default_ulps" in rest or not nums:
        nums.append(DEFAULT_ULPS)
    return max(nums), half


def scenarios(body):
    """Splits a test body where its first data vector is declared again."""
    starts = [m.start() for m in re.finditer(r"const vector<float> (?:x_data|a_data) ", body)]
    if len(starts) <= 1:
        return [body]
    return [body[s:e] for s, e in zip(starts, starts[1:] + [len(body)])]


def declarations(body, k=None):
    vectors, tensors, consts = {}, {}, {}
    for m in re.finditer(r"const vector<float> (\w+)\s*\{([^}]*)\};", body):
        if m.group(1) != "ks":
            vectors[m.group(1)] = elements(m.group(2), k)
    m = re.search(r"const float k = ([^;]+);", body)
    if m:
        consts["k"] = float(evaluate(m.group(1)))
    pat = (r"Tensor (\w+) = dev->new_tensor_by_(vector|constant)\(\s*"
           r"((?:Shape\(\{[^}]*\}(?:,\s*\d+)?\))|(?:\{[^}]*\})|(?:\w+\.shape\(\))),\s*"
           r"(\{[^}]*\}|[-\w.]+)\)")
    fw = re.compile(r"Tensor (\w+) = dev->\w+_fw\(([^;]*)\);")
    events = sorted(list(re.finditer(pat, body)) + list(fw.finditer(body)), key=lambda m: m.start())
    for m in events:
        if m.re is fw:   # a forward result: its shape follows from the tensor arguments
            args = [tensors[a.strip()]["shape"] for a in m.group(2).split(",") if a.strip() in tensors]
            tensors[m.group(1)] = {"shape": (args[0][0], max(a[1] for a in args)), "data": None}
            continue
        name, how, shape, arg = m.groups()
        volume, batch = shape_of(shape, tensors)
        if how == "constant":
            data = [float(evaluate(arg))] * (volume * batch)
        elif arg.startswith("{"):
            data = elements(arg[1:-1], k)
        else:
            data = vectors[arg]
        assert len(data) == volume * batch, (name, len(data), volume, batch)
        tensors[name] = {"shape": (volume, batch), "data": data}
    return vectors, tensors, consts


def forward_cases(name, line, body, src):
    """Cases of one forward test: every `const Tensor yN = f(args)` statement."""
    out = []
    ulps, ulps16 = ulps_of(body)
    ks = re.search(r"const vector<float> ks\s*\{([^}]*)\};", body)
    for k in (elements(ks.group(1)) if ks else [None]):
        for part in scenarios(body):
            vectors, tensors, consts = declarations(part, k)
            kval = consts.get("k", k)
            seen = set()
            checked = dict((r, v) for v, r in
                           re.findall(r"vector_match(?:_ulps)?\(\s*(\w+),\s*(\w+)\.to_vector\(\)", part))
            pat = r"const Tensor (y\d?) = (?:(\w+)\(([^;]*)\)|(-?\w+)(?: ([-+*/]) (\w+))?);"
            for m in re.finditer(pat, part):
                y, func, args, lhs, oper, rhs = m.groups()
                if func:
                    args = [a.strip() for a in args.split(",")]
                elif oper:
                    func, args = oper, [lhs, rhs]
                elif lhs.startswith("-"):
                    func, args = "negate", [lhs[1:]]
                else:
                    continue
                expected = vectors[checked[y]]
                case = {"source": "%s:%d %s" % (src, line, name), "ulps": ulps, "ulps16": ulps16,
                        "expected": expected}
                if func == "negate" or func in UNARY:
                    case.update(kind="unary_fw", op=func, x=tensors[args[0]]["data"])
                elif func in ("relu", "lrelu", "prelu", "elu"):
                    kk = {"relu": 0.0, "lrelu": 0.01}.get(func, kval)
                    case.update(kind="const_fw", op="elu" if func == "elu" else "prelu",
                                x=tensors[args[0]]["data"], k=float(F(kk)))
                elif func == "pown":
                    kk = int(args[1], 0)
                    case.update(kind="pown_fw", x=tensors[args[0]]["data"], k=kk - (1 << 32) if kk >= 1 << 31 else kk)
                elif func in ARITH:
                    op = ARITH[func]
                    a, b = args
                    if a == "k" and "k" not in tensors or b == "k" and "k" not in tensors:
                        left = a == "k"
                        x = tensors[b if left else a]
                        cname = op + "_const" + ("" if op in ("add", "multiply") else "_l" if left else "_r")
                        case.update(kind="const_fw", op=cname, x=x["data"], k=float(F(kval)))
                    elif "k" in (a, b):
                        left = a == "k"
                        x, kt = tensors[b if left else a], tensors["k"]
                        case.update(kind="scalar_fw", op=op, k_on_left=left, x=x["data"], k=kt["data"],
                                    volume=x["shape"][0], bx=x["shape"][1], bk=kt["shape"][1])
                    else:
                        ta, tb = tensors[a], tensors[b]
                        case.update(kind="binary_fw", op=op, a=ta["data"], b=tb["data"], volume=ta["shape"][0],
                                    ba=ta["shape"][1], bb=tb["shape"][1])
                else:
                    raise ValueError("%s: unknown function %s" % (name, func))
                key = json.dumps({k2: v for k2, v in case.items() if k2 != "source"}, sort_keys=True)
                if key not in seen:   # `add(a, b)` and `a + b` are the same case
                    seen.add(key)
                    out.append(case)
    assert out, name
    return out


def backward_cases(name, line, body, src):
    """Cases of one backward test: the `dev->NAME_bw(...)` call and its *_val vectors."""
    out = []
    ulps, ulps16 = ulps_of(body)
    ks = re.search(r"const vector<float> ks\s*\{([^}]*)\};", body)
    for k in (elements(ks.group(1)) if ks else [None]):
        vectors, tensors, _ = declarations(body, k)
        m = re.search(r"dev->(\w+)_bw\(([^;]*)\);", body)
        op, args = m.group(1), [a.strip() for a in m.group(2).split(",")]
        case = {"source": "%s:%d %s" % (src, line, name), "ulps": ulps, "ulps16": ulps16}
        if op in UNARY:
            case.update(kind="unary_bw", op=op, x=tensors["x"]["data"], gy=tensors["gy"]["data"],
                        gx0=tensors["gx"]["data"], expected=vectors["gx_val"])
        elif op in ARITH:
            ta, tb = tensors["a"], tensors["b"]
            case.update(kind="binary_bw", op=op, a=ta["data"], b=tb["data"], gy=tensors["gy"]["data"],
                        volume=ta["shape"][0], ba=ta["shape"][1], bb=tb["shape"][1],
                        expected_ga=vectors["ga_val"], expected_gb=vectors["gb_val"])
        else:
            case.update(kind="const_bw", op=op, x=tensors["x"]["data"], gy=tensors["gy"]["data"], k=float(F(k)),
                        gx0=tensors["gx"]["data"], expected=vectors["gx_val"])
        assert len(args) >= 4
        out.append(case)
    return out


def inplace_cases(name, line, body, src):
    out = []
    vectors = {m.group(1): elements(m.group(2))
               for m in re.finditer(r"const vector<float> (\w+)\s*\{([^}]*)\};", body)}
    if "MultiplyConst" in name:
        for k, y in ((2.0, "y1_data"), (0.5, "y2_data")):
            out.append({"source": "%s:%d %s" % (src, line, name), "kind": "inplace_multiply_const", "k": k,
                        "x": vectors["x_data"], "expected": vectors[y], "ulps": 0, "ulps16": 0})
    else:
        shapes = re.findall(r"Tensor (a|b) = dev->new_tensor_by_vector\(((?:Shape\(\{[^}]*\}(?:,\s*\d+)?\))|(?:\{[^}]*\})),",
                            body)
        sh = {n: shape_of(s, {}) for n, s in shapes}
        out.append({"source": "%s:%d %s" % (src, line, name), "kind": "inplace_subtract",
                    "x": vectors["b_data"], "y": vectors["a_data"], "volume": sh["a"][0], "bx": sh["b"][1],
                    "by": sh["a"][1], "expected": vectors["y_data"], "ulps": 0, "ulps16": 0})
    return out


FORWARD = """CheckNegate CheckAddConst CheckAddScalar CheckAddScalarBatchBroadcast CheckAdd CheckAddBatchBroadcast
CheckSubtractConst CheckSubtractScalar CheckSubtractScalarBatchBroadcast CheckSubtract CheckSubtractBatchBroadcast
CheckMultiplyConst CheckMultiplyScalar CheckMultiplyScalarBatchBroadcast CheckMultiply CheckMultiplyBatchBroadcast
CheckDivideConst CheckDivideScalar CheckDivideScalarBatchBroadcast CheckDivide CheckDivideBatchBroadcast
CheckPowConstR CheckPowConstL CheckPowScalarR CheckPowScalarL CheckPowScalarRBatchBroadcast
CheckPowScalarLBatchBroadcast CheckPow CheckPowBatchBroadcast CheckAbs CheckSqrt CheckExp CheckLog CheckPowNPositive
CheckPowNNegative CheckPowNUpperBound CheckPowNLowerBound CheckPowNPositiveConvergence CheckPowNNegativeConvergence
CheckTanh CheckSigmoid CheckSoftplus CheckSin CheckCos CheckTan CheckReLU CheckLReLU CheckPReLU CheckELU""".split()
BACKWARD = """CheckAbs CheckSqrt CheckExp CheckLog CheckTanh CheckSigmoid CheckSoftplus CheckSin CheckCos CheckTan
CheckAddConst CheckSubtractConstR CheckSubtractConstL CheckMultiplyConst CheckDivideConstR CheckDivideConstL
CheckPReLU CheckELU CheckAdd11 CheckAddNN CheckAdd1N CheckAddN1 CheckSubtract11
CheckSubtractNN CheckSubtract1N CheckSubtractN1 CheckMultiply11 CheckMultiplyNN CheckMultiply1N CheckMultiplyN1
CheckDivide11 CheckDivideNN CheckDivide1N CheckDivideN1""".split()
INPLACE = "CheckInplaceMultiplyConst CheckInplaceSubtractNN CheckInplaceSubtract1N CheckInplaceSubtractN1".split()


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    cases = []
    for fname, fixture, wanted, handler in (
            ("test/tensor_forward_test.cc", "TensorForwardTest", FORWARD, forward_cases),
            ("test/tensor_backward_test.cc", "TensorBackwardTest", BACKWARD, backward_cases),
            ("test/tensor_test.cc", "TensorTest", INPLACE, inplace_cases)):
        text = open(os.path.join(root, fname)).read()
        text = re.sub(r"//[^\n]*", "", text)
        found = {}
        for name, line, body in blocks(text, fixture):
            if name in wanted:
                found[name] = handler(name, line, body, fname)
        missing = [w for w in wanted if w not in found]
        assert not missing, missing
        for w in wanted:
            cases.extend(found[w])
    # test/tensor_forward_test.cc:92-112 CheckIdentity keeps its vectors in a table of structs
    for rows in (1, 2, 3, 4):
        cases.append({"source": "test/tensor_forward_test.cc:92 CheckIdentity", "kind": "identity", "rows": rows,
                      "expected": [float(i % (rows + 1) == 0) for i in range(rows * rows)], "ulps": 0, "ulps16": 0})
    doc = {"_comment": "Golden vectors transcribed from the reference's tests by extract_pointwise_vectors.py; "
                       "ulps = bound for 32-bit devices (0: exact), ulps16 = bound for half storage.",
           "cases": cases}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "pointwise_vectors.json")
    with open(path, "w") as f:   # one case per line
        f.write('{"_comment": %s,\n"cases": [\n' % json.dumps(doc["_comment"]))
        f.write(",\n".join(json.dumps(c, separators=(",", ":")) for c in cases))
        f.write("\n]}\n")
    kinds = {}
    for c in cases:
        kinds[c["kind"]] = kinds.get(c["kind"], 0) + 1
    print("wrote %d cases to %s: %s" % (len(cases), path, kinds))


if __name__ == "__main__":
    main()
