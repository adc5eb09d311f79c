"""Replays the golden data-movement / reduction cases
(tests/golden/indexing_vectors.json) on a backend: the oracle on the CPU, the
HIP devices on the GPU.  A backend takes and returns flat float32 arrays with
(dims, batch) alongside."""
import json
import os

import numpy as np

_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "indexing_vectors.json")
with open(_PATH) as _f:
    CASES = json.load(_f)["cases"]


def case_id(c):
    bits = [c["kind"], c["source"].split()[-1], c.get("op", "")]
    for k in ("dim", "lower", "ids", "size"):
        if k in c:
            bits.append("%s%s" % (k, "".join(map(str, c[k])) if isinstance(c[k], list) else c[k]))
    if "x_constant" in c:
        bits.append("n%d" % c["dims"][0])
    return "-".join(b for b in bits if b)


def _x(c):
    if "x_constant" in c:
        n = int(np.prod(c["dims"])) * c["batch"] if c["dims"] else c["batch"]
        return np.full(n, c["x_constant"], dtype=np.float32)
    return np.asarray(c["x"], dtype=np.float32)


def run_case_on(be, c):
    """Result of case `c` on backend `be` (a float32 or uint32 array)."""
    kind, dims, batch = c["kind"], c["dims"], c["batch"]
    if kind == "pick_fw":
        return be.pick_fw(_x(c), dims, batch, c["ids"], c["dim"])
    if kind == "slice_fw":
        return be.slice_fw(_x(c), dims, batch, c["dim"], c["lower"], c["upper"])
    if kind == "transpose_fw":
        return be.transpose_fw(_x(c), dims[0], dims[1], batch)
    if kind == "reduce_fw":
        return be.reduce_fw(c["op"], _x(c), dims, batch, c["dim"])
    if kind == "broadcast_fw":
        return be.broadcast_fw(_x(c), dims, batch, c["dim"], c["size"])
    if kind == "batch_pick_fw":
        return be.batch_pick_fw(_x(c), dims, batch, c["ids"])
    if kind == "argmax":
        return be.arg_extremum("max", _x(c), dims, batch, c["dim"])
    if kind == "pick_bw":
        return be.pick_bw(np.asarray(c["gy"], np.float32), np.asarray(c["gx0"], np.float32), dims, batch,
                          c["ids"], c["dim"])
    if kind == "extremum_bw":
        return be.extremum_bw(c["op"], _x(c), np.asarray(c["y"], np.float32), np.asarray(c["gy"], np.float32),
                              np.asarray(c["gx0"], np.float32), dims, batch, c["dim"])
    raise ValueError(kind)
