"""Matmul calls on two lanes (streams): whatever the library overlaps, the caller must see the
results of its calls in the order it made them.  Every case runs the same program once with the
lanes on and once with every launch on one stream and asks for the same bits (forward products are
reproducible by construction, gradient products with phip_set_deterministic), and checks the
in-order run against the oracle."""
import os

import numpy as np
import pytest

import oracle
import primitiv_amd as pa
from util import norm_rel_err

pytestmark = pytest.mark.gpu

S = pa.Shape


def _device(overlap, deterministic=True, storage="f32"):
    # the library engages its second lane only in a long run of matmul calls and backs off when a run
    # was short; here it is engaged by the first call, every time (read when the context is created)
    saved = {k: os.environ.get(k) for k in ("PHIP_OVERLAP_AFTER", "PHIP_OVERLAP_BACKOFF")}
    os.environ["PHIP_OVERLAP_AFTER"], os.environ["PHIP_OVERLAP_BACKOFF"] = "1", "0"
    try:
        d = pa.HIP(0) if storage == "f32" else pa.HIP16(0, storage=storage)
    finally:
        for k, v in saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    d.set_deterministic(deterministic)
    d.set_overlap(overlap)
    return d


def _run_both(program, deterministic=True, storage="f32"):
    """program(dev) -> list of numpy arrays; returns (with lanes, in order)."""
    out = []
    for overlap in (True, False):
        d = _device(overlap, deterministic, storage)
        try:
            out.append([np.asarray(v, dtype=np.float32) for v in program(d)])
        finally:
            d.close()
    return out


def _same_bits(a, b):
    assert len(a) == len(b)
    for i, (x, y) in enumerate(zip(a, b)):
        assert x.shape == y.shape and np.array_equal(x.view(np.uint32), y.view(np.uint32)), "result %d differs" % i


# one shape of each kernel family that the per-timestep workloads use (m, k, n = minibatch)
SHAPES = [(512, 512, 64), (650, 650, 64), (1000, 650, 64), (96, 200, 16)]


@pytest.mark.parametrize("m,k,n", SHAPES)
def test_a_product_that_reads_two_earlier_products_waits_for_both(m, k, n):
    rng = np.random.default_rng(1)
    a1 = rng.standard_normal(m * k).astype(np.float32) / np.sqrt(k)
    b1 = rng.standard_normal(k * n).astype(np.float32)
    a2 = rng.standard_normal(k * m).astype(np.float32) / np.sqrt(m)

    def program(d):
        ta1, tb1, ta2 = (d.new_tensor_by_vector(S([m, k]), a1), d.new_tensor_by_vector(S([k, n]), b1),
                         d.new_tensor_by_vector(S([k, m]), a2))
        outs = []
        for _ in range(6):
            y1 = d.matmul_fw(ta1, tb1)        # [m x n]
            y1b = d.matmul_fw(ta1, tb1)       # independent of y1: may take the other lane
            y2 = d.matmul_fw(ta2, y1)         # [k x n], reads y1
            y3 = d.matmul_fw(ta1, y2)         # [m x n], reads y2
            y4 = d.matmul_fw(ta2, y1b)        # reads the product that ran on the other lane
            outs += [y1.to_vector(), y3.to_vector(), y4.to_vector()]
        return outs

    lanes, in_order = _run_both(program)
    _same_bits(lanes, in_order)
    y1 = oracle.matmul_fw(a1, b1, m, k, n, 1, 1)
    y3 = oracle.matmul_fw(a1, oracle.matmul_fw(a2, y1, k, m, n, 1, 1), m, k, n, 1, 1)
    assert norm_rel_err(in_order[0], y1) <= 1e-4
    assert norm_rel_err(in_order[1], y3) <= 1e-4


@pytest.mark.parametrize("m,k,n", SHAPES)
def test_gradients_accumulated_by_calls_on_different_lanes(m, k, n):
    rng = np.random.default_rng(2)
    a = rng.standard_normal(m * k).astype(np.float32) / np.sqrt(k)
    steps = 5
    bs = [rng.standard_normal(k * n).astype(np.float32) for _ in range(steps)]
    gys = [rng.standard_normal(m * n).astype(np.float32) for _ in range(steps)]

    def program(d):
        ta = d.new_tensor_by_vector(S([m, k]), a)
        tb = [d.new_tensor_by_vector(S([k, n]), b) for b in bs]
        tgy = [d.new_tensor_by_vector(S([m, n]), g) for g in gys]
        ga = d.new_tensor_by_constant(S([m, k]), 0)
        gbs = [d.new_tensor_by_constant(S([k, n]), 0) for _ in range(steps)]
        ys = []
        for t in range(steps):                 # forward and backward calls alternate, as in bench.py
            y = d.matmul_fw(ta, tb[t])
            d.matmul_bw(ta, tb[t], y, tgy[t], ga, gbs[t])     # every call adds into ga
            ys.append(y)
        return [ga.to_vector()] + [g.to_vector() for g in gbs] + [y.to_vector() for y in ys]

    lanes, in_order = _run_both(program)
    _same_bits(lanes, in_order)
    # the default way of adding split products (atomics, both gradients in one launch): right to rounding
    for got, want in zip(*_run_both(program, deterministic=False)):
        assert norm_rel_err(got, want) <= 1e-5
    ga = np.zeros(m * k, np.float32)
    for t in range(steps):
        ga, gb = oracle.matmul_bw(a, bs[t], gys[t], ga, np.zeros(k * n, np.float32), m, k, n, 1, 1)
        assert norm_rel_err(in_order[1 + t], gb) <= 1e-4
    assert norm_rel_err(in_order[0], ga) <= 1e-4


def test_other_operations_and_readbacks_wait_for_both_lanes():
    m, k, n = 650, 650, 64
    rng = np.random.default_rng(3)
    a = rng.standard_normal(m * k).astype(np.float32) / np.sqrt(k)
    b = rng.standard_normal(k * n).astype(np.float32)

    def program(d):
        ta, tb = d.new_tensor_by_vector(S([m, k]), a), d.new_tensor_by_vector(S([k, n]), b)
        outs = []
        for _ in range(8):
            y1 = d.matmul_fw(ta, tb)
            y2 = d.matmul_fw(ta, tb)                     # may run beside y1
            h = d.unary_fw("tanh", y2)                   # an elementwise kernel on the product of either lane
            y3 = d.matmul_fw(ta, h)                      # a product behind other work
            outs += [y2.to_vector(), y3.to_vector()]     # read straight after the call
            d.inplace_add(y1, y3)                        # y3 += y1
            tb = y3                                      # the next round's operand
        return outs

    lanes, in_order = _run_both(program)
    _same_bits(lanes, in_order)
    y = oracle.matmul_fw(a, b, m, k, n, 1, 1)
    assert norm_rel_err(in_order[0], y) <= 1e-4
    assert norm_rel_err(in_order[1], oracle.matmul_fw(a, np.tanh(y), m, k, n, 1, 1)) <= 1e-4


def test_an_operand_overwritten_by_a_later_call_is_read_first():
    # y = a.b1 runs on one lane; the next call overwrites b1's memory (same pool block, new tensor):
    # it has to wait for the reader
    m, k, n = 1000, 650, 64
    rng = np.random.default_rng(4)
    a = rng.standard_normal(m * k).astype(np.float32) / np.sqrt(k)
    at = rng.standard_normal(k * m).astype(np.float32) / np.sqrt(m)
    b = rng.standard_normal(k * n).astype(np.float32)

    def program(d):
        ta, tat = d.new_tensor_by_vector(S([m, k]), a), d.new_tensor_by_vector(S([k, m]), at)
        x = d.new_tensor_by_vector(S([k, n]), b)
        outs = []
        for _ in range(10):
            y = d.matmul_fw(ta, x)          # reads x
            x_old = x
            x = d.matmul_fw(tat, y)         # new x; the old one goes back to the pool below
            del x_old                       # its block is the next raw tensor of that size
            outs.append(y.to_vector() if len(outs) % 3 == 0 else None)
        outs = [o for o in outs if o is not None]
        return outs + [x.to_vector()]

    lanes, in_order = _run_both(program)
    _same_bits(lanes, in_order)
    assert norm_rel_err(in_order[0], oracle.matmul_fw(a, b, m, k, n, 1, 1)) <= 1e-4


def test_random_programs_give_the_same_bits_with_and_without_lanes():
    n = 256
    for seed in range(6):
        rng = np.random.default_rng(100 + seed)
        init = [rng.standard_normal(n * n).astype(np.float32) / np.sqrt(n) for _ in range(6)]
        ops = []
        for _ in range(60):
            kind = rng.choice(["fw", "fw", "bw", "tanh", "add", "read"])
            ops.append((kind,) + tuple(int(v) for v in rng.integers(0, 6, 5)))

        def program(d):
            ts = [d.new_tensor_by_vector(S([n, n]), v) for v in init]
            outs = []
            for kind, i, j, k2, l, q in ops:
                if kind == "fw":
                    ts[k2] = d.matmul_fw(ts[i], ts[j])
                elif kind == "bw":
                    if len({i, j, k2, l, q}) < 5:
                        continue                      # operands and gradients must be distinct tensors
                    d.matmul_bw(ts[i], ts[j], ts[k2], ts[k2], ts[l], ts[q])
                elif kind == "tanh":
                    ts[j] = d.unary_fw("tanh", ts[i])
                elif kind == "add":
                    if i != j:
                        d.inplace_add(ts[i], ts[j])
                else:
                    outs.append(ts[i].to_vector())
            return outs + [t.to_vector() for t in ts]

        lanes, in_order = _run_both(program)
        _same_bits(lanes, in_order)
        assert all(np.isfinite(v).all() for v in in_order)


def test_switching_the_lanes_off_and_on():
    m, k, n = 512, 512, 64
    rng = np.random.default_rng(5)
    a = rng.standard_normal(m * k).astype(np.float32) / np.sqrt(k)
    b = rng.standard_normal(k * n).astype(np.float32)
    d = pa.HIP(0)
    try:
        ta, tb = d.new_tensor_by_vector(S([m, k]), a), d.new_tensor_by_vector(S([k, n]), b)
        want = oracle.matmul_fw(a, b, m, k, n, 1, 1)
        for on in (True, False, True):
            d.set_overlap(on)
            ys = [d.matmul_fw(ta, tb) for _ in range(4)]
            for y in ys:
                assert norm_rel_err(y.to_vector(), want) <= 1e-4
    finally:
        d.close()


def test_default_policy_long_runs_of_calls_and_runs_cut_short():
    # default settings: the second lane is engaged by the sixth matmul call in a row and released by
    # any other operation; results as in order either way
    m, k, n = 650, 650, 64
    rng = np.random.default_rng(6)
    a = rng.standard_normal(m * k).astype(np.float32) / np.sqrt(k)
    bs = [rng.standard_normal(k * n).astype(np.float32) for _ in range(4)]

    def program(d):
        ta = d.new_tensor_by_vector(S([m, k]), a)
        tb = [d.new_tensor_by_vector(S([k, n]), b) for b in bs]
        ga = d.new_tensor_by_constant(S([m, k]), 0)
        gb = [d.new_tensor_by_constant(S([k, n]), 0) for _ in bs]
        outs = []
        for run in (40, 3, 7, 12, 2, 30):                 # matmul calls in a row, then another kind of operation
            ys = []
            for i in range(run):
                y = d.matmul_fw(ta, tb[i % 4])
                d.matmul_bw(ta, tb[i % 4], y, y, ga, gb[i % 4])
                ys.append(y)
                if i % 5 == 4:
                    outs.append(y.to_vector())            # a read-back in the middle of a run: the lanes stay engaged
                if i % 11 == 10:
                    d.sync()
            h = d.unary_fw("tanh", ys[-1])
            outs += [h.to_vector(), ys[0].to_vector()]
        return outs + [ga.to_vector()] + [g.to_vector() for g in gb]

    results = []
    for overlap in (True, False):
        d = pa.HIP(0)
        d.set_deterministic(True)
        d.set_overlap(overlap)
        try:
            results.append([np.asarray(v, dtype=np.float32) for v in program(d)])
        finally:
            d.close()
    _same_bits(*results)


def test_gradients_reset_between_calls_as_a_backward_pass_does():
    # new gradient tensor, zero fill, products added into it, the tensor handed back: per timestep, as
    # primitiv's backward pass does; the fill takes a lane like a product
    m, k, n = 650, 650, 64
    rng = np.random.default_rng(7)
    a = rng.standard_normal(m * k).astype(np.float32) / np.sqrt(k)
    steps = 24
    bs = [rng.standard_normal(k * n).astype(np.float32) for _ in range(4)]
    gys = [rng.standard_normal(m * n).astype(np.float32) for _ in range(4)]

    def program(d):
        ta = d.new_tensor_by_vector(S([m, k]), a)
        tb = [d.new_tensor_by_vector(S([k, n]), b) for b in bs]
        tgy = [d.new_tensor_by_vector(S([m, n]), g) for g in gys]
        ga = d.new_tensor_by_constant(S([m, k]), 0)
        outs = []
        for t in range(steps):
            y = d.matmul_fw(ta, tb[t % 4])
            gb = d.new_tensor_by_constant(S([k, n]), 0)       # pool block of the previous timestep, refilled
            d.matmul_bw(ta, tb[t % 4], y, tgy[t % 4], ga, gb)
            if t % 6 == 5:
                outs += [gb.to_vector(), y.to_vector()]
            del gb, y
        return outs + [ga.to_vector()]

    for deterministic in (True, False):
        results = []
        for overlap in (True, False):
            d = pa.HIP(0)
            d.set_deterministic(deterministic)
            d.set_overlap(overlap)
            try:
                results.append([np.asarray(v, dtype=np.float32) for v in program(d)])
            finally:
                d.close()
        if deterministic:
            _same_bits(*results)
        else:
            for got, want in zip(*results):
                assert norm_rel_err(got, want) <= 1e-5
    _, gb = oracle.matmul_bw(a, bs[1], gys[1], np.zeros(m * k, np.float32), np.zeros(k * n, np.float32), m, k, n, 1, 1)
    assert norm_rel_err(results[1][0], gb) <= 1e-4      # timestep 5 uses operands 5 % 4 = 1


def test_scratch_of_a_split_product_never_becomes_a_tensor_of_the_other_lane():
    # A forward product with few output tiles and a long K meets through partial tiles in scratch
    # memory, which goes back to its pool when the launch has been enqueued.  The outputs allocated
    # next cover every power-of-two size class that scratch block can have, and their products have
    # operands of their own, so they run on the other lane: if a scratch block could come back as one
    # of them, it would be overwritten under the first product.  Also the other way round: tensors
    # released while a product on the other lane may still read them.
    m, k, n = 96, 4000, 15
    rng = np.random.default_rng(8)
    a = rng.standard_normal(m * k).astype(np.float32) / np.sqrt(k)
    b = rng.standard_normal(k * n).astype(np.float32)
    small_a = rng.standard_normal(64 * 8).astype(np.float32)
    classes = [1 << s for s in range(12, 23)]               # 4 KiB ... 4 MiB outputs
    small_b = {c: rng.standard_normal(8 * (c // 256)).astype(np.float32) for c in classes}

    def program(d):
        ta, tb = d.new_tensor_by_vector(S([m, k]), a), d.new_tensor_by_vector(S([k, n]), b)
        tsa = d.new_tensor_by_vector(S([64, 8]), small_a)
        tsb = {c: d.new_tensor_by_vector(S([8, c // 256]), small_b[c]) for c in classes}
        outs = []
        for it in range(6):
            y = d.matmul_fw(ta, tb)                          # split: partial tiles in scratch
            fresh = [d.matmul_fw(tsa, tsb[c]) for c in classes]   # new outputs of every class, other operands
            y2 = d.matmul_fw(ta, tb)                         # again, while the small products are in flight
            outs += [y.to_vector(), y2.to_vector(), fresh[it % len(fresh)].to_vector()]
            del fresh                                        # blocks back to the pool for the next round
        return outs

    lanes, in_order = _run_both(program)
    _same_bits(lanes, in_order)
    want = oracle.matmul_fw(a, b, m, k, n, 1, 1)
    for i in range(0, len(in_order), 3):
        assert norm_rel_err(lanes[i], want) <= 1e-4 and norm_rel_err(lanes[i + 1], want) <= 1e-4


@pytest.mark.parametrize("storage", ["f16", "bf16"])
@pytest.mark.parametrize("m,k,n", [(2048, 512, 64), (1000, 650, 64), (96, 200, 16)])
def test_sixteen_bit_products_on_two_lanes(storage, m, k, n):
    # the per-timestep products of the 16-bit devices take lanes like the fp32 ones: forward products that
    # feed one another, gradients accumulated by calls on different lanes, gradients reset per timestep
    rng = np.random.default_rng(9)
    a = rng.standard_normal(m * k).astype(np.float32) / np.sqrt(k)
    at = rng.standard_normal(k * m).astype(np.float32) / np.sqrt(m)
    bs = [rng.standard_normal(k * n).astype(np.float32) for _ in range(4)]
    gys = [rng.standard_normal(m * n).astype(np.float32) for _ in range(4)]

    def program(d):
        ta, tat = d.new_tensor_by_vector(S([m, k]), a), d.new_tensor_by_vector(S([k, m]), at)
        tb = [d.new_tensor_by_vector(S([k, n]), b) for b in bs]
        tgy = [d.new_tensor_by_vector(S([m, n]), g) for g in gys]
        ga = d.new_tensor_by_constant(S([m, k]), 0)
        outs = []
        x = tb[0]
        for t in range(12):
            y = d.matmul_fw(ta, tb[t % 4])                     # independent of the chain below
            gb = d.new_tensor_by_constant(S([k, n]), 0)        # reset per timestep: the pool's block of the last one
            d.matmul_bw(ta, tb[t % 4], y, tgy[t % 4], ga, gb)  # every call adds into ga
            y2 = d.matmul_fw(ta, x)                            # a chain: x -> y2 -> x
            x = d.matmul_fw(tat, y2)
            if t % 4 == 3:
                outs += [y.to_vector(), gb.to_vector(), x.to_vector()]
            del gb, y, y2
        return outs + [ga.to_vector()]

    lanes, in_order = _run_both(program, storage=storage)
    _same_bits(lanes, in_order)
    want = oracle.matmul_fw(a, bs[3], m, k, n, 1, 1)
    assert norm_rel_err(in_order[0], want) <= 2e-2
