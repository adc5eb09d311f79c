"""Zero fills that are only noted (phip_set_deferred_zero_fill): a fill with +0 launches nothing, the
gradient operation that follows writes instead of adding, and every other entry point sees the
memory as if the fill had run.  Each case runs with the notes on and with every fill launched at
once and asks for the same bits; the values themselves are checked against numpy."""
import ctypes

import numpy as np
import pytest

import primitiv_amd as pa
from primitiv_amd import _lib

pytestmark = pytest.mark.gpu

S = pa.Shape
STORAGES = ["f32", "f16", "bf16"]


def _device(storage, deferred):
    d = pa.HIP(0) if storage == "f32" else pa.HIP16(0, storage=storage)
    d.set_deferred_zero_fill(deferred)
    return d


def _both(storage, program):
    out = []
    for deferred in (True, False):
        d = _device(storage, deferred)
        try:
            out.append([np.asarray(v, dtype=np.float32) for v in program(d)])
        finally:
            d.close()
    assert len(out[0]) == len(out[1])
    for i, (x, y) in enumerate(zip(*out)):
        assert x.shape == y.shape and np.array_equal(x.view(np.uint32), y.view(np.uint32)), "result %d differs" % i
    return out[0]


def _tol(storage):
    return 1e-6 if storage == "f32" else 2e-2


@pytest.mark.parametrize("storage", STORAGES)
@pytest.mark.parametrize("n,bs", [(2600, 64), (7, 3), (1, 1), (4099, 2)])
def test_gradient_operations_into_fresh_zeros(storage, n, bs):
    rng = np.random.default_rng(n + bs)
    x = rng.uniform(-1, 1, n * bs).astype(np.float32)
    y = rng.uniform(-1, 1, n * bs).astype(np.float32)
    g = rng.uniform(-1, 1, n * bs).astype(np.float32)
    bias = rng.uniform(-1, 1, n).astype(np.float32)

    def program(d):
        tx, ty, tg = (d.new_tensor_by_vector(S([n], bs), v) for v in (x, y, g))
        tb = d.new_tensor_by_vector(S([n]), bias)
        outs = []
        gx = d.new_tensor_by_constant(S([n], bs), 0)
        d.unary_bw("tanh", tx, ty, tg, gx)                          # gx = (1 - y^2) g
        outs.append(gx.to_vector())
        d.unary_bw("tanh", tx, ty, tg, gx)                          # a second call adds
        outs.append(gx.to_vector())
        gx = d.new_tensor_by_constant(S([n], bs), 0)
        d.const_bw("multiply_const", tx, ty, tg, 3.0, gx)
        outs.append(gx.to_vector())
        ga, gb = d.new_tensor_by_constant(S([n], bs), 0), d.new_tensor_by_constant(S([n], bs), 0)
        d.binary_bw("multiply", tx, ty, tx, tg, ga, gb)             # both gradients fresh
        outs += [ga.to_vector(), gb.to_vector()]
        ga = d.new_tensor_by_constant(S([n], bs), 0)
        d.binary_bw("multiply", tx, ty, tx, tg, ga, gb)             # one fresh, one holding values
        outs += [ga.to_vector(), gb.to_vector()]
        g2 = d.new_tensor_by_constant(S([n], bs), 0)
        d.binary_bw("multiply", tx, tx, tx, tg, g2, g2)             # x * x: one gradient tensor for both operands
        outs.append(g2.to_vector())
        gfull, gbias = d.new_tensor_by_constant(S([n], bs), 0), d.new_tensor_by_constant(S([n]), 0)
        d.binary_bw("add", tx, tb, tx, tg, gfull, gbias)            # bias: gradient summed over the minibatch
        outs += [gfull.to_vector(), gbias.to_vector()]
        gfull = d.new_tensor_by_constant(S([n], bs), 0)
        d.binary_bw("add", tb, tx, tx, tg, gbias, gfull)            # the shared operand on the left; gbias adds
        outs += [gfull.to_vector(), gbias.to_vector()]
        acc = d.new_tensor_by_constant(S([n], bs), 0)
        d.inplace_add(tx, acc)                                      # acc = x
        outs.append(acc.to_vector())
        acc1 = d.new_tensor_by_constant(S([n]), 0)
        d.inplace_add(tg, acc1)                                     # summed over the minibatch
        outs.append(acc1.to_vector())
        accb = d.new_tensor_by_constant(S([n], bs), 0)
        d.inplace_add(tb, accb)                                     # shared x repeated per sample
        outs.append(accb.to_vector())
        sub = d.new_tensor_by_constant(S([n], bs), 0)
        d.inplace_subtract(tx, sub)
        outs.append(sub.to_vector())
        return outs

    got = _both(storage, program)
    if storage == "f32":
        t = _tol(storage)
        G = g.reshape(bs, n)
        assert np.allclose(got[0], (1 - y * y) * g, atol=t)
        assert np.allclose(got[1], 2 * (1 - y * y) * g, atol=2 * t)
        assert np.allclose(got[2], 3 * g, atol=4 * t)
        assert np.allclose(got[3], y * g, atol=t) and np.allclose(got[4], x * g, atol=t)
        assert np.allclose(got[5], y * g, atol=t) and np.allclose(got[6], 2 * x * g, atol=2 * t)
        assert np.allclose(got[7], 2 * x * g, atol=2 * t)
        assert np.allclose(got[8], g, atol=t) and np.allclose(got[9], G.sum(axis=0), atol=bs * t)
        assert np.allclose(got[10], g, atol=t) and np.allclose(got[11], 2 * G.sum(axis=0), atol=2 * bs * t)
        assert np.allclose(got[12], x, atol=t)
        assert np.allclose(got[13], G.sum(axis=0), atol=bs * t)
        assert np.allclose(got[14], np.tile(bias, bs), atol=t)
        assert np.allclose(got[15], -x, atol=t)


@pytest.mark.parametrize("storage", STORAGES)
def test_everything_else_sees_the_zeros(storage):
    n = 1000
    rng = np.random.default_rng(5)
    x = rng.uniform(-1, 1, n).astype(np.float32)
    m = rng.uniform(-1, 1, 64).astype(np.float32)

    def program(d):
        tx = d.new_tensor_by_vector(S([n]), x)
        outs = []
        z = d.new_tensor_by_constant(S([n]), 0)
        outs.append(z.to_vector())                                  # read back at once
        z = d.new_tensor_by_constant(S([n]), 0)
        outs.append(d.unary_fw("exp", z).to_vector())               # an operation that reads it: exp(0) = 1
        z = d.new_tensor_by_constant(S([n]), 0)
        outs.append(d.copy_tensor(z).to_vector())                   # device-to-device copy
        z = d.new_tensor_by_constant(S([n]), 0)
        d.inplace_add(z, tx)                                        # the zeros as the OTHER operand: tx unchanged
        outs.append(tx.to_vector())
        z = d.new_tensor_by_constant(S([n]), 0)
        d.reset_tensor(0.5, z)                                                # a later fill replaces the noted one
        outs.append(z.to_vector())
        d.reset_tensor(0.0, z)
        d.reset_tensor(0.0, z)
        outs.append(z.to_vector())
        z1, z2 = d.new_tensor_by_constant(S([n]), 0), d.new_tensor_by_constant(S([n]), 0)
        d.inplace_add(tx, z1)                                       # takes z1's note only
        outs += [z2.to_vector(), z1.to_vector()]
        zs = [d.new_tensor_by_constant(S([n + i]), 0) for i in range(20)]   # more notes than the list holds
        outs += [t.to_vector() for t in zs]
        big = d.new_tensor_by_constant(S([4, n]), 0)
        part = d.slice_fw(big, 0, 1, 3)                             # a strided read of the zeros
        outs.append(part.to_vector())
        gbig = d.new_tensor_by_constant(S([4, n]), 0)
        d.slice_bw(part, 0, 2, gbig)                                # added into a part of them
        outs.append(gbig.to_vector())
        a = d.new_tensor_by_vector(S([8, 8]), m)
        ga, gb = d.new_tensor_by_constant(S([8, 8]), 0), d.new_tensor_by_constant(S([8, 8]), 0)
        d.matmul_bw(a, a, a, a, ga, gb)                             # products added into noted zeros
        outs += [ga.to_vector(), gb.to_vector()]
        mz = d.new_tensor_by_constant(S([8, 8]), 0)
        outs.append(d.matmul_fw(a, mz).to_vector())                 # zeros as an operand of a product
        nz = d.new_tensor_by_constant(S([n]), -0.0)                 # -0 is not +0: filled at once
        outs.append(nz.to_vector())
        return outs

    got = _both(storage, program)
    assert not got[0].any() and np.allclose(got[1], 1) and not got[2].any()
    assert np.allclose(got[4], 0.5) and not got[5].any() and not got[6].any()
    assert all(not v.any() for v in got[8:28])
    assert not got[28].any() and not got[29].any()
    assert not got[32].any()
    assert np.all(np.signbit(got[33]))


def test_a_block_handed_back_forgets_its_fill_and_stale_notes_never_fire_late():
    # zeros(A); A released; the same block comes back as a raw tensor that is uploaded: the upload wins
    d = _device("f32", True)
    try:
        n = 4096
        for _ in range(5):
            z = d.new_tensor_by_constant(S([n]), 0)
            del z
            t = d.new_tensor_by_vector(S([n]), np.arange(n, dtype=np.float32))     # same size class: same block
            assert np.array_equal(t.to_vector(), np.arange(n, dtype=np.float32))
            del t
        # through the raw entry points: fill noted, block freed, pool emptied (hipFree), other work follows
        p = ctypes.c_void_p()
        _lib.call("phip_pool_alloc", d.ctx(), 1 << 20, ctypes.byref(p), None)
        _lib.call("phip_fill_f32", d.ctx(), p, 0.0, (1 << 20) // 4)
        _lib.call("phip_pool_free", d.ctx(), p)
        _lib.call("phip_pool_release_reserved", d.ctx())
        x = d.new_tensor_by_constant(S([100]), 2.0)
        assert float(x.to_vector()[99]) == 2.0
        # memory of the caller's own pool (phip_malloc / phip_free): the fill is launched before the memory goes
        q = ctypes.c_void_p()
        _lib.call("phip_malloc", d.ctx(), 1 << 16, ctypes.byref(q))
        _lib.call("phip_fill_f32", d.ctx(), q, 0.0, (1 << 16) // 4)
        _lib.call("phip_free", d.ctx(), q)
        d.sync()
    finally:
        d.close()


def test_random_programs_give_the_same_bits_either_way():
    n = 300
    for seed in range(6):
        rng = np.random.default_rng(200 + seed)
        init = [rng.uniform(-1, 1, n).astype(np.float32) for _ in range(5)]
        ops = [(str(rng.choice(["zero", "zero", "tanh_bw", "mul_bw", "add", "read", "exp", "fill"])),) +
               tuple(int(v) for v in rng.integers(0, 5, 4)) for _ in range(80)]

        def program(d):
            ts = [d.new_tensor_by_vector(S([n]), v) for v in init]
            outs = []
            for kind, i, j, k, l in ops:
                if kind == "zero":
                    ts[i] = d.new_tensor_by_constant(S([n]), 0)
                elif kind == "fill":
                    d.reset_tensor(0.0 if j % 2 else 0.25, ts[i])
                elif kind == "tanh_bw":
                    d.unary_bw("tanh", ts[i], ts[j], ts[k], ts[l])
                elif kind == "mul_bw":
                    if k != l:
                        d.binary_bw("multiply", ts[i], ts[j], ts[i], ts[i], ts[k], ts[l])
                elif kind == "add":
                    if i != j:
                        d.inplace_add(ts[i], ts[j])
                elif kind == "exp":
                    ts[j] = d.unary_fw("tanh", ts[i])
                else:
                    outs.append(ts[i].to_vector())
            return outs + [t.to_vector() for t in ts]

        got = _both("f32", program)
        assert all(np.isfinite(v).all() for v in got)
