"""The five benchmark workloads of the matmul path and their seeded inputs.

Inputs are drawn on the host with the randomizer that restates primitiv's
`DefaultRandomizer` (primitiv/core/random.h:15-87; std::mt19937 + one
standard-library distribution per fill), so every device sees bit-identical
values.  Draw order per workload: one generator seeded with `seed`; W (or a)
first, then for each timestep its b, then its gy.
"""
import ctypes
import math

import numpy as np

from . import _lib


class Randomizer:
    def __init__(self, seed):
        self._r = ctypes.c_void_p()
        _lib.call("phip_randomizer_create", int(seed), ctypes.byref(self._r))

    def __del__(self):
        try:
            if self._r:
                _lib.lib().phip_randomizer_destroy(self._r)
        except Exception:
            pass

    def uniform(self, lower, upper, n):
        out = np.empty(n, dtype=np.float32)
        _lib.call("phip_randomizer_fill_uniform", self._r, lower, upper, n, out.ctypes.data)
        return out

    def normal(self, mean, sd, n):
        out = np.empty(n, dtype=np.float32)
        _lib.call("phip_randomizer_fill_normal", self._r, mean, sd, n, out.ctypes.data)
        return out


class Workload:
    def __init__(self, name, di, dj, dk, ba, bb, steps, a_dist, b_dist, gy_dist, storage="f32",
                 tolerance=1e-4, note=""):
        self.name, self.di, self.dj, self.dk = name, di, dj, dk
        self.ba, self.bb, self.steps = ba, bb, steps
        self.a_dist, self.b_dist, self.gy_dist = a_dist, b_dist, gy_dist
        self.storage, self.tolerance, self.note = storage, tolerance, note

    @property
    def bs(self):
        return max(self.ba, self.bb)

    def sizes(self):
        return (self.di * self.dj * self.ba, self.dj * self.dk * self.bb, self.di * self.dk * self.bs)

    def flops_per_step(self):
        """fw + both gradients: 3 products of 2*di*dj*dk flops per sample."""
        return 3 * 2 * self.di * self.dj * self.dk * self.bs

    def bytes_per_step(self):
        """Algorithmic traffic: fw reads a, b and writes y; bw reads a, b, gy
        and reads and writes ga, gb; every tensor counted once."""
        na, nb, ny = self.sizes()
        item = 4 if self.storage == "f32" else 2
        return item * ((na + nb + ny) + (na + nb + ny) + 2 * (na + nb))

    def _draw(self, rng, dist, n):
        kind, p, q = dist
        return rng.uniform(p, q, n) if kind == "uniform" else rng.normal(p, q, n)

    def inputs(self, seed=0, steps=None):
        """Returns (a, [b_t], [gy_t]) as flat float32 arrays."""
        steps = self.steps if steps is None else steps
        rng = Randomizer(seed)
        na, nb, ny = self.sizes()
        a = self._draw(rng, self.a_dist, na)
        bs, gys = [], []
        for _ in range(steps):
            bs.append(self._draw(rng, self.b_dist, nb))
            gys.append(self._draw(rng, self.gy_dist, ny))
        return a, bs, gys


_XAVIER = math.sqrt(6.0 / (256 + 784))  # primitiv/core/initializer_impl.cc:34-42

WORKLOADS = {
    # broadcast dense layer: W {256,784}, x {784} x 128
    "dense": Workload("dense", 256, 784, 1, 1, 128, 1,
                      ("uniform", -_XAVIER, _XAVIER), ("uniform", 0.0, 1.0), ("normal", 0.0, 1.0)),
    # recurrent gate: W {2048,512}, h {512} x 64, 30 timesteps, gW accumulates
    "rnn_gate": Workload("rnn_gate", 2048, 512, 1, 1, 64, 30,
                         ("uniform", -0.1, 0.1), ("normal", 0.0, 1.0), ("normal", 0.0, 1.0)),
    # square batched: a, b, gy {1024,1024} x 16
    "square_batched": Workload("square_batched", 1024, 1024, 1024, 16, 16, 1,
                               ("normal", 0.0, 1.0), ("normal", 0.0, 1.0), ("normal", 0.0, 1.0)),
    # output projection: W {10000,650}, h {650} x 64, 35 timesteps
    "output_projection": Workload("output_projection", 10000, 650, 1, 1, 64, 35,
                                  ("uniform", -0.05, 0.05), ("normal", 0.0, 1.0), ("normal", 0.0, 1e-2),
                                  note="h ~ N(0,1) (not stated by the workload definition)"),
    # half storage: a {4096,4096}, b, gy {4096,4096} x 8
    "half_storage": Workload("half_storage", 4096, 4096, 4096, 1, 8, 1,
                             ("normal", 0.0, 0.02), ("normal", 0.0, 1.0), ("normal", 0.0, 1.0),
                             storage="f16", tolerance=2e-2),
}
