"""The oracle's random tensors: the generator against the published
known-answer vectors, the distributions against their moments."""
import numpy as np

import oracle


def test_philox_known_answers():
    # Random123's kat_vectors for philox4x32, 10 rounds (Salmon et al., SC'11)
    kat = [
        ([0] * 4, [0] * 2, [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
        ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
        ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
         [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]),
    ]
    for counter, key, want in kat:
        assert oracle.philox4x32_10(counter, key) == want


def test_stream_layout():
    # element i is word i%4 of block offset + i/4: a shorter draw is a prefix, and
    # moving the offset by one block drops four elements
    a = oracle.random("uniform", 12345, 0, 0.0, 1.0, 64)
    assert np.array_equal(oracle.random("uniform", 12345, 0, 0.0, 1.0, 37), a[:37])
    assert np.array_equal(oracle.random("uniform", 12345, 1, 0.0, 1.0, 60), a[4:])
    assert not np.array_equal(oracle.random("uniform", 12346, 0, 0.0, 1.0, 64), a)
    w = oracle.philox4x32_10([3, 0, 0, 0], [12345, 0])
    assert np.array_equal(a[12:16], [((v >> 8) + 1) * 2.0 ** -24 for v in w])


def test_distributions():
    n = 1 << 20
    u = oracle.random("uniform", 1, 0, -9.0, 9.0, n)
    assert u.min() > -9.0 and u.max() <= 9.0                  # (lower, upper]
    assert abs(u.mean()) < 0.03 and abs(u.var() - 27.0) < 0.1
    b = oracle.random("bernoulli", 2, 0, 0.3, 0.0, n)
    assert set(np.unique(b)) == {0.0, 1.0} and abs(b.mean() - 0.3) < 2e-3
    z = oracle.random("normal", 3, 0, 1.0, 3.0, n)
    assert abs(z.mean() - 1.0) < 0.02 and abs(z.std() - 3.0) < 0.02
    zs = (z - 1.0) / 3.0
    assert abs((zs ** 3).mean()) < 0.02 and abs((zs ** 4).mean() - 3.0) < 0.05
    assert abs(np.corrcoef(zs[0::2], zs[1::2])[0, 1]) < 5e-3  # the two halves of a Box-Muller pair
    ln = oracle.random("log_normal", 4, 0, 0.5, 0.25, n)
    assert np.allclose(np.log(ln), oracle.random("normal", 4, 0, 0.5, 0.25, n), atol=1e-5)
