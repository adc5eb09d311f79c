"""Random tensors of the HIP devices against the oracle's Philox stream and the
properties the reference's device tests check (test/cuda_device_test.cc:81-240:
a seed fixes the stream, unseeded devices differ, an odd count is a prefix)."""
import numpy as np
import pytest

import oracle
import primitiv_amd as pa

pytestmark = pytest.mark.gpu

S = pa.Shape


@pytest.mark.parametrize("n", [1, 3, 4, 63, 1000, (1 << 20) + 1])
def test_stream_matches_oracle(n):
    dev = pa.HIP(0, 12345)
    u = dev.random_uniform(S([n]), -9, 9).to_vector()
    assert np.array_equal(u, oracle.random("uniform", 12345, 0, -9.0, 9.0, n))
    off = (n + 3) // 4                      # the next call continues the stream
    b = dev.random_bernoulli(S([n]), 0.3).to_vector()
    assert np.array_equal(b, oracle.random("bernoulli", 12345, off, 0.3, 0.0, n))
    z = dev.random_normal(S([n]), 1, 3).to_vector()
    assert np.allclose(z, oracle.random("normal", 12345, 2 * off, 1.0, 3.0, n), rtol=1e-5, atol=1e-5)
    ln = dev.random_log_normal(S([n]), 0.5, 0.25).to_vector()
    assert np.allclose(ln, oracle.random("log_normal", 12345, 3 * off, 0.5, 0.25, n), rtol=1e-5)


def test_seed_fixes_the_stream_and_unseeded_devices_differ():
    a = pa.HIP(0, 12345).random_uniform(S([4, 4], 4), -9, 9).to_vector()
    b = pa.HIP(0, 12345).random_uniform(S([4, 4], 4), -9, 9).to_vector()
    assert np.array_equal(a, b)
    odd = pa.HIP(0, 12345).random_uniform(S([3, 3], 7), -9, 9).to_vector()
    assert np.array_equal(odd, a[:63])      # test/cuda_device_test.cc:174-186
    history = [pa.HIP(0).random_normal(S([2, 2], 2), 1, 3).to_vector() for _ in range(10)]
    for i in range(10):
        for j in range(i):
            assert not np.array_equal(history[i], history[j])


def test_moments_and_half_storage():
    n = 1 << 20
    dev = pa.HIP(0, 7)
    z = dev.random_normal(S([n]), 0, 1).to_vector()
    assert abs(z.mean()) < 5e-3 and abs(z.std() - 1) < 5e-3
    b = dev.random_bernoulli(S([n]), 0.3).to_vector()
    assert abs(b.mean() - 0.3) < 2e-3
    for storage in ("f16", "bf16"):
        d16 = pa.HIP16(0, 7, storage=storage)
        u = d16.random_uniform(S([1000], 3), -1, 1).to_vector()
        want = oracle.random("uniform", 7, 0, -1.0, 1.0, 3000)
        assert np.max(np.abs(u - want)) <= 2e-2
        assert np.array_equal(d16.random_bernoulli(S([1000]), 0.5).to_vector(),
                              oracle.random("bernoulli", 7, 750, 0.5, 0.0, 1000))


def test_invalid_parameters():
    dev = pa.HIP(0)
    for call in (lambda: dev.random_bernoulli(S([2]), 1.5), lambda: dev.random_uniform(S([2]), 1, 0),
                 lambda: dev.random_normal(S([2]), 0, 0), lambda: dev.random_log_normal(S([2]), 0, -1)):
        with pytest.raises(pa.Error):
            call()
