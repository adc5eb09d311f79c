"""Every other family of Device virtuals of the C++ class primitiv::devices::HIP
(elementwise, moving and reducing along a dimension, random tensors,
convolution and pooling), run on the CPU against the real primitiv core with a
host stand-in for libphip (see test_host_class_runs.py).

The cases and bounds are those of the GPU tests - the reference's own golden
vectors replayed through Device::tanh_fw, Device::pick_bw, ... - so a virtual
that forwards the wrong operation code, swaps two operands or computes an
offset wrongly fails here without a GPU.
"""
import numpy as np
import pytest

import conv_pool_cases
import host_class_lib as hc
import indexing_cases
import oracle
import pointwise_cases
import primitiv_amd as pa
import test_gpu_conv_pool
import test_gpu_indexing
import test_gpu_pointwise

pytestmark = pytest.mark.skipif(not hc.available(), reason=hc.REASON)

S = pa.Shape


@pytest.fixture(scope="module")
def dev():
    d = hc.HostDevice("f32")
    yield d
    d.close()


@pytest.fixture(scope="module", params=["f16", "bf16"])
def dev16(request):
    d = hc.HostDevice(request.param)
    yield d
    d.close()


@pytest.mark.parametrize("case", pointwise_cases.CASES, ids=pointwise_cases.case_id)
def test_elementwise_reference_vectors(dev, case):
    test_gpu_pointwise.test_f32_matches_reference_vectors(dev, case)


@pytest.mark.parametrize("case", pointwise_cases.CASES, ids=pointwise_cases.case_id)
def test_elementwise_reference_vectors_half_storage(dev16, case):
    test_gpu_pointwise.test_half_storage_matches_reference_vectors(dev16, case)


@pytest.mark.parametrize("case", indexing_cases.CASES, ids=indexing_cases.case_id)
def test_dimension_ops_reference_tables(dev, case):
    test_gpu_indexing.test_f32_matches_reference_tables(dev, case)


@pytest.mark.parametrize("case", indexing_cases.CASES, ids=indexing_cases.case_id)
def test_dimension_ops_reference_tables_half_storage(dev16, case):
    test_gpu_indexing.test_half_storage_matches_reference_tables(dev16, case)


@pytest.mark.parametrize("dims,batch", [([7], 1), ([5, 3], 4), ([3, 4, 5], 3), ([2, 3, 2, 3], 2)])
def test_dimension_ops_random(dev, dims, batch):
    # slices, concatenation, flips, permutations, reductions and their gradients on asymmetric shapes
    test_gpu_indexing.test_dimension_ops_match_oracle(dev, dims, batch)


@pytest.mark.parametrize("kc", conv_pool_cases.CASES, ids=conv_pool_cases.case_id)
def test_convolution_and_pooling_reference_vectors(dev, kc):
    test_gpu_conv_pool.test_reference_vectors(dev, kc)


def test_random_tensors_follow_the_seeded_stream():
    # the class owns the position in the stream: every call moves it on by ceil(n / 4) blocks
    n = 63
    d = hc.HostDevice("f32", seed=12345)
    off = (n + 3) // 4
    assert np.array_equal(d.random_uniform(S([n]), -9, 9).to_vector(), oracle.random("uniform", 12345, 0, -9.0, 9.0, n))
    assert np.array_equal(d.random_bernoulli(S([n]), 0.3).to_vector(),
                          oracle.random("bernoulli", 12345, off, 0.3, 0.0, n))
    assert np.allclose(d.random_normal(S([n]), 1, 3).to_vector(), oracle.random("normal", 12345, 2 * off, 1.0, 3.0, n),
                       rtol=1e-6)
    assert np.allclose(d.random_log_normal(S([3, 7], 3), 0.5, 0.25).to_vector(),
                       oracle.random("log_normal", 12345, 3 * off, 0.5, 0.25, n), rtol=1e-6)
    d.close()
    a = hc.HostDevice("f32", seed=5).random_uniform(S([4, 4], 4), -9, 9).to_vector()
    b = hc.HostDevice("f32", seed=5).random_uniform(S([4, 4], 4), -9, 9).to_vector()
    c = hc.HostDevice("f32", seed=6).random_uniform(S([4, 4], 4), -9, 9).to_vector()
    assert np.array_equal(a, b) and not np.array_equal(a, c)
