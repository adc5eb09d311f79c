"""A whole small network through the device: the 3-layer perceptron of the
reference's graph test (test/graph_test.cc:362-435, every node value is a
golden vector there), forward and backward, op by op as primitiv's graph
would call the device."""
import numpy as np
import pytest

import primitiv_amd as pa

pytestmark = pytest.mark.gpu

S = pa.Shape


@pytest.fixture(scope="module", params=["f32", "f16", "bf16"])
def dev(request):
    return pa.HIP(0) if request.param == "f32" else pa.HIP16(0, storage=request.param)


def test_xor_perceptron_forward_and_backward(dev):
    f32 = dev._SUFFIX == "f32"
    x = dev.new_tensor_by_vector(S([2], 4), [1, 1, 1, -1, -1, 1, -1, -1])
    w1 = dev.new_tensor_by_vector(S([2, 2]), [1, -1, 1, -1])
    b1 = dev.new_tensor_by_vector(S([2]), [-1, -1])
    w2 = dev.new_tensor_by_vector(S([1, 2]), [1, 1])
    b2 = dev.new_tensor_by_vector(S([]), [1])
    t = dev.new_tensor_by_vector(S([], 4), [1, -1, -1, 1])

    n5 = dev.matmul_fw(w1, x)
    n6 = dev.binary_fw("add", n5, b1)
    n7 = dev.unary_fw("tanh", n6)
    n8 = dev.matmul_fw(w2, n7)
    n9 = dev.binary_fw("add", n8, b2)
    n11 = dev.binary_fw("subtract", n9, t)
    n12 = dev.binary_fw("multiply", n11, n11)
    n13 = dev.batch_sum_fw(n12)

    h1, h2, h3, h4 = .76159416, .99505475, -.23346060, -1.5231883
    h5, h6, h7 = .76653940, -.52318831, .47681169
    expected = [
        (n5, [2, -2, 0, 0, 0, 0, -2, 2]), (n6, [1, -3, -1, -1, -1, -1, -3, 1]),
        (n7, [h1, -h2, -h1, -h1, -h1, -h1, -h2, h1]), (n8, [h3, h4, h4, h3]), (n9, [h5, h6, h6, h5]),
        (n11, [h3, h7, h7, h3]), (n12, [h3 * h3, h7 * h7, h7 * h7, h3 * h3]), (n13, [2 * (h3 * h3 + h7 * h7)]),
    ]
    for node, want in expected:
        got, want = node.to_vector(), np.asarray(want, dtype=np.float32)
        if f32:
            # the test's constants carry 8 digits; differences such as h3 = tanh(1) - tanh(3) lose a few more
            assert np.allclose(got, want, rtol=0, atol=2e-7), (got, want)
        else:
            assert np.allclose(got, want, rtol=0, atol=2e-2), (got, want)

    # backward, in the order primitiv's Graph::backward walks the operators
    zeros = lambda like: dev.new_tensor_by_constant(like.shape(), 0)
    g13 = dev.new_tensor_by_constant(n13.shape(), 1)
    g12 = zeros(n12)
    dev.inplace_add(g13, g12)                       # batch::sum backward: gx += gy
    g11 = zeros(n11)
    dev.binary_bw("multiply", n11, n11, n12, g12, g11, g11)   # both operands are node 11
    g9, gt = zeros(n9), zeros(t)
    dev.binary_bw("subtract", n9, t, n11, g11, g9, gt)
    g8, gb2 = zeros(n8), zeros(b2)
    dev.binary_bw("add", n8, b2, n9, g9, g8, gb2)
    gw2, g7 = zeros(w2), zeros(n7)
    dev.matmul_bw(w2, n7, n8, g8, gw2, g7)
    g6 = zeros(n6)
    dev.unary_bw("tanh", n6, n7, g7, g6)
    g5, gb1 = zeros(n5), zeros(b1)
    dev.binary_bw("add", n5, b1, n6, g6, g5, gb1)
    gw1, gx = zeros(w1), zeros(x)
    dev.matmul_bw(w1, x, n5, g5, gw1, gx)

    # the same derivative in float64
    X = np.array([[1, 1], [1, -1], [-1, 1], [-1, -1]], dtype=np.float64)        # samples x inputs
    W1 = np.array([[1, 1], [-1, -1]], dtype=np.float64)                         # rows x cols of the column-major {1,-1,1,-1}
    B1, W2, B2, T = np.array([-1., -1.]), np.array([1., 1.]), 1.0, np.array([1., -1., -1., 1.])
    A = X @ W1.T + B1
    H = np.tanh(A)
    Y = H @ W2 + B2
    D = 2 * (Y - T)                                                              # dL/dy per sample
    GW2, GB2 = D @ H, D.sum()
    GA = np.outer(D, W2) * (1 - H ** 2)
    GW1, GB1 = GA.T @ X, GA.sum(axis=0)
    tol = 1e-5 if f32 else 3e-2
    assert np.allclose(gw2.to_vector(), GW2, atol=tol)
    assert np.allclose(gb2.to_vector(), [GB2], atol=tol)
    assert np.allclose(gb1.to_vector(), GB1, atol=tol)
    assert np.allclose(gw1.to_vector(), GW1.T.reshape(-1), atol=tol)             # back to column-major
    assert np.allclose(gt.to_vector(), -D, atol=tol)


def test_matmul_gradients_of_one_tensor_used_twice(dev):
    # a . a hands the same gradient tensor to both operands (primitiv/core/graph.cc:205-216)
    rng = np.random.default_rng(0)
    n = 96
    a = rng.standard_normal(n * n).astype(np.float32)
    gy = rng.standard_normal(n * n).astype(np.float32)
    ta = dev.new_tensor_by_vector(S([n, n]), a)
    tgy = dev.new_tensor_by_vector(S([n, n]), gy)
    y = dev.matmul_fw(ta, ta)
    g = dev.new_tensor_by_constant(S([n, n]), 0)
    dev.matmul_bw(ta, ta, y, tgy, g, g)
    A = ta.to_vector().reshape(n, n).T.astype(np.float64)
    G = tgy.to_vector().reshape(n, n).T.astype(np.float64)
    want = (G @ A.T + A.T @ G).T.reshape(-1)
    tol = 1e-4 if dev._SUFFIX == "f32" else 2e-2
    assert np.max(np.abs(g.to_vector() - want)) <= tol * np.max(np.abs(want))
