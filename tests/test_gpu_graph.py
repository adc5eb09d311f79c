"""A whole small network through the device: the 3-layer perceptron of the
reference's graph test (test/graph_test.cc:362-435, every node value is a
golden vector there), forward and backward, op by op as primitiv's graph
would call the device."""
import json
import os

import numpy as np
import pytest

import primitiv_amd as pa
from graph_tape import Tape

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


def test_small_convolutional_network_against_oracle(dev):
    # conv 3x3 -> relu -> 2x2 max pooling, twice, then a dense layer: the layer sequence of the
    # reference's examples/mnist/mnist_cnn (smaller), forward and backward, every node compared
    # with the CPU oracle fed the same values
    import oracle
    from util import norm_rel_err
    tol = 1e-4 if dev._SUFFIX == "f32" else 3e-2
    rng = np.random.default_rng(11)
    bs = 4
    x = rng.standard_normal(12 * 12 * bs).astype(np.float32)
    w1 = (0.4 * rng.standard_normal(3 * 3 * 1 * 4)).astype(np.float32)
    w2 = (0.3 * rng.standard_normal(3 * 3 * 4 * 8)).astype(np.float32)
    w3 = (0.2 * rng.standard_normal(10 * 72)).astype(np.float32)
    conv, pool = (1, 1, 1, 1, 1, 1), (2, 2, 0, 0, 2, 2)
    tx = dev.new_tensor_by_vector(S([12, 12, 1], bs), x)
    tw1 = dev.new_tensor_by_vector(S([3, 3, 1, 4]), w1)
    tw2 = dev.new_tensor_by_vector(S([3, 3, 4, 8]), w2)
    tw3 = dev.new_tensor_by_vector(S([10, 72]), w3)

    # forward on the device
    c1 = dev.conv2d_fw(tx, tw1, *conv)
    r1 = dev.const_fw("prelu", c1, 0.0)
    p1 = dev.max_pool2d_fw(r1, *pool)
    c2 = dev.conv2d_fw(p1, tw2, *conv)
    r2 = dev.const_fw("prelu", c2, 0.0)
    p2 = dev.max_pool2d_fw(r2, *pool)
    assert p2.shape() == S([3, 3, 8], bs)
    flat = dev.new_tensor_by_vector(S([72], bs), p2.to_vector())      # flatten: same memory order
    out = dev.matmul_fw(tw3, flat)

    # the same on the oracle, each layer fed the DEVICE's input of that layer so that
    # 16-bit rounding does not pile up across layers
    def near(t, want, what):
        assert norm_rel_err(t.to_vector(), want) <= tol, what

    near(c1, oracle.conv2d_fw(x, w1, [12, 12, 1], bs, [3, 3, 1, 4], 1, *conv), "conv1")
    near(r1, oracle.const_fw("prelu", c1.to_vector(), 0.0), "relu1")
    near(p1, oracle.max_pool2d_fw(r1.to_vector(), [12, 12, 4], bs, *pool), "pool1")
    near(c2, oracle.conv2d_fw(p1.to_vector(), w2, [6, 6, 4], bs, [3, 3, 4, 8], 1, *conv), "conv2")
    near(p2, oracle.max_pool2d_fw(r2.to_vector(), [6, 6, 8], bs, *pool), "pool2")
    near(out, oracle.matmul_fw(w3, flat.to_vector(), 10, 72, 1, 1, bs), "dense")

    # backward from d(out) = 1, gradients starting at zero
    zeros = lambda like: dev.new_tensor_by_constant(like.shape(), 0)
    g_out = dev.new_tensor_by_constant(out.shape(), 1)
    g_w3, g_flat = zeros(tw3), zeros(flat)
    dev.matmul_bw(tw3, flat, out, g_out, g_w3, g_flat)
    g_p2 = dev.new_tensor_by_vector(p2.shape(), g_flat.to_vector())
    g_r2 = zeros(r2)
    dev.max_pool2d_bw(r2, p2, g_p2, *pool, g_r2)
    g_c2 = zeros(c2)
    dev.const_bw("prelu", c2, r2, g_r2, 0.0, g_c2)
    g_p1, g_w2 = zeros(p1), zeros(tw2)
    dev.conv2d_bw(p1, tw2, c2, g_c2, *conv, g_p1, g_w2)
    g_r1 = zeros(r1)
    dev.max_pool2d_bw(r1, p1, g_p1, *pool, g_r1)
    g_c1 = zeros(c1)
    dev.const_bw("prelu", c1, r1, g_r1, 0.0, g_c1)
    g_x, g_w1 = zeros(tx), zeros(tw1)
    dev.conv2d_bw(tx, tw1, c1, g_c1, *conv, g_x, g_w1)

    z = lambda n: np.zeros(n, np.float32)
    ones = np.ones(10 * bs, np.float32)
    rg_w3, rg_flat = oracle.matmul_bw(w3, flat.to_vector(), ones, z(720), z(72 * bs), 10, 72, 1, 1, bs)
    near(g_w3, rg_w3, "g_w3")
    near(g_flat, rg_flat, "g_flat")
    near(g_r2, oracle.max_pool2d_bw(r2.to_vector(), p2.to_vector(), g_p2.to_vector(), z(6 * 6 * 8 * bs), [6, 6, 8], bs,
                                    *pool), "g_r2")
    near(g_c2, oracle.const_bw("prelu", c2.to_vector(), r2.to_vector(), g_r2.to_vector(), 0.0, z(6 * 6 * 8 * bs)), "g_c2")
    rg_p1, rg_w2 = oracle.conv2d_bw(p1.to_vector(), w2, g_c2.to_vector(), z(6 * 6 * 4 * bs), z(w2.size), [6, 6, 4], bs,
                                    [3, 3, 4, 8], 1, *conv)
    near(g_p1, rg_p1, "g_p1")
    near(g_w2, rg_w2, "g_w2")
    rg_x, rg_w1 = oracle.conv2d_bw(x, w1, g_c1.to_vector(), z(x.size), z(w1.size), [12, 12, 1], bs, [3, 3, 1, 4], 1, *conv)
    near(g_x, rg_x, "g_x")
    near(g_w1, rg_w1, "g_w1")


# ---- the reference's two LSTM graph tests (test/graph_test.cc:437-551, 553-646) -----------------
#
# Both build one LSTM step on a minibatch of two, loss = sum of squares of the new hidden state:
# CheckLSTM with eight weight matrices and four biases, CheckConcatLSTM with the gates' weights
# stacked and `slice` to take the gates apart ("all values and gradients should be same").  What
# the tests hold as numbers - parameters, inputs, operator count and the four losses at 1e-6 - is in
# tests/golden/graph_vectors.json (written from the test's text by extract_graph_vectors.py).

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "graph_vectors.json")) as _f:
    GRAPH_VECTORS = json.load(_f)


def _lstm_float64(case):
    """Values and gradients of the stacked-weights LSTM step in float64 (closed form of one step)."""
    P = case["parameters"]
    col = lambda p: np.asarray(p["values"], dtype=np.float64).reshape(p["shape"][::-1]).T     # column-major
    Wx, Wh, b = col(P["pWx"]), col(P["pWh"]), np.asarray(P["pb"]["values"], dtype=np.float64)
    X = np.asarray(case["inputs"]["x"]["values"], dtype=np.float64).reshape(2, 2)          # samples x inputs
    H = np.asarray(case["inputs"]["h"]["values"], dtype=np.float64).reshape(2, 2)
    sig = lambda v: 1 / (1 + np.exp(-v))
    U = X @ Wx.T + H @ Wh.T + b                                                               # samples x 8
    i, f, o, j = sig(U[:, 0:2]), sig(U[:, 2:4]), sig(U[:, 4:6]), np.tanh(U[:, 6:8])
    c = np.zeros(2)
    cc = f * c + i * j
    hh = o * np.tanh(cc)
    loss = hh * hh
    dhh = 2 * hh
    do, dcc = dhh * np.tanh(cc), dhh * o * (1 - np.tanh(cc) ** 2)
    di, dj, df = dcc * j, dcc * i, dcc * c
    dU = np.concatenate([di * i * (1 - i), df * f * (1 - f), do * o * (1 - o), dj * (1 - j ** 2)], axis=1)
    return {"loss": loss.reshape(-1), "i": i, "f": f, "o": o, "j": j, "cc": cc, "hh": hh,
            "gWx": dU.T @ X, "gWh": dU.T @ H, "gb": dU.sum(axis=0), "gx": dU @ Wx, "gh": dU @ Wh,
            "gc": (dcc * f).sum(axis=0)}


def _colmajor(m):
    return np.asarray(m).T.reshape(-1)


def _lstm_tolerances(dev):
    f32 = dev._SUFFIX == "f32"
    # fp32: the reference's own bound on the losses.  16-bit storage: every node value is rounded to
    # 11 (fp16) or 8 (bf16) significant bits; the losses are squares of values around 0.05 - 0.17.
    return (1e-6, 2e-6) if f32 else ((1e-3, 2e-2) if dev._SUFFIX == "f16" else (4e-3, 5e-2))


def test_lstm_with_separate_gate_weights(dev):
    case, ref = GRAPH_VECTORS["CheckLSTM"], _lstm_float64(GRAPH_VECTORS["CheckConcatLSTM"])
    loss_tol, grad_tol = _lstm_tolerances(dev)
    S, P = pa.Shape, case["parameters"]
    g = Tape(dev)
    x = g.input(S(case["inputs"]["x"]["shape"], 2), case["inputs"]["x"]["values"])
    h = g.input(S(case["inputs"]["h"]["shape"], 2), case["inputs"]["h"]["values"])
    c = g.constant(S([2]), 0)
    names = ["pWix", "pWfx", "pWox", "pWjx", "pWih", "pWfh", "pWoh", "pWjh", "pbi", "pbf", "pbo", "pbj"]
    n = {k: g.input(S(P[k]["shape"]), P[k]["values"]) for k in names}       # parameter nodes, in the test's order

    def gate(act, wx, wh, b):
        return act(g.add(g.add(g.matmul(n[wx], x), g.matmul(n[wh], h)), n[b]))

    i = gate(g.sigmoid, "pWix", "pWih", "pbi")
    f = gate(g.sigmoid, "pWfx", "pWfh", "pbf")
    o = gate(g.sigmoid, "pWox", "pWoh", "pbo")
    j = gate(g.tanh, "pWjx", "pWjh", "pbj")
    cc = g.add(g.multiply(f, c), g.multiply(i, j))
    hh = g.multiply(o, g.tanh(cc))
    t = g.constant(S([2]), 0)
    diff = g.subtract(hh, t)
    loss = g.multiply(diff, diff)
    sum_loss = g.batch_sum(g.sum(loss, 0))
    assert g.num_operators() == case["num_operators"] == 45

    want = np.asarray(case["expected_losses"], dtype=np.float32)
    assert np.allclose(g.value(loss).to_vector(), want, rtol=0, atol=loss_tol)
    assert abs(g.value(sum_loss).to_float() - float(want.sum())) <= 4 * loss_tol
    assert np.allclose(ref["loss"], want, rtol=0, atol=1e-7)                # the float64 closed form agrees with the test
    for node, key in ((i, "i"), (f, "f"), (o, "o"), (j, "j"), (cc, "cc"), (hh, "hh")):
        assert np.allclose(g.value(node).to_vector(), ref[key].reshape(-1), rtol=0, atol=max(loss_tol, grad_tol / 4)), key

    g.backward(sum_loss)
    rows = {"i": slice(0, 2), "f": slice(2, 4), "o": slice(4, 6), "j": slice(6, 8)}
    for gate_name, r in rows.items():
        assert np.allclose(g.gradient(n["pW%sx" % gate_name]).to_vector(), _colmajor(ref["gWx"][r]), rtol=0, atol=grad_tol)
        assert np.allclose(g.gradient(n["pW%sh" % gate_name]).to_vector(), _colmajor(ref["gWh"][r]), rtol=0, atol=grad_tol)
        assert np.allclose(g.gradient(n["pb%s" % gate_name]).to_vector(), ref["gb"][r], rtol=0, atol=grad_tol)
    assert np.allclose(g.gradient(x).to_vector(), ref["gx"].reshape(-1), rtol=0, atol=grad_tol)
    assert np.allclose(g.gradient(h).to_vector(), ref["gh"].reshape(-1), rtol=0, atol=grad_tol)
    assert np.allclose(g.gradient(c).to_vector(), ref["gc"], rtol=0, atol=grad_tol)


def test_lstm_with_stacked_gate_weights(dev):
    case = GRAPH_VECTORS["CheckConcatLSTM"]
    ref = _lstm_float64(case)
    loss_tol, grad_tol = _lstm_tolerances(dev)
    S, P = pa.Shape, case["parameters"]
    g = Tape(dev)
    x = g.input(S(case["inputs"]["x"]["shape"], 2), case["inputs"]["x"]["values"])
    h = g.input(S(case["inputs"]["h"]["shape"], 2), case["inputs"]["h"]["values"])
    c = g.constant(S([2]), 0)
    Wx, Wh, b = (g.input(S(P[k]["shape"]), P[k]["values"]) for k in ("pWx", "pWh", "pb"))
    u = g.add(g.add(g.matmul(Wx, x), g.matmul(Wh, h)), b)
    i = g.sigmoid(g.slice(u, 0, 0, 2))
    f = g.sigmoid(g.slice(u, 0, 2, 4))
    o = g.sigmoid(g.slice(u, 0, 4, 6))
    j = g.tanh(g.slice(u, 0, 6, 8))
    cc = g.add(g.multiply(f, c), g.multiply(i, j))
    hh = g.multiply(o, g.tanh(cc))
    t = g.constant(S([2]), 0)
    diff = g.subtract(hh, t)
    loss = g.multiply(diff, diff)
    sum_loss = g.batch_sum(g.sum(loss, 0))
    assert g.num_operators() == case["num_operators"] == 28

    want = np.asarray(case["expected_losses"], dtype=np.float32)
    assert np.allclose(g.value(loss).to_vector(), want, rtol=0, atol=loss_tol)
    assert abs(g.value(sum_loss).to_float() - float(want.sum())) <= 4 * loss_tol
    for node, key in ((i, "i"), (f, "f"), (o, "o"), (j, "j"), (cc, "cc"), (hh, "hh")):
        assert np.allclose(g.value(node).to_vector(), ref[key].reshape(-1), rtol=0, atol=max(loss_tol, grad_tol / 4)), key

    g.backward(sum_loss)
    assert np.allclose(g.gradient(Wx).to_vector(), _colmajor(ref["gWx"]), rtol=0, atol=grad_tol)
    assert np.allclose(g.gradient(Wh).to_vector(), _colmajor(ref["gWh"]), rtol=0, atol=grad_tol)
    assert np.allclose(g.gradient(b).to_vector(), ref["gb"], rtol=0, atol=grad_tol)
    assert np.allclose(g.gradient(x).to_vector(), ref["gx"].reshape(-1), rtol=0, atol=grad_tol)
    assert np.allclose(g.gradient(h).to_vector(), ref["gh"].reshape(-1), rtol=0, atol=grad_tol)
    assert np.allclose(g.gradient(c).to_vector(), ref["gc"], rtol=0, atol=grad_tol)
