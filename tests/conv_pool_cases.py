"""The reference's convolution and pooling test cases (fixture
``golden/conv_pool_vectors.json``) replayed on any backend, and the closed-form
VGG16-sized cases of the same tests.

A backend offers conv2d_fw(x, w, x_dims, bx, w_dims, bw, *args),
conv2d_bw(x, w, gy, gx, gw, x_dims, bx, w_dims, bw, *args) -> (gx, gw),
max_pool2d_fw(x, x_dims, bs, *args), max_pool2d_bw(x, y, gy, gx, x_dims, bs, *args)
on flat float32 arrays.
"""
import json
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
VECTORS = json.load(open(os.path.join(_HERE, "golden", "conv_pool_vectors.json")))

CASES = [(kind, c) for kind in ("conv2d_fw", "conv2d_bw", "max_pool2d_fw", "max_pool2d_bw") for c in VECTORS[kind]]


def case_id(kc):
    return kc[0] + ":" + kc[1]["source"].split()[-1]


def iota(n):
    return np.arange(1, n + 1, dtype=np.float32)


def size(dims, batch):
    return int(np.prod(dims)) * batch if dims else batch


def run_case_on(backend, kind, c):
    """Returns [(expected, got), ...] for one fixture case."""
    a = c["args"]
    xs, bx = c["x_shape"], c["x_batch"]
    if kind == "conv2d_fw":
        y = backend.conv2d_fw(np.float32(c["x_data"]), np.float32(c["w_data"]), xs, bx, c["w_shape"], c["w_batch"], *a)
        return [(c["y_data"], y)]
    if kind == "conv2d_bw":
        # inputs as the reference's macro builds them (tensor_backward_test.cc:1920-1937)
        ws, bw = c["w_shape"], c["w_batch"]
        x, w = iota(size(xs, bx)), iota(size(ws, bw))
        gy = np.ones(size(c["y_shape"], c["y_batch"]), np.float32)
        gx, gw = backend.conv2d_bw(x, w, gy, np.ones_like(x), np.ones_like(w), xs, bx, ws, bw, *a)
        return [(c["gx_data"], gx), (c["gw_data"], gw)]
    if kind == "max_pool2d_fw":
        return [(c["y_data"], backend.max_pool2d_fw(np.float32(c["x_data"]), xs, bx, *a))]
    # max_pool2d_bw (tensor_backward_test.cc:2600-2612)
    x = iota(size(xs, bx))
    y = backend.max_pool2d_fw(x, xs, bx, *a)
    gy = np.ones(size(c["y_shape"], c["y_batch"]), np.float32)
    return [(c["gx_data"], backend.max_pool2d_bw(x, y, gy, np.ones_like(x), xs, bx, *a))]


# ---- VGG16-sized cases: expected values are closed forms ------------------------

def vgg_conv_case():
    """CheckConv2D_VGG16FirstLayer (tensor_forward_test.cc:3609-3630, tensor_backward_test.cc:2545-2598):
    all-ones 224x224x3 image and 3x3x3x64 kernel, padding 1.  Returns the inputs and expected y, gx, gw
    (gy all ones, gx and gw starting at 1)."""
    n = 224
    # taps inside the image per output position: 3 per axis, 2 on the border
    per_axis = np.full(n, 3.0, np.float32)
    per_axis[[0, -1]] = 2
    plane = np.outer(per_axis, per_axis) * 3          # three input channels
    y = np.tile(plane.reshape(-1), 64)
    gx_plane = 1 + np.outer(per_axis, per_axis) * 64  # every output channel
    gx = np.tile(gx_plane.reshape(-1), 3)
    # gw element (i, j): outputs whose tap (i, j) lies inside the image
    taps = np.array([n - 1, n, n - 1], np.float32)
    gw = np.tile(1 + np.outer(taps, taps).reshape(-1), 3 * 64)
    return dict(x=np.ones(n * n * 3, np.float32), w=np.ones(27 * 64, np.float32), x_dims=[n, n, 3],
                w_dims=[3, 3, 3, 64], args=(1, 1, 1, 1, 1, 1), y=y.astype(np.float32), gx=gx.astype(np.float32),
                gw=gw.astype(np.float32))


def vgg_pool_case():
    """CheckMaxPool2D_VGG16ThirdLayer (tensor_forward_test.cc:3999-4025, tensor_backward_test.cc:2912-2950):
    x[b][col][row] = col + row on 224x224x64, 2x2 windows with stride 2."""
    n, c = 224, 64
    i = np.arange(n, dtype=np.float32)
    x = np.tile((i[:, None] + i[None, :]).reshape(-1), c)
    j = np.arange(n // 2, dtype=np.float32)
    y = np.tile(((2 * j[:, None] + 1) + (2 * j[None, :] + 1)).reshape(-1), c)
    gx_plane = np.ones((n, n), np.float32)
    gx_plane[1::2, 1::2] += 1
    return dict(x=x, x_dims=[n, n, c], args=(2, 2, 0, 0, 2, 2), y=y, gx=np.tile(gx_plane.reshape(-1), c))
