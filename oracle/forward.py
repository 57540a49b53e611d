"""CPU-oracle forward passes of the benchmark configurations, composed from the
oracle's operators in the order the reference's CPU graph executes them.
TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import numpy as np

from . import binding as O


def _bcast_add_rows(h, b):
    return O.bcast_binop("add", h.reshape(-1), b.reshape(-1), h.shape[0], h.shape[1], 1).reshape(h.shape)


def mlp(inp):
    h = inp["x"]
    for i in range(3):
        h = _bcast_add_rows(O.gemm(h, inp[f"w{i}"]), inp[f"b{i}"])
        if i < 2:
            h = O.relu(h).reshape(h.shape)
    return O.softmax(h)


def elementwise(inp):
    n = inp["x"].shape[0]
    xy = O.binop("mul", "vv", inp["x"].reshape(-1), inp["y"].reshape(-1))
    s = O.bcast_binop("add", xy, inp["b"].reshape(-1), n, inp["x"].shape[1], 1)
    z = O.unary("sigmoid", s)
    return {"z": z.reshape(inp["x"].shape), "tanh": O.unary("tanh", z).reshape(inp["x"].shape),
            "pow": O.binop("pow", "vs", z, np.array([2.0], np.float32)).reshape(inp["x"].shape)}


def convnet(inp):
    h = inp["x"]
    for i in range(3):
        h = O.conv2d(h, inp[f"w{i}"], (1, 1), (1, 1), (1, 1))
        h = O.relu(h).reshape(h.shape)
        h = O.maxpool2d(h, (2, 2), (0, 0), (2, 2))
    h = h.reshape(h.shape[0], -1)
    h = O.relu(O.gemm(h, inp["w3"])).reshape(h.shape[0], -1)
    h = O.gemm(h, inp["w4"])
    return O.softmax(h)


def yolo(inp):
    h = inp["x"]
    for i in range(7):
        h = O.conv2d(h, inp[f"w{i}"], (1, 1), (1, 1), (1, 1))
        h = O.bn_infer(h, inp[f"mean{i}"], inp[f"var{i}"], 1e-5, inp[f"gamma{i}"], inp[f"beta{i}"])
        h = O.leaky_relu(h, 0.1).reshape(h.shape)
        if i < 5:
            h = O.maxpool2d(h, (2, 2), (0, 0), (2, 2))
        elif i == 5:
            h = O.maxpool2d(h, (2, 2), (1, 0, 1, 0), (1, 1))
    return O.conv2d(h, inp["w7"], (0, 0), (1, 1), (1, 1))
