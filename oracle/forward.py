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


def convnet_train_step(inp, onehot, lr):
    """One forward + backward + vanilla-SGD step of the convnet configuration with
    cost = -Mean(out * onehot) (examples/convnet/main.go:173-180), every gradient
    written out as the reference's diff ops compute it.  Returns (out, cost,
    grads, new_weights)."""
    B = inp["x"].shape[0]
    acts, h = [], inp["x"]
    for i in range(3):
        z = O.conv2d(h, inp[f"w{i}"], (1, 1), (1, 1), (1, 1))
        a = O.relu(z).reshape(z.shape)
        p = O.maxpool2d(a, (2, 2), (0, 0), (2, 2))
        acts.append((h, z, a))
        h = p
    r = h.reshape(B, -1)
    z3 = O.gemm(r, inp["w3"])
    a3 = O.relu(z3).reshape(z3.shape)
    z4 = O.gemm(a3, inp["w4"])
    out = O.softmax(z4)
    scale = np.float32(-1.0 / out.size)
    cost = float(np.float32(-(out * onehot).mean(dtype=np.float64)))
    gout = O.binop("mul", "vs", onehot.reshape(-1).copy(), np.array([scale], np.float32)).reshape(out.shape)
    g4 = O.softmax_bwd(out, gout)
    grads = {"w4": O.gemm(a3, g4, True, False)}
    da3 = O.gemm(g4, inp["w4"], False, True)
    mask = lambda z: O.binop("gte", "vs", z.reshape(-1).copy(), np.zeros(1, np.float32)).reshape(z.shape)
    dz3 = (da3 * mask(z3)).astype(np.float32)
    grads["w3"] = O.gemm(r, dz3, True, False)
    g = O.gemm(dz3, inp["w3"], False, True).reshape(h.shape)
    for i in (2, 1, 0):
        x_in, z, a = acts[i]
        da = O.maxpool2d_bwd(a, g, (2, 2), (0, 0), (2, 2))
        dz = (da * mask(z)).astype(np.float32)
        dx, dw = O.conv2d_bwd(x_in, inp[f"w{i}"], dz, (1, 1), (1, 1), (1, 1))
        grads[f"w{i}"] = dw
        g = dx
    new = {k: (inp[k] - grads[k] * np.float32(lr)).astype(np.float32) for k in grads}
    return out, cost, grads, new


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
