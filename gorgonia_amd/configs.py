"""The five benchmark configurations as seeded inputs plus graph builders.

Each builder returns (graph, outputs dict of Read() arrays, inputs dict) for a
TapeMachine.  Inputs come from gorgonia_amd.synth (seeded); weights are bound
as resident values unless resident=False (the reference re-uploads every input,
weights included, on every run: vm_tape_cuda.go:227-230).
"""
from __future__ import annotations

import numpy as np

from . import graph as G
from . import synth


# ---- inputs --------------------------------------------------------------------------

def mlp_inputs(batch=256):
    """Config 1: 3-layer MLP 784 -> 300 -> 100 -> 10."""
    return {
        "x": synth.uniform01(101, (batch, 784)),
        "w0": synth.glorot_uniform(102, (784, 300)),
        "w1": synth.glorot_uniform(103, (300, 100)),
        "w2": synth.glorot_uniform(104, (100, 10)),
        "b0": np.zeros((1, 300), np.float32), "b1": np.zeros((1, 100), np.float32),
        "b2": np.zeros((1, 10), np.float32),
    }


def elementwise_inputs(n=4096):
    """Config 2: x, y ~ U[-4, 4) (n x n), b ~ U[-4, 4) (1 x n)."""
    return {"x": synth.uniform(201, (n, n), -4, 4), "y": synth.uniform(202, (n, n), -4, 4),
            "b": synth.uniform(203, (1, n), -4, 4), "two": np.array(2.0, np.float32)}


def convnet_inputs(batch=128):
    """Config 4: examples/convnet/main.go:57-159 shapes."""
    return {
        "x": synth.uniform01(401, (batch, 1, 28, 28)),
        "w0": synth.he_normal(402, (32, 1, 3, 3)),
        "w1": synth.he_normal(403, (64, 32, 3, 3)),
        "w2": synth.he_normal(404, (128, 64, 3, 3)),
        "w3": synth.he_normal(405, (128 * 3 * 3, 625)),
        "w4": synth.he_normal(406, (625, 10)),
    }


YOLO_CHANNELS = [3, 16, 32, 64, 128, 256, 512, 1024]


def yolo_inputs(batch=8, size=416):
    """Config 5: Tiny-YOLO-v2-shaped stack (examples/tiny-yolo-v2-coco/feedforward.go:10-186)."""
    d = {"x": synth.uniform01(501, (batch, 3, size, size))}
    for i in range(7):
        cin, cout = YOLO_CHANNELS[i], YOLO_CHANNELS[i + 1]
        d[f"w{i}"] = synth.he_normal(510 + i, (cout, cin, 3, 3))
        d[f"mean{i}"] = synth.normal(520 + i, (cout,), 0.0, 0.1)
        d[f"var{i}"] = synth.uniform(530 + i, (cout,), 0.5, 1.5)
        d[f"gamma{i}"] = synth.uniform(540 + i, (cout,), 0.5, 1.5)
        d[f"beta{i}"] = synth.normal(550 + i, (cout,), 0.0, 0.1)
    d["w7"] = synth.he_normal(517, (425, 1024, 1, 1))
    return d


# ---- graphs -----------------------------------------------------------------------------

def build_mlp(inp, resident=True, resident_input=False):
    g = G.NewGraph()
    x = G.NewTensor(g, inp["x"], resident=resident_input)
    h = x
    for i in range(3):
        w = G.NewTensor(g, inp[f"w{i}"], resident)
        b = G.NewTensor(g, inp[f"b{i}"], resident)
        h = G.BroadcastAdd(G.Mul(h, w), b)
        if i < 2:
            h = G.Rectify(h)
    out = G.SoftMax(h)
    return g, {"out": G.Read(out)}


def build_elementwise(inp):
    """z = Sigmoid(Add(HadamardProd(x, y), b)); Tanh(z); Pow(z, 2)."""
    g = G.NewGraph()
    x, y, b = (G.NewTensor(g, inp[k]) for k in ("x", "y", "b"))
    two = G.NewScalar(g, inp["two"])
    z = G.Sigmoid(G.BroadcastAdd(G.HadamardProd(x, y), b))
    t = G.Tanh(z)
    p = G.Pow(z, two)
    return g, {"z": G.Read(z), "tanh": G.Read(t), "pow": G.Read(p)}


def build_convnet(inp, resident=True, resident_input=False):
    g = G.NewGraph()
    h = G.NewTensor(g, inp["x"], resident_input)
    for i in range(3):
        w = G.NewTensor(g, inp[f"w{i}"], resident)
        h = G.Conv2d(h, w, (3, 3), (1, 1), (1, 1), (1, 1))
        h = G.Rectify(h)
        h = G.MaxPool2D(h, (2, 2), (0, 0), (2, 2))
    b = inp["x"].shape[0]
    h = G.Reshape(h, (b, 128 * 3 * 3))
    h = G.Rectify(G.Mul(h, G.NewTensor(g, inp["w3"], resident)))
    h = G.Mul(h, G.NewTensor(g, inp["w4"], resident))
    out = G.SoftMax(h)
    return g, {"out": G.Read(out)}


def build_convnet_train(inp, onehot, lr, read_grads=True, solver="set"):
    """Config 4 as one training step (examples/convnet/main.go:57-180 with vanilla
    SGD): forward, the diff ops the reference's symbolic differentiation would
    insert, and w <- w - lr * dw through Set, so the resident weights carry over
    to the next RunAll.  cost = -Mean(out * onehot)."""
    g = G.NewGraph()
    b = inp["x"].shape[0]
    x = G.NewTensor(g, inp["x"], True)
    y = G.NewTensor(g, onehot, True)
    w = [G.NewTensor(g, inp[f"w{i}"], True) for i in range(5)]
    dt = np.asarray(inp["x"]).dtype   # the scalars in the tensors' own type, as the reference's type inference demands
    lr_s = G.NewScalar(g, lr, dtype=dt)
    scale = G.NewScalar(g, -1.0 / onehot.size, dtype=dt)
    conv = dict(kernelShape=(3, 3), pad=(1, 1), stride=(1, 1), dilation=(1, 1))
    acts, h = [], x
    for i in range(3):
        z = G.Conv2d(h, w[i], (3, 3), (1, 1), (1, 1), (1, 1))
        a = G.Rectify(z)
        acts.append((h, z, a))
        h = G.MaxPool2D(a, (2, 2), (0, 0), (2, 2))
    r = G.Reshape(h, (b, 128 * 3 * 3))
    z3 = G.Mul(r, w[3])
    a3 = G.Rectify(z3)
    out = G.SoftMax(G.Mul(a3, w[4]))
    outs = {"out": G.Read(out)}
    # backward
    g4 = G.SoftMaxDiff(out, G.HadamardProd(y, scale))
    dw = {4: G.Mul(a3, g4, transA=True)}
    dz3 = G.RectifyDiff(z3, G.Mul(g4, w[4], transB=True))
    dw[3] = G.Mul(r, dz3, transA=True)
    grad = G.Reshape(G.Mul(dz3, w[3], transB=True), h.Shape())
    for i in (2, 1, 0):
        x_in, z, a = acts[i]
        dz = G.RectifyDiff(z, G.MaxPool2DDiff(a, grad, (2, 2), (0, 0), (2, 2)))
        dw[i] = G.Conv2dDiffFilter(x_in, dz, **conv)
        if i:
            grad = G.Conv2dDiffImage(dz, w[i], x_in.Shape(), **conv)
    if read_grads:
        for i in range(5):
            outs[f"dw{i}"] = G.Read(dw[i])
    # updates last: every gradient above was taken at the old weights
    for i in range(5):
        if solver == "set":      # w <- w - lr*dw spelled with graph ops
            G.Set(w[i], G.Sub(w[i], G.HadamardProd(dw[i], lr_s)))
        elif solver == "vanilla":
            G.SolverStep("vanilla", w[i], dw[i], eta=lr)
        else:                     # RMSProp as in examples/convnet/main.go:195
            cache = G.NewTensor(g, np.zeros_like(inp[f"w{i}"]), True)
            G.SolverStep("rmsprop", w[i], dw[i], [cache], eta=lr, l2reg=1e-6, clip=5.0)
    return g, outs


def build_yolo(inp, resident=True, resident_input=False, borrow_output=False, borrow_input=False):
    g = G.NewGraph()
    h = G.NewTensor(g, inp["x"], resident_input)
    if borrow_input:   # the batch is written into TapeMachine.input(g.x_node), the machine's pinned buffer
        G.LetBorrowed(h)
    g.x_node = h
    for i in range(7):
        w = G.NewTensor(g, inp[f"w{i}"], resident)
        h = G.Conv2d(h, w, (3, 3), (1, 1), (1, 1), (1, 1))
        m, v, ga, be = (G.NewTensor(g, inp[f"{k}{i}"], resident) for k in ("mean", "var", "gamma", "beta"))
        h = G.BatchNorm(h, ga, be, m, v, 1e-5)
        h = G.LeakyRelu(h, 0.1)
        if i < 5:
            h = G.MaxPool2D(h, (2, 2), (0, 0), (2, 2))
        elif i == 5:
            h = G.MaxPool2D(h, (2, 2), (1, 0, 1, 0), (1, 1))  # darknet stride-1 pool
    out = G.Conv2d(h, G.NewTensor(g, inp["w7"], resident), (1, 1), (0, 0), (1, 1), (1, 1))
    # borrow_output: the 2.3 MB result stays in the machine's pinned buffer (TapeMachine.value)
    return g, {"out": G.ReadBorrowed(out) if borrow_output else G.Read(out)}


FLOPS = {  # algorithmic flop per forward pass at the configured batch sizes
    "mlp": 136_294_400, "convnet": 2_093_410_816, "yolo": 31_080_857_600,
}
