"""Seeded random graphs on both machines: the reference's main test pattern (one graph on the
TapeMachine and on the LispMachine, equal values required - nn_test.go:25-79,
operatorPointwise_unary_test.go:14-95) over graphs nobody wrote by hand.

The lisp machine runs a graph node by node, a fresh value for every node and nothing folded; the
tape machine batches, overwrites dead operands, folds followers into their producer's command
(BatchNorm, activation, pooling, bias, SoftMax, a first layer into the second, a kept
pre-activation value) and replays.  Every value a graph reads must come out with the same bits
either way, on every run: what a random graph adds to the hand-written ones is intermediate values
with a second reader or a Read, created before or after the node that would otherwise swallow them,
and (every fifth graph) the gradient operators behind a stack of conv -> Rectify -> pool layers."""
import numpy as np
import pytest

from gorgonia_amd import graph as G, synth
from tests.util import assert_bits_equal

pytestmark = pytest.mark.gpu


class Builder:
    def __init__(self, seed, dtype):
        self.rng = np.random.default_rng(seed)
        self.seed = seed * 1000
        self.dtype = np.dtype(dtype)
        self.g = G.NewGraph()
        self.reads = {}
        self.pending = []   # second readers to be created later, after more of the graph exists

    def pick(self, seq):
        return seq[int(self.rng.integers(len(seq)))]

    def chance(self, p):
        return bool(self.rng.random() < p)

    def tensor(self, shape, lo=-1.0, hi=1.0, resident=None):
        self.seed += 1
        v = synth.uniform(self.seed, shape, lo, hi).astype(self.dtype)
        return G.NewTensor(self.g, v, self.chance(0.6) if resident is None else resident)

    def read(self, node, what):
        self.reads[f"{len(self.reads)}:{what}"] = G.Read(node)

    def second_reader(self, node):
        """Another operator on `node`'s value, read by the caller; never overwrites what others still need."""
        kind = self.pick(["neg", "sigmoid", "add", "rectify", "pool"])
        if kind == "neg":
            return G.Neg(node)
        if kind == "sigmoid":
            return G.Sigmoid(node)
        if kind == "add":
            return G.Add(node, node)
        if kind == "rectify":
            return G.Rectify(node)
        shp = node.Shape()
        if len(shp) == 4 and shp[2] >= 3 and shp[3] >= 3:
            return G.MaxPool2D(node, (2, 2), (0, 0), (1, 1))
        return G.Square(node)

    def tap(self, node, what, p_read=0.2, p_second=0.2):
        """Maybe read an intermediate value, maybe give it a second reader - now, or after the
        nodes that follow it have been created."""
        if self.chance(p_read):
            self.read(node, what)
        if self.chance(p_second):
            if self.chance(0.5):
                self.read(self.second_reader(node), what + "/second")
            else:
                self.pending.append((node, what))

    def flush_pending(self):
        for node, what in self.pending:
            self.read(self.second_reader(node), what + "/second-late")
        self.pending = []


def conv_stack(b, first_layer_like=False):
    rng = b.rng
    B = int(rng.integers(1, 4))
    if first_layer_like:   # a grey-scale first layer in front of a 32-channel convolution
        C, H, W = 1, 2 * int(rng.integers(4, 15)), 2 * int(rng.integers(4, 15))
    else:
        C = b.pick([1, 3, 4, 8, 16, 32])
        H, W = int(rng.integers(5, 23)), int(rng.integers(5, 23))
    h = b.tensor((B, C, H, W), 0.0, 1.0, resident=False)
    for layer in range(int(rng.integers(1, 4))):
        _, C, H, W = h.Shape()
        if first_layer_like and layer < 2:
            k, pad, F = 3, 1, (32 if layer == 0 else b.pick([16, 32, 64]))
        else:
            k = b.pick([1, 3, 3, 3])
            pad = b.pick([0, 1]) if k == 3 else 0
            F = b.pick([4, 8, 16, 17, 32, 33, 64])
        if H + 2 * pad - k + 1 < 1 or W + 2 * pad - k + 1 < 1:
            break
        w = b.tensor((F, C, k, k), -0.5, 0.5)
        h = G.Conv2d(h, w, (k, k), (pad, pad), (1, 1), (1, 1))
        b.tap(h, f"conv{layer}")
        if b.chance(0.0 if first_layer_like and layer == 0 else 0.5):
            mean, var = b.tensor((F,), -0.2, 0.2), b.tensor((F,), 0.5, 1.5)
            if b.chance(0.7):
                h = G.BatchNorm(h, b.tensor((F,), 0.5, 1.5), b.tensor((F,), -0.2, 0.2), mean, var, 1e-5)
            else:
                h = G.BatchNorm(h, None, None, mean, var, 1e-5)
            b.tap(h, f"bn{layer}")
        act = "relu" if first_layer_like and layer == 0 else b.pick([None, "relu", "relu", "leaky"])
        if act == "relu":
            h = G.Rectify(h)
        elif act == "leaky":
            h = G.LeakyRelu(h, 0.1)
        if act:
            b.tap(h, f"act{layer}", 0.15, 0.15)
        _, _, H, W = h.Shape()
        pool = "2x2" if first_layer_like and layer == 0 else b.pick([None, "2x2", "2x2", "2x2s1", "3x3"])
        if pool == "2x2" and H >= 2 and W >= 2:
            h = G.MaxPool2D(h, (2, 2), (0, 0), (2, 2))
        elif pool == "2x2s1" and H >= 2 and W >= 2:
            h = G.MaxPool2D(h, (2, 2), (1, 0, 1, 0), (1, 1))
        elif pool == "3x3" and H >= 3 and W >= 3:
            h = G.MaxPool2D(h, (3, 3), (1, 1), (2, 2))
        else:
            pool = None
        if pool:
            b.tap(h, f"pool{layer}", 0.15, 0.15)
        if b.chance(0.3):
            b.flush_pending()
    return h


def dense_tail(b, h):
    shp = h.Shape()
    rows = shp[0]
    cols = int(np.prod(shp[1:]))
    if len(shp) != 2:
        h = G.Reshape(h, (rows, cols))
    for layer in range(int(b.rng.integers(1, 3))):
        n = b.pick([3, 10, 16, 37, 64])
        w = b.tensor((cols, n), -0.3, 0.3)
        h = G.Mul(h, w)
        b.tap(h, f"mul{layer}", 0.15, 0.15)
        if b.chance(0.6):
            h = G.BroadcastAdd(h, b.tensor((1, n), -0.5, 0.5))
            b.tap(h, f"bias{layer}", 0.15, 0.15)
        if b.chance(0.5):
            h = G.Rectify(h)
            b.tap(h, f"relu{layer}", 0.15, 0.15)
        cols = n
    kind = b.pick(["softmax", "softmax", "softmax", "matvec", "vecmat", None])
    if kind == "softmax":
        h = G.SoftMax(h)
    elif kind == "matvec":      # matrix x vector, then the inner product with a vector (operations.go:52-74)
        h = G.Mul(h, b.tensor((cols,), -0.5, 0.5))
        b.tap(h, "matvec", 0.3, 0.0)
        h = G.Mul(h, b.tensor((rows,), -0.5, 0.5))
    elif kind == "vecmat":      # vector x matrix: the product with the transposed matrix
        h = G.Mul(b.tensor((rows,), -0.5, 0.5), h)
    return h


def elementwise_web(b):
    """Values with several readers and operators that may overwrite a dead operand."""
    n = (int(b.rng.integers(1, 40)), int(b.rng.integers(1, 300)))
    vals = [b.tensor(n, -2.0, 2.0, resident=False) for _ in range(3)]
    row = b.tensor((1, n[1]), -1.0, 1.0)
    unary = [G.Neg, G.Square, G.Sigmoid, G.Tanh, G.Abs, G.Rectify, G.Cube, G.Exp]
    binary = [G.Add, G.Sub, G.HadamardProd, G.Lt, G.Gte]
    for step in range(int(b.rng.integers(4, 12))):
        a = b.pick(vals)
        kind = b.pick(["unary", "binary", "binary", "bcast", "leaky"])
        if kind == "unary":
            v = b.pick(unary)(a)
        elif kind == "binary":
            v = b.pick(binary)(a, b.pick(vals))
        elif kind == "bcast":
            v = b.pick([G.BroadcastAdd, G.BroadcastHadamardProd])(a, row)
        else:
            v = G.LeakyRelu(a, 0.25)
        b.tap(v, f"ew{step}", 0.3, 0.0)
        vals.append(v)
    return vals[-1]


def training_stack(b):
    """Forward layers conv -> Rectify [-> pool] and the diff operators symbolic differentiation would insert
    behind them, from a drawn gradient of the last value: the values between the layers have readers in both
    directions, which is where the pool takes over a kept convolution and reads through a Rectify."""
    rng = b.rng
    B = int(rng.integers(1, 5))
    C = b.pick([1, 3, 8, 16, 32])
    H, W = int(rng.integers(6, 20)), int(rng.integers(6, 20))
    h = b.tensor((B, C, H, W), 0.0, 1.0, resident=False)
    layers = []
    for layer in range(int(rng.integers(1, 4))):
        _, C, H, W = h.Shape()
        pad = b.pick([0, 1])
        if H + 2 * pad - 2 < 2 or W + 2 * pad - 2 < 2:
            break
        F = b.pick([8, 16, 32, 64])
        w = b.tensor((F, C, 3, 3), -0.5, 0.5, resident=True)
        z = G.Conv2d(h, w, (3, 3), (pad, pad), (1, 1), (1, 1))
        a = G.Rectify(z)
        pooled = None
        kind = b.pick(["2x2", "2x2", "3x3", None])
        if kind == "2x2":
            pooled = G.MaxPool2D(a, (2, 2), (0, 0), (2, 2))
        elif kind == "3x3" and a.Shape()[2] >= 3 and a.Shape()[3] >= 3:
            pooled = G.MaxPool2D(a, (3, 3), (1, 1), (2, 2))
        else:
            kind = None
        layers.append((h, w, z, a, pooled, kind, pad))
        h = pooled if pooled is not None else a
        if b.chance(0.2):
            b.read(h, f"fwd{layer}")
    b.read(h, "fwd")
    grad = b.tensor(h.Shape(), -1.0, 1.0, resident=False)
    for layer in reversed(range(len(layers))):
        x_in, w, z, a, pooled, kind, pad = layers[layer]
        if kind == "2x2":
            grad = G.MaxPool2DDiff(a, grad, (2, 2), (0, 0), (2, 2))
        elif kind == "3x3":
            grad = G.MaxPool2DDiff(a, grad, (3, 3), (1, 1), (2, 2))
        dz = G.RectifyDiff(z, grad)
        b.read(G.Conv2dDiffFilter(x_in, dz, (3, 3), (pad, pad), (1, 1), (1, 1)), f"dw{layer}")
        if layer or b.chance(0.5):
            grad = G.Conv2dDiffImage(dz, w, x_in.Shape(), (3, 3), (pad, pad), (1, 1), (1, 1))
            if layer == 0:
                b.read(grad, "dx")
    return None


def build(seed, dtype):
    b = Builder(seed, dtype)
    shape = seed % 5
    if shape == 4:
        training_stack(b)
        return b.g, b.reads
    if shape == 3:
        out = elementwise_web(b)
    else:
        h = conv_stack(b, first_layer_like=(shape == 2))
        out = dense_tail(b, h) if b.chance(0.7) else h
    b.flush_pending()
    b.read(out, "out")
    return b.g, b.reads


def run_both(seed, dtype):
    g, reads = build(seed, dtype)
    lisp = G.NewLispMachine(g)
    lisp.RunAll()
    want = {k: v.copy() for k, v in reads.items()}
    lisp.Close()
    folded = 0
    for kw in (dict(), dict(fuse_activations=True), dict(fuse_activations=True, graph_replay=True)):
        g2, reads2 = build(seed, dtype)
        assert list(reads2) == list(want)
        m = G.NewTapeMachine(g2, **kw)
        folded = max(folded, m.fused)
        for run in range(3):
            for v in reads2.values():
                v[...] = -7.0
            m.RunAll()
            for k in reads2:
                assert_bits_equal(reads2[k], want[k], f"seed {seed} {np.dtype(dtype).name} {kw} run {run}: {k}\n{m.program()}")
        m.Close()
    return folded


@pytest.mark.parametrize("block", range(8))
def test_random_graphs_float32(ctx, block):
    folded = 0
    for seed in range(block * 12, block * 12 + 12):
        folded += run_both(seed, np.float32)
    assert folded > 0, "twelve random graphs and nothing to fold: the generator has lost its point"


@pytest.mark.parametrize("block", range(2))
def test_random_graphs_float64(ctx, block):
    for seed in range(1000 + block * 12, 1000 + block * 12 + 12):
        run_both(seed, np.float64)
