"""Pins the oracle's backward passes (MaxPool2D, Conv2d, BatchNorm, SoftMax
gradients) before the GPU kernels are compared to them: the reference's own
gradient goldens where its tests hold any (BatchNorm input gradients), the
definition in float64 / brute force on small inputs, adjoint identities against
the already pinned forward oracle, and finite differences.  No GPU."""
import json
import os

import numpy as np
import pytest

from oracle import binding as O
from tests.test_oracle_pins import _init, _ranged

G = os.path.join(os.path.dirname(__file__), "golden")


def load(name):
    with open(os.path.join(G, name)) as f:
        return json.load(f)


# ---- MaxPool2D -----------------------------------------------------------------

POOL_CASES = [((2, 2), (0, 0), (2, 2), (5, 6)), ((2, 2), (0, 0), (1, 1), (3, 4)), ((3, 3), (1, 1), (2, 2), (7, 7)),
              ((2, 2), (1, 0, 1, 0), (1, 1), (6, 5)), ((3, 2), (1, 1), (1, 2), (6, 7))]


def _pool_bwd_bruteforce(x, dy, kernel, pad, stride):
    """Pure-Python restatement from the definition: argmax = first strictly larger element."""
    B, C, H, W = x.shape
    if len(pad) == 4:
        ph_, pw_ = pad[1], pad[3]  # explicit padding offsets by south / east (op_nn.go:871-875)
    else:
        ph_, pw_ = pad
    oh, ow = dy.shape[2:]
    dx = np.zeros_like(x)
    for b in range(B):
        for c in range(C):
            for ph in range(oh):
                for pw in range(ow):
                    best, arg = -np.finfo(np.float32).max, None
                    for hi in range(max(ph * stride[0] - ph_, 0), min(ph * stride[0] - ph_ + kernel[0], H)):
                        for wi in range(max(pw * stride[1] - pw_, 0), min(pw * stride[1] - pw_ + kernel[1], W)):
                            if x[b, c, hi, wi] > best:
                                best, arg = x[b, c, hi, wi], (hi, wi)
                    if arg is not None:
                        dx[b, c, arg[0], arg[1]] = np.float32(dx[b, c, arg[0], arg[1]] + dy[b, c, ph, pw])
    return dx


@pytest.mark.parametrize("kernel,pad,stride,hw", POOL_CASES)
def test_maxpool_bwd_bruteforce(kernel, pad, stride, hw):
    rng = np.random.default_rng(3)
    x = rng.integers(-3, 4, (2, 3) + hw).astype(np.float32)  # many ties: the first maximum must win
    y = O.maxpool2d(x, kernel, pad, stride)
    dy = rng.standard_normal(y.shape).astype(np.float32)
    got = O.maxpool2d_bwd(x, dy, kernel, pad, stride)
    assert np.array_equal(got, _pool_bwd_bruteforce(x, dy, kernel, pad, stride))
    # every dy lands somewhere: plane sums agree (float64 sums of float32 values)
    assert np.allclose(got.sum(axis=(2, 3), dtype=np.float64), dy.sum(axis=(2, 3), dtype=np.float64), atol=1e-5)


def test_maxpool_bwd_reference_example():
    """nn_test.go:140-193 TestMaxPool2D: x = 0..23 as (1,2,3,4), 2x2 window, stride 1, cost = Sum(y):
    each window's maximum is its bottom-right element, so the gradient counts windows per element."""
    x = np.arange(24, dtype=np.float32).reshape(1, 2, 3, 4)
    dy = np.ones((1, 2, 2, 3), np.float32)
    dx = O.maxpool2d_bwd(x, dy, (2, 2), (0, 0), (1, 1))
    want = np.zeros((3, 4), np.float32)
    want[1:, 1:] = 1.0
    assert np.array_equal(dx[0, 0], want) and np.array_equal(dx[0, 1], want)


def test_maxpool_bwd_on_golden_forward():
    """The 3072-float darknet-style pool of nn_test.go:91-138: gradient of Sum(y) puts, on every
    element, the number of windows it wins; the wins reproduce the golden forward output."""
    g = load("maxpool_asym.json")
    x = np.array(g["x"], dtype=np.float32).reshape(g["shape"])
    y = np.array(g["y"], dtype=np.float32).reshape(g["shape"])
    dx = O.maxpool2d_bwd(x, np.ones_like(y), g["kernel"], g["pad"], g["stride"])
    assert dx.sum() == y.size
    assert np.isclose((dx * x).sum(dtype=np.float64), y.sum(dtype=np.float64))


# ---- Conv2d ---------------------------------------------------------------------

CONV_BWD_CASES = [
    (2, 3, 8, 9, 5, 3, 3, (1, 1), (1, 1), (1, 1)),
    (1, 4, 7, 7, 6, 1, 1, (0, 0), (1, 1), (1, 1)),
    (2, 2, 10, 11, 3, 3, 2, (2, 1), (2, 3), (1, 1)),
    (1, 3, 12, 12, 4, 3, 3, (2, 2), (1, 1), (2, 2)),
    (2, 5, 9, 9, 7, 5, 5, (2, 2), (1, 1), (1, 1)),
    (3, 8, 6, 6, 16, 3, 3, (0, 0), (2, 2), (1, 1)),
]


@pytest.mark.parametrize("cfg", CONV_BWD_CASES)
def test_conv_bwd_definition_and_adjoint(cfg):
    B, C, H, W, F, kh, kw, pad, stride, dil = cfg
    rng = np.random.default_rng(5)
    x = rng.standard_normal((B, C, H, W)).astype(np.float32)
    w = rng.standard_normal((F, C, kh, kw)).astype(np.float32)
    y64 = O.conv2d_direct_f64(x, w, pad, stride, dil)
    dy = rng.standard_normal(y64.shape).astype(np.float32)
    dx, dw = O.conv2d_bwd(x, w, dy, pad, stride, dil)
    dx64, dw64 = O.conv2d_bwd_direct_f64(x, w, dy, pad, stride, dil)
    for got, ref in ((dx, dx64), (dw, dw64)):
        assert np.linalg.norm(got - ref) <= 1e-5 * np.linalg.norm(ref)
    # adjoint identities against the pinned forward pass: <conv(x, w), dy> = <x, dx> = <w, dw>
    lhs = float((y64 * dy).sum())
    assert np.isclose(lhs, float((x.astype(np.float64) * dx64).sum()), rtol=1e-9)
    assert np.isclose(lhs, float((w.astype(np.float64) * dw64).sum()), rtol=1e-9)
    # integer data: the float32 port is exact whatever its summation order
    xi = rng.integers(-3, 4, x.shape).astype(np.float32)
    wi = rng.integers(-3, 4, w.shape).astype(np.float32)
    di = rng.integers(-3, 4, dy.shape).astype(np.float32)
    dxi, dwi = O.conv2d_bwd(xi, wi, di, pad, stride, dil)
    rx, rw = O.conv2d_bwd_direct_f64(xi, wi, di, pad, stride, dil)
    assert np.array_equal(dxi, rx.astype(np.float32)) and np.array_equal(dwi, rw.astype(np.float32))


def test_conv_bwd_finite_difference():
    rng = np.random.default_rng(6)
    x = rng.standard_normal((1, 2, 5, 5)).astype(np.float32)
    w = rng.standard_normal((3, 2, 3, 3)).astype(np.float32)
    dy = rng.standard_normal((1, 3, 5, 5)).astype(np.float32)
    dx64, dw64 = O.conv2d_bwd_direct_f64(x, w, dy, (1, 1))
    f = lambda xx, ww: float((O.conv2d_direct_f64(xx, ww, (1, 1)) * dy).sum())
    for idx in [(0, 0, 0, 0), (0, 1, 2, 3), (0, 1, 4, 4)]:
        xp, xm = x.copy(), x.copy()
        xp[idx] += 0.25; xm[idx] -= 0.25   # the loss is linear in x: any step is exact up to rounding
        assert np.isclose((f(xp, w) - f(xm, w)) / 0.5, dx64[idx], rtol=1e-6)
    for idx in [(0, 0, 0, 0), (2, 1, 1, 2)]:
        wp, wm = w.copy(), w.copy()
        wp[idx] += 0.25; wm[idx] -= 0.25
        assert np.isclose((f(x, wp) - f(x, wm)) / 0.5, dw64[idx], rtol=1e-6)


# ---- BatchNorm ------------------------------------------------------------------

@pytest.mark.parametrize("idx", range(6))
def test_batchnorm_input_grad_goldens(idx):
    """nn_amd64_test.go bnAllCases ExpectedOutputGrad / ExpectedInputGrad through the graph of
    nn_test.go:319-417: out = (gamma*BN(x) + beta) . fcWeight^T, cost = Mean(out)."""
    c = load("batchnorm.json")["cases"][idx]
    shp = c["x_shape"]
    n = int(np.prod(shp))
    x = (_ranged(*c["x_ranged"], n) if "x_ranged" in c else np.array(c["x"], np.float32)).reshape(shp)
    B, Cn = shp[0], shp[1]
    feat = n // B
    S = feat // Cn
    gamma = _init(c["scale_init"], Cn)
    fcw = _init(c["scale_init"], B * feat).reshape(B, feat)
    y, rm, rv, sm, sv = O.bn_train_stats(x, np.zeros(Cn, np.float32), np.ones(Cn, np.float32), 0.9, 1e-5)
    y0, rm0, rv0 = O.bn_train(x, np.zeros(Cn, np.float32), np.ones(Cn, np.float32), 0.9, 1e-5)
    assert np.array_equal(y, y0) and np.array_equal(rm, rm0) and np.array_equal(rv, rv0)
    dout = np.full((B, B), 1.0 / (B * B), np.float32)
    assert np.allclose(dout.reshape(-1), c["expected_output_grad"])
    dz = (dout @ fcw).astype(np.float32)                           # out = z . fcw^T
    dbn = (dz.reshape(B, Cn, S) * gamma[None, :, None]).astype(np.float32).reshape(shp)
    dx = O.bn_bwd(x, dbn, sm, sv, 1e-5, training=True)
    want = np.array(c["expected_input_grad"], np.float32).reshape(shp)
    assert np.allclose(dx, want, rtol=2e-3, atol=2e-6), (dx.reshape(-1), want.reshape(-1))


def _bn_train_f64(x, eps):
    B, Cn = x.shape[:2]
    x3 = x.reshape(B, Cn, -1).astype(np.float64)
    mean = x3.mean(axis=(0, 2), keepdims=True)
    var = ((x3 - mean) ** 2).mean(axis=(0, 2), keepdims=True)
    return ((x3 - mean) / np.sqrt(var + eps)).reshape(x.shape)


@pytest.mark.parametrize("shape", [(4, 3, 5, 5), (6, 4)])
def test_batchnorm_bwd_is_the_gradient_of_the_training_forward(shape):
    rng = np.random.default_rng(8)
    x = rng.standard_normal(shape).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    Cn = shape[1]
    y, _, _, sm, sv = O.bn_train_stats(x, np.zeros(Cn, np.float32), np.ones(Cn, np.float32), 0.9, 1e-5)
    assert np.allclose(y, _bn_train_f64(x, 1e-5), atol=1e-5)
    x3 = x.reshape(shape[0], Cn, -1).astype(np.float64)
    assert np.allclose(sm, x3.mean(axis=(0, 2)), atol=1e-6)
    assert np.allclose(sv, ((x3 - x3.mean(axis=(0, 2), keepdims=True)) ** 2).sum(axis=(0, 2)), rtol=1e-5)
    dx = O.bn_bwd(x, dy, sm, sv, 1e-5, training=True)
    loss = lambda xx: float((_bn_train_f64(xx, 1e-5) * dy).sum())
    h = 1e-3
    for idx in [tuple(0 for _ in shape), tuple(s - 1 for s in shape), tuple(s // 2 for s in shape)]:
        xp, xm = x.astype(np.float64), x.astype(np.float64)
        xp[idx] += h; xm[idx] -= h
        fd = (loss(xp) - loss(xm)) / (2 * h)
        assert np.isclose(dx[idx], fd, rtol=2e-3, atol=2e-5), (idx, dx[idx], fd)
    # a gradient of a function that ignores the batch mean and scale: orthogonal to 1 and to x - mean
    d3 = dx.reshape(shape[0], Cn, -1).astype(np.float64)
    assert np.allclose(d3.sum(axis=(0, 2)), 0, atol=1e-4)
    # eval branch: dy / sqrt(var + eps)
    de = O.bn_bwd(x, dy, sm, sv, 1e-5, training=False)
    n = x.size // Cn
    inv = 1.0 / np.sqrt(sv.astype(np.float64) / n + 1e-5)
    assert np.allclose(de.reshape(shape[0], Cn, -1), dy.reshape(shape[0], Cn, -1) * inv[None, :, None], rtol=1e-6)


# ---- SoftMax ----------------------------------------------------------------------

def test_softmax_bwd_finite_difference_and_identities():
    rng = np.random.default_rng(9)
    x = rng.standard_normal((5, 10))
    dy = rng.standard_normal((5, 10)).astype(np.float32)
    y64 = O.softmax(x)                                  # float64 oracle, pinned by the goldens
    dx = O.softmax_bwd(y64.astype(np.float32), dy)
    jac = y64[:, :, None] * (np.eye(10)[None] - y64[:, None, :])       # dy_i/dx_j = y_i (delta_ij - y_j)
    want = np.einsum("ri,rij->rj", dy.astype(np.float64), jac)
    assert np.allclose(dx, want, rtol=1e-5, atol=1e-7)
    h = 1e-6
    for (r, j) in [(0, 0), (2, 7), (4, 9)]:
        xp, xm = x.copy(), x.copy()
        xp[r, j] += h; xm[r, j] -= h
        fd = ((O.softmax(xp) - O.softmax(xm)) * dy).sum() / (2 * h)
        assert np.isclose(dx[r, j], fd, rtol=1e-4, atol=1e-7)
    assert np.allclose(dx.sum(axis=1), 0, atol=1e-6)   # softmax ignores a shift of its input
    # old-vs-new softmax example of op_softmax_test.go:283-290: cost = Sum(softmax(a)) has zero gradient
    a = np.array([[0.1, 0.1, 0.3, 0.1, 0.4]])
    assert np.allclose(O.softmax_bwd(O.softmax(a).astype(np.float32), np.ones((1, 5), np.float32)), 0, atol=1e-7)


# ---- solvers ------------------------------------------------------------------------

def test_rmsprop_manual_closed_form():
    """solvers_test.go:100-143 manualRMSProp32 (TestRMSPropSolverManual): lr 0.01, l2reg 1e-6, clip 5,
    weights [1,2,3,4], gradients [0.5,-10,10,0.5] (zeroed by the first step), five iterations, 1e-4."""
    f = np.float32
    w = np.array([1, 2, 3, 4], f)
    g = np.array([0.5, -10, 10, 0.5], f)
    cache = np.zeros(4, f)
    correct_w, correct_c = w.copy(), np.zeros(4, f)
    decay, l2reg, eta, eps, clip = f(0.999), f(1e-6), f(0.01), f(1e-8), f(5.0)
    grad = g.copy()
    for it in range(5):
        for j in range(4):
            decayed = f(correct_c[j] * decay + f(f(f(1.0) - decay) * grad[j]) * grad[j])
            correct_c[j] = decayed
            gc = min(max(grad[j], -clip), clip)
            upd = f(f(f(-eta * gc) / np.sqrt(f(decayed + eps))) - f(l2reg * correct_w[j]))
            correct_w[j] = f(correct_w[j] + upd)
        w, _, cache, _ = O.solver_step("rmsprop", w, grad, cache, eta=0.01, l2reg=1e-6, clip=5.0, decay=0.999)
        grad = np.zeros(4, f)   # gt.Zero() at the end of Step (solvers.go:366)
        assert np.allclose(w, correct_w, rtol=1e-4, atol=0), it
        assert np.allclose(cache, correct_c, rtol=1e-4, atol=0), it


def test_adam_precision_golden():
    """solvers_test.go:355-437 TestAdamSolverPrecision float32: weights ones(4), the gradient of
    Mean(x . w) wrt w is x = d for d = 0, 0.1, ... (float32 accumulation) < 1; lr 0.1; ten steps."""
    f = np.float32
    w, m, v = np.ones(4, f), np.zeros(4, f), np.zeros(4, f)
    d, it = f(0.0), 0
    while d < f(1.0):
        it += 1
        w, _, m, v = O.solver_step("adam", w, np.full(4, d, f), m, v, eta=0.1, iteration=it)
        d = f(d + f(0.1))
    assert it == 10
    assert np.allclose(w, [0.18293014] * 4, rtol=1e-5, atol=1e-6), w


def test_vanilla_step_is_w_minus_eta_g_with_the_options_in_order():
    f = np.float32
    rng = np.random.default_rng(11)
    w = rng.standard_normal(1000).astype(f)
    g = rng.standard_normal(1000).astype(f)
    w1, _, _, _ = O.solver_step("vanilla", w, g, eta=0.05)
    assert np.array_equal(w1, (w + g * f(-0.05)).astype(f))
    w2, _, _, _ = O.solver_step("vanilla", w, g, eta=0.05, l1reg=0.01, l2reg=0.02, clip=0.5, batch=4.0)
    gg = g + f(0.01) * np.sign(w).astype(f)
    gg = gg + w * f(0.02)
    gg = gg * (f(1) / f(4))
    gg = np.clip(gg, f(-0.5), f(0.5))
    assert np.array_equal(w2, (w + gg * f(-0.05)).astype(f))


# ---- dropout -------------------------------------------------------------------------

@pytest.mark.parametrize("prob,expected,input_grad", [
    (0.2, [1.25, 1.25, 1.25, 0.0, 0.0], [1, 1, 1, 0, 0]),
    (0.5, [2.0, 2.0, 0.0, 0.0, 0.0], [0.4, 0.4, 0, 0, 0]),
])
def test_dropout_goldens(prob, expected, input_grad):
    """op_dropout_test.go:14-102 TestDropoutAll, Float32 rows: x = ones(5), the random source
    returns 0, 0.2, 0.5, 0.8, 1.0, cost = Mean(y) so the output gradient is 0.2 everywhere."""
    x = np.ones(5, np.float32)
    r = np.array([0.0, 0.2, 0.5, 0.8, 1.0], np.float32)
    y = O.dropout(x, r, prob)
    assert np.array_equal(y, np.array(expected, np.float32))
    dx = O.dropout_bwd(y, np.full(5, 0.2, np.float32), prob)
    assert np.array_equal(dx, np.array(input_grad, np.float32))
    assert np.array_equal(O.dropout(x, r, 0.0), x) and np.array_equal(O.dropout(x, r, prob, training=False), x)


def test_uniform_source_is_the_synthetic_stream():
    from gorgonia_amd import synth
    assert np.array_equal(O.uniform01(1000, 77), synth.uniform01(77, (1000,)))
    a = O.uniform01(1 << 16, 5)
    assert np.array_equal(O.uniform01(100, 5, offset=1000), a[1000:1100])
    assert 0.0 <= a.min() and a.max() < 1.0 and abs(a.mean() - 0.5) < 0.01


# ---- float64 twins of the backward operators ---------------------------------------------

def test_float64_backward_twins_against_the_float32_oracle():
    """Each float64 twin equals its pinned float32 counterpart where float32 arithmetic is
    exact (small integers, divisions by powers of two) and stays within float32 rounding of
    it on random data - a dropped term or a wrong index in a twin fails both."""
    rng = np.random.default_rng(5)
    # max-pool backward: integer gradients (every sum exact); ties and padding included
    x = rng.integers(-3, 4, (2, 3, 7, 9)).astype(np.float32)
    for kernel, pad, stride in [((2, 2), (0, 0), (2, 2)), ((3, 3), (1, 1), (2, 2)), ((2, 2), (1, 0, 1, 0), (1, 1))]:
        oh, ow = O.maxpool2d(x, kernel, pad, stride).shape[2:]
        dy = rng.integers(-5, 6, (2, 3, oh, ow)).astype(np.float32)
        d32 = O.maxpool2d_bwd(x, dy, kernel, pad, stride)
        d64 = O.maxpool2d_bwd(x.astype(np.float64), dy.astype(np.float64), kernel, pad, stride)
        assert d64.dtype == np.float64 and np.array_equal(d64, d32.astype(np.float64))
    # softmax backward: integer y and dy (exact), then random (within float32 rounding)
    y = rng.integers(-3, 4, (5, 7)).astype(np.float32)
    dy = rng.integers(-3, 4, (5, 7)).astype(np.float32)
    assert np.array_equal(O.softmax_bwd(y.astype(np.float64), dy.astype(np.float64)), O.softmax_bwd(y, dy).astype(np.float64))
    y = O.softmax(rng.standard_normal((6, 10)).astype(np.float32))
    dy = rng.standard_normal((6, 10)).astype(np.float32)
    np.testing.assert_allclose(O.softmax_bwd(y.astype(np.float64), dy.astype(np.float64)), O.softmax_bwd(y, dy), rtol=0, atol=1e-6)
    # dropout: keep = 0.5 divides exactly
    xd = rng.integers(-8, 9, 64).astype(np.float32)
    r = rng.random(64).astype(np.float32)
    y32 = O.dropout(xd, r, 0.5)
    y64 = O.dropout(xd.astype(np.float64), r.astype(np.float64), 0.5)
    assert np.array_equal(y64, y32.astype(np.float64))
    assert np.array_equal(O.dropout(xd.astype(np.float64), r.astype(np.float64), 0.5, training=False), xd)
    g = rng.integers(-8, 9, 64).astype(np.float32)
    assert np.array_equal(O.dropout_bwd(y64, g.astype(np.float64), 0.5), O.dropout_bwd(y32, g, 0.5).astype(np.float64))
    # solver steps: three steps of each kind within float32 rounding of the float32 oracle
    for kind, kw in [("vanilla", dict(eta=0.1, l2reg=0.01, clip=1.5, batch=4.0)), ("rmsprop", dict(eta=0.01, clip=2.0, l2reg=0.001)),
                     ("adam", dict(eta=0.001, iteration=2, l1reg=0.01))]:
        w32 = rng.standard_normal(500).astype(np.float32)
        w64 = w32.astype(np.float64)
        c32 = [None, None]
        c64 = [None, None]
        for step in range(3):
            g32 = (rng.standard_normal(500) * 3).astype(np.float32)
            w32, _, c32[0], c32[1] = O.solver_step(kind, w32, g32, c32[0], c32[1], **kw)
            w64, _, c64[0], c64[1] = O.solver_step(kind, w64, g32.astype(np.float64), c64[0], c64[1], **kw)
        assert w64.dtype == np.float64
        np.testing.assert_allclose(w64, w32, rtol=2e-5, atol=2e-6)
        if kind != "vanilla":
            np.testing.assert_allclose(c64[0], c32[0], rtol=2e-5, atol=1e-7)
    # vanilla without options is w - eta*g exactly
    w = rng.standard_normal(100)
    g = rng.standard_normal(100)
    got, _, _, _ = O.solver_step("vanilla", w, g, eta=0.25)
    assert np.array_equal(got, w + g * -0.25)


def test_float64_conv_gradients_against_the_float32_oracle():
    """The float64 conv gradients equal the pinned float32 ones on integer-valued operands
    (every order of summation exact) and agree within float32 rounding on random ones."""
    rng = np.random.default_rng(6)
    for (B, C, H, W, F, kh, kw, pad, stride, dil) in [(2, 3, 7, 6, 4, 3, 3, (1, 1), (1, 1), (1, 1)),
                                                      (1, 2, 9, 9, 3, 3, 2, (2, 0), (2, 1), (1, 2))]:
        x = rng.integers(-3, 4, (B, C, H, W)).astype(np.float32)
        w = rng.integers(-3, 4, (F, C, kh, kw)).astype(np.float32)
        oh, ow = O.conv2d(x, w, pad, stride, dil).shape[2:]
        dy = rng.integers(-3, 4, (B, F, oh, ow)).astype(np.float32)
        dx32, dw32 = O.conv2d_bwd(x, w, dy, pad, stride, dil)
        dx64, dw64 = O.conv2d_bwd(x.astype(np.float64), w.astype(np.float64), dy.astype(np.float64), pad, stride, dil)
        assert dx64.dtype == np.float64 and np.array_equal(dx64, dx32) and np.array_equal(dw64, dw32)
        xr, wr, dyr = (rng.standard_normal(a.shape).astype(np.float32) for a in (x, w, dy))
        dx32, dw32 = O.conv2d_bwd(xr, wr, dyr, pad, stride, dil)
        dx64, dw64 = O.conv2d_bwd(xr.astype(np.float64), wr.astype(np.float64), dyr.astype(np.float64), pad, stride, dil)
        assert np.linalg.norm(dx64 - dx32) <= 1e-5 * np.linalg.norm(dx64)
        assert np.linalg.norm(dw64 - dw32) <= 1e-5 * np.linalg.norm(dw64)


def test_float64_batchnorm_training_twins_against_the_float32_oracle():
    """The float64 BatchNorm training forward and gradient agree with the pinned float32 oracle
    within float32 rounding, and the gradient is the derivative of the training forward."""
    rng = np.random.default_rng(8)
    for shape in [(6, 3, 4, 5), (16, 7)]:
        x = rng.standard_normal(shape).astype(np.float32)
        dy = rng.standard_normal(shape).astype(np.float32)
        Cn = shape[1]
        rm, rv = rng.standard_normal(Cn).astype(np.float32), (rng.random(Cn) + 0.5).astype(np.float32)
        out32 = O.bn_train_stats(x, rm, rv, 0.9, 1e-5)
        out64 = O.bn_train_stats(x.astype(np.float64), rm.astype(np.float64), rv.astype(np.float64), 0.9, 1e-5)
        for a, b in zip(out64, out32):
            assert a.dtype == np.float64
            np.testing.assert_allclose(a, b, rtol=2e-5, atol=2e-5)
        for training in (True, False):
            d32 = O.bn_bwd(x, dy, out32[3], out32[4], 1e-5, training)
            d64 = O.bn_bwd(x.astype(np.float64), dy.astype(np.float64), out64[3], out64[4], 1e-5, training)
            np.testing.assert_allclose(d64, d32, rtol=1e-4, atol=2e-5)
        # finite differences of the float64 training forward: d/dx sum(y * dy)
        x64, dy64 = x.astype(np.float64), dy.astype(np.float64)
        grad = O.bn_bwd(x64, dy64, out64[3], out64[4], 1e-5, True)
        idx = tuple(int(v) // 2 for v in shape)
        h = 1e-6
        xp, xm = x64.copy(), x64.copy()
        xp[idx] += h
        xm[idx] -= h
        fp = (O.bn_train_stats(xp, rm, rv, 0.9, 1e-5)[0] * dy64).sum()
        fm = (O.bn_train_stats(xm, rm, rv, 0.9, 1e-5)[0] * dy64).sum()
        assert abs((fp - fm) / (2 * h) - grad[idx]) <= 1e-6 * max(1.0, abs(grad[idx]))


def test_uniform_source_float64_extends_the_float32_stream():
    """The 53-bit numbers are the same stream at a finer grain: their top 24 bits are the float32
    values (which are pinned to the synthetic-input generator)."""
    u64 = O.uniform01(5000, 42, 7, dtype=np.float64)
    u32 = O.uniform01(5000, 42, 7)
    assert u64.dtype == np.float64 and np.all((u64 >= 0) & (u64 < 1))
    assert np.array_equal(np.floor(u64 * 2**24) / 2**24, u32.astype(np.float64))
    assert len(np.unique(u64)) == 5000
