"""GPU parity of the float64 backward operators, dropout and solver steps (max-pool, softmax
and activation gradients, dropout forward/backward, Vanilla / RMSProp / Adam steps) through
the C ABI against the CPU oracle's float64 twins.  Bar: bit-exact (same operation order, one
IEEE rounding per step; division and square root are correctly rounded on both sides)."""
import ctypes as C

import numpy as np
import pytest

from gorgonia_amd import _ffi
from gorgonia_amd import device as D
from oracle import binding as O
from tests.util import assert_bits_equal

pytestmark = pytest.mark.gpu
F64 = _ffi.F64


def _rand(seed, shape, scale=1.0):
    return np.random.default_rng(seed).standard_normal(shape) * scale


def _up(ctx, a):
    return ctx.upload(np.ascontiguousarray(a, dtype=np.float64))


@pytest.mark.parametrize("kernel,pad,stride,shape", [
    ((2, 2), (0, 0), (2, 2), (3, 4, 14, 14)),
    ((2, 2), (0, 0), (2, 2), (2, 3, 7, 7)),
    ((3, 3), (1, 1), (2, 2), (2, 2, 9, 11)),
    ((2, 2), (1, 0, 1, 0), (1, 1), (1, 3, 13, 13)),
    ((3, 2), (1, 1), (1, 1), (2, 2, 6, 5)),
])
def test_maxpool_backward_float64(ctx, kernel, pad, stride, shape):
    x = _rand(1, shape)
    x[0, 0, :2, :2] = 0.5   # a tie: the first element of the window wins
    oh, ow = O.maxpool2d(x, kernel, pad, stride).shape[2:]
    dy = _rand(2, shape[:2] + (oh, ow))
    want = O.maxpool2d_bwd(x, dy, kernel, pad, stride)
    px, pdy, pdx = _up(ctx, x), _up(ctx, dy), ctx.malloc(x.size * 8)
    ctx.run(D.cmd_maxpool2d_bwd(px, pdy, pdx, *shape, kernel[0], kernel[1], pad, stride, dtype=F64))
    assert_bits_equal(ctx.d2h(pdx, shape, np.float64), want, "max-pool backward float64")
    for p in (px, pdy, pdx):
        ctx.free(p)


@pytest.mark.parametrize("rows,cols", [(1, 1), (128, 10), (37, 129), (1000, 3)])
def test_softmax_backward_float64(ctx, rows, cols):
    y = O.softmax(_rand(3, (rows, cols)))
    dy = _rand(4, (rows, cols))
    want = O.softmax_bwd(y, dy)
    py, pdy, pdx = _up(ctx, y), _up(ctx, dy), ctx.malloc(rows * cols * 8)
    ctx.run(D.cmd_softmax_bwd(py, pdy, pdx, rows, cols, dtype=F64))
    assert_bits_equal(ctx.d2h(pdx, (rows, cols), np.float64), want, "softmax backward float64")
    for p in (py, pdy, pdx):
        ctx.free(p)


@pytest.mark.parametrize("n", [1, 5, 1000, 70001])
def test_relu_backward_and_dropout_float64(ctx, n):
    x = _rand(5, (n,))
    dy = _rand(6, (n,))
    special = np.array([0.0, -0.0, np.nan, np.inf, -np.inf], np.float64)
    k = min(n, special.size)
    x[:k] = special[:k]
    mask = O.binop("gte", "vs", x, np.zeros(1))
    want = O.binop("mul", "vv", dy, mask)
    px, pdy, pdx = _up(ctx, x), _up(ctx, dy), ctx.malloc(n * 8)
    ctx.run(D.cmd_relu_bwd(px, pdy, pdx, n, dtype=F64))
    assert_bits_equal(ctx.d2h(pdx, (n,), np.float64), want, "relu backward float64")
    # dropout forward (training and not) and backward
    r = np.random.default_rng(7).random(n)
    pr, py = _up(ctx, r), ctx.malloc(n * 8)
    for prob in (0.3, 0.0):
        ctx.run(D.cmd_dropout(px, py, pr, n, prob, dtype=F64))
        y = ctx.d2h(py, (n,), np.float64)
        assert_bits_equal(y, O.dropout(x, r, prob), f"dropout float64 p={prob}")
        ctx.run(D.cmd_dropout_bwd(py, pdy, pdx, n, prob, dtype=F64))
        assert_bits_equal(ctx.d2h(pdx, (n,), np.float64), O.dropout_bwd(y, dy, prob), f"dropout backward float64 p={prob}")
    ctx.run(D.cmd_dropout(px, py, pr, n, 0.3, training=False, dtype=F64))
    assert_bits_equal(ctx.d2h(py, (n,), np.float64), x, "dropout float64 outside training")
    for p in (px, pdy, pdx, pr, py):
        ctx.free(p)


@pytest.mark.parametrize("kind,kw", [
    ("vanilla", dict(eta=0.1, l1reg=0.01, l2reg=0.02, clip=1.5, batch=4.0)),
    ("rmsprop", dict(eta=0.01, clip=2.0, l2reg=0.001, decay=0.9)),
    ("adam", dict(eta=0.001, iteration=1, l2reg=0.01, clip=3.0)),
])
def test_solver_steps_float64(ctx, kind, kw):
    n = 50021
    w, c1, c2 = _rand(8, (n,)), np.zeros(n), np.zeros(n)
    pw, pc1, pc2 = _up(ctx, w), _up(ctx, c1), _up(ctx, c2)
    for step in range(3):
        g = _rand(9 + step, (n,), 3.0)
        if kind == "adam":
            kw = dict(kw, iteration=kw["iteration"] + (1 if step else 0))
        par, use = O.solver_params(kind=kind, dtype=np.float64, **kw)
        pg = _up(ctx, g)
        ctx.run(D.cmd_solver_step(kind, pw, pg, n, par, use, pc1, pc2, dtype=F64))
        ctx.free(pg)
        w, _, c1, c2 = O.solver_step(kind, w, g, c1, c2, **kw)
        assert_bits_equal(ctx.d2h(pw, (n,), np.float64), w, f"{kind} float64 weights, step {step}")
        if kind != "vanilla":
            assert_bits_equal(ctx.d2h(pc1, (n,), np.float64), c1, f"{kind} float64 cache, step {step}")
        if kind == "adam":
            assert_bits_equal(ctx.d2h(pc2, (n,), np.float64), c2, f"adam float64 v, step {step}")
    for p in (pw, pc1, pc2):
        ctx.free(p)


def test_float64_flags_validate(ctx):
    buf = C.create_string_buffer(256)
    ok = D.cmd_dropout(1, 2, 3, 10, 0.25, dtype=F64)
    assert ctx.lib.gh_validate(C.byref(ok), 1, buf, 256) == 0
    bad = D.cmd_dropout(1, 2, 3, 10, 1.5, dtype=F64)
    assert ctx.lib.gh_validate(C.byref(bad), 1, buf, 256) != 0 and b"probability" in buf.value
    assert ctx.lib.gh_validate(C.byref(D.cmd_rand_uniform(1, 10, 3, dtype=F64)), 1, buf, 256) == 0


def test_uniform_source_float64(ctx):
    """53-bit uniform numbers: bit-identical to the oracle's twin, the float32 stream's values
    are their top 24 bits, and a device-side counter moves the stream on."""
    n = 10007
    out = ctx.malloc(n * 8)
    ctx.run(D.cmd_rand_uniform(out, n, 12345, 77, dtype=F64))
    got = ctx.d2h(out, (n,), np.float64)
    assert_bits_equal(got, O.uniform01(n, 12345, 77, dtype=np.float64), "float64 uniform stream")
    assert np.all((got >= 0) & (got < 1)) and abs(got.mean() - 0.5) < 0.02
    assert np.array_equal(np.floor(got * 2**24) / 2**24, O.uniform01(n, 12345, 77).astype(np.float64))
    state = ctx.upload(np.array([5], np.uint64).view(np.float64))
    ctx.run(D.cmd_rand_uniform(out, 100, 9, state=state, dtype=F64))
    ctx.run(D.cmd_rand_uniform(out, 100, 9, state=state, dtype=F64))
    assert_bits_equal(ctx.d2h(out, (100,), np.float64), O.uniform01(100, 9, 105, dtype=np.float64), "second draw")
    ctx.free(out); ctx.free(state)


def test_float64_training_ops_on_the_tape(ctx):
    """A float64 dense layer trained on the tape machine: MatMul, SoftMax, SoftMaxDiff,
    RectifyDiff, MaxPool2DDiff-free path, RMSProp step - every command carries the float64
    flag and the solver's constants stay doubles; two steps against the oracle's twins."""
    from gorgonia_amd import graph as G
    rng = np.random.default_rng(11)
    x = rng.standard_normal((16, 12))
    w0 = rng.standard_normal((12, 5)) * 0.3
    onehot = np.zeros((16, 5))
    onehot[np.arange(16), np.arange(16) % 5] = 1.0
    g = G.NewGraph()
    xn = G.NewTensor(g, x)
    wn = G.NewTensor(g, w0.copy(), resident=True)
    cache = G.NewTensor(g, np.zeros_like(w0), resident=True)
    yn = G.NewTensor(g, onehot)
    scale = G.NewScalar(g, -1.0 / onehot.size, dtype=np.float64)
    z = G.Mul(xn, wn)
    a = G.Rectify(z)
    out = G.SoftMax(a)
    gout = G.SoftMaxDiff(out, G.HadamardProd(yn, scale))
    dz = G.RectifyDiff(z, gout)
    dw = G.Mul(xn, dz, transA=True)
    res = {"out": G.Read(out, dtype=np.float64), "dw": G.Read(dw, dtype=np.float64)}
    G.SolverStep("rmsprop", wn, dw, [cache], eta=0.01, decay=0.9)
    res["w"] = G.Read(wn, dtype=np.float64)
    m = G.NewTapeMachine(g)
    w, c = w0.copy(), np.zeros_like(w0)
    for step in range(2):
        m.RunAll()
        zz = x @ w
        aa = O.relu(zz).reshape(zz.shape)
        oo = O.softmax(aa)
        go = O.softmax_bwd(oo, O.binop("mul", "vs", onehot.reshape(-1), np.array([-1.0 / onehot.size])).reshape(onehot.shape))
        dzz = O.binop("mul", "vv", go.reshape(-1), O.binop("gte", "vs", zz.reshape(-1), np.zeros(1))).reshape(zz.shape)
        dww = x.T @ dzz
        assert np.allclose(res["out"], oo, rtol=0, atol=1e-12), f"step {step}"
        assert np.allclose(res["dw"], dww, rtol=0, atol=1e-12), f"step {step}"
        w_new, _, c, _ = O.solver_step("rmsprop", w.reshape(-1), res["dw"].reshape(-1), c.reshape(-1), eta=0.01, decay=0.9)
        assert_bits_equal(res["w"].reshape(-1), w_new, f"float64 RMSProp step {step} on the device's own gradient")
        w = w_new.reshape(w0.shape)
    m.Close()


@pytest.mark.parametrize("cfg", [
    (2, 3, 9, 8, 5, 3, 3, (1, 1), (1, 1), (1, 1)),
    (1, 8, 14, 14, 16, 3, 3, (1, 1), (1, 1), (1, 1)),
    (2, 4, 10, 11, 6, 1, 1, (0, 0), (1, 1), (1, 1)),
    (2, 2, 12, 9, 3, 5, 3, (2, 1), (2, 1), (1, 1)),
    (1, 3, 13, 13, 4, 3, 3, (2, 2), (1, 2), (2, 2)),
    # large enough for the matrix-core kernels (filter gradient cut into slices over the pixels,
    # image gradient as a convolution with mirrored filters)
    (8, 32, 14, 14, 64, 3, 3, (1, 1), (1, 1), (1, 1)),
    (32, 1, 28, 28, 32, 3, 3, (1, 1), (1, 1), (1, 1)),
    (3, 16, 21, 20, 40, 3, 3, (1, 1), (2, 2), (1, 1)),
    (2, 20, 23, 23, 24, 5, 3, (4, 2), (1, 1), (2, 2)),
    (5, 70, 7, 7, 130, 3, 3, (1, 1), (1, 1), (1, 1)),
])
def test_conv_gradients_float64(ctx, cfg):
    """Image and filter gradients of Conv2d in float64: relative Frobenius error <= 1e-12
    against the oracle's float64 definition, and equal on integer-valued operands."""
    B, Cn, H, W, F, kh, kw, pad, stride, dil = cfg
    for integer in (False, True):
        rng = np.random.default_rng(21)
        gen = (lambda s: rng.integers(-3, 4, s).astype(np.float64)) if integer else (lambda s: rng.standard_normal(s))
        x, w = gen((B, Cn, H, W)), gen((F, Cn, kh, kw))
        oh, ow = O.conv2d(x, w, pad, stride, dil).shape[2:]
        dy = gen((B, F, oh, ow))
        dx_ref, dw_ref = O.conv2d_bwd(x, w, dy, pad, stride, dil)
        px, pw, pdy = _up(ctx, x), _up(ctx, w), _up(ctx, dy)
        pdx, pdw = ctx.malloc(x.size * 8), ctx.malloc(w.size * 8)
        ctx.run([D.cmd_conv2d_bwd_data(pdy, pw, pdx, B, Cn, H, W, F, kh, kw, pad, stride, dil, dtype=F64),
                 D.cmd_conv2d_bwd_filter(px, pdy, pdw, B, Cn, H, W, F, kh, kw, pad, stride, dil, dtype=F64)])
        dx, dw = ctx.d2h(pdx, x.shape, np.float64), ctx.d2h(pdw, w.shape, np.float64)
        if integer:
            assert np.array_equal(dx, dx_ref) and np.array_equal(dw, dw_ref)
        else:
            assert np.linalg.norm(dx - dx_ref) <= 1e-12 * np.linalg.norm(dx_ref)
            assert np.linalg.norm(dw - dw_ref) <= 1e-12 * np.linalg.norm(dw_ref)
        for p in (px, pw, pdy, pdx, pdw):
            ctx.free(p)


@pytest.mark.parametrize("shape", [(8, 5, 6, 7), (4, 16, 14, 14), (64, 10), (3, 2, 1, 1)])
def test_batchnorm_training_and_gradient_float64(ctx, shape):
    """BN_TRAIN and BN_BWD in float64 against the oracle's twins: relative error <= 1e-12
    (the device sums a channel by a tree, the oracle in sequence)."""
    B, Cn = shape[:2]
    S = int(np.prod(shape[2:])) if len(shape) > 2 else 1
    x, dy = _rand(31, shape), _rand(32, shape)
    rm, rv = _rand(33, (Cn,)), np.random.default_rng(34).random(Cn) + 0.5
    y_ref, rm_ref, rv_ref, sm_ref, sv_ref = O.bn_train_stats(x, rm, rv, 0.9, 1e-5)
    px, py, prm, prv = _up(ctx, x), ctx.malloc(x.size * 8), _up(ctx, rm), _up(ctx, rv)
    psm, psv = ctx.malloc(Cn * 8), ctx.malloc(Cn * 8)
    ctx.run(D.cmd_bn_train(px, py, prm, prv, psm, psv, B, Cn, S, 1e-5, 0.9, dtype=F64))
    close = lambda a, b: np.linalg.norm(a - b) <= 1e-12 * max(np.linalg.norm(b), 1e-300)
    assert close(ctx.d2h(py, shape, np.float64), y_ref)
    assert close(ctx.d2h(prm, (Cn,), np.float64), rm_ref) and close(ctx.d2h(prv, (Cn,), np.float64), rv_ref)
    sm, sv = ctx.d2h(psm, (Cn,), np.float64), ctx.d2h(psv, (Cn,), np.float64)
    assert close(sm, sm_ref) and close(sv, sv_ref)
    pdy, pdx = _up(ctx, dy), ctx.malloc(x.size * 8)
    for training in (True, False):
        ctx.run(D.cmd_bn_bwd(px, pdy, pdx, psm, psv, B, Cn, S, 1e-5, training, dtype=F64))
        want = O.bn_bwd(x, dy, sm, sv, 1e-5, training)
        got = ctx.d2h(pdx, shape, np.float64)
        assert np.linalg.norm(got - want) <= 1e-10 * max(np.linalg.norm(want), 1e-300), (training, shape)
    for p in (px, py, prm, prv, psm, psv, pdy, pdx):
        ctx.free(p)
