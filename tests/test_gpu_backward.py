"""GPU parity of the backward passes and the training-mode BatchNorm forward,
through the C ABI against the CPU oracle.  Bars: max-pool gradient bit-exact
(pure selection and ordered adds); softmax gradient <= 2 ulp; conv gradients
<= 1e-5 relative Frobenius against the float64 definition (exact on integer
data); BatchNorm statistics, output and gradient <= 1e-5 relative (parallel
reduction order differs from the CPU's sequential sums)."""
import numpy as np
import pytest

from gorgonia_amd import _ffi
from gorgonia_amd import device as D
from gorgonia_amd import synth
from oracle import binding as O
from tests.util import assert_bits_equal, rel_frobenius, ulp_diff

pytestmark = pytest.mark.gpu
TOL = 1e-5


POOL_CASES = [
    # B, C, H, W, kernel, pad, stride
    (2, 3, 8, 10, (2, 2), (0, 0), (2, 2)),
    (2, 3, 9, 11, (2, 2), (0, 0), (2, 2)),
    (1, 2, 3, 4, (2, 2), (0, 0), (1, 1)),
    (2, 4, 13, 13, (2, 2), (1, 0, 1, 0), (1, 1)),   # darknet stride-1 pool
    (2, 3, 12, 9, (3, 3), (1, 1), (2, 2)),
    (1, 2, 7, 8, (3, 2), (1, 1), (1, 2)),
    (16, 32, 28, 28, (2, 2), (0, 0), (2, 2)),        # convnet pool 0 (batch trimmed)
    (8, 16, 14, 14, (2, 2), (0, 0), (2, 2)),         # convnet pool 1: rows of 14 (no multiple of four)
    (8, 16, 7, 7, (2, 2), (0, 0), (2, 2)),           # convnet pool 2: odd size, last row and column unpooled
    (1, 1, 2, 3, (2, 2), (0, 0), (2, 2)),
    (1, 2, 3, 2, (2, 2), (0, 0), (2, 2)),
    (1, 1, 2, 2, (2, 2), (0, 0, 0, 0), (2, 2)),      # explicit four-value padding of zero
]


@pytest.mark.parametrize("cfg", POOL_CASES)
def test_maxpool_backward_bit_exact(ctx, cfg):
    B, C, H, W, kernel, pad, stride = cfg
    rng = np.random.default_rng(1)
    for x in (synth.normal(7, (B, C, H, W)), rng.integers(-2, 3, (B, C, H, W)).astype(np.float32)):
        oh, ow = O.maxpool_out_hw(H, W, kernel[0], kernel[1], pad, stride)
        dy = synth.normal(8, (B, C, oh, ow))
        dx_, dy_, dd = ctx.upload(x), ctx.upload(dy), ctx.malloc(x.size * 4)
        ctx.run(D.cmd_fill(dd, x.size, np.nan))
        ctx.run(D.cmd_maxpool2d_bwd(dx_, dy_, dd, B, C, H, W, kernel[0], kernel[1], pad, stride))
        got = ctx.d2h(dd, x.shape)
        for p in (dx_, dy_, dd):
            ctx.free(p)
        assert_bits_equal(got, O.maxpool2d_bwd(x, dy, kernel, pad, stride), f"maxpool backward {cfg}")


@pytest.mark.parametrize("cfg", POOL_CASES)
def test_maxpool_through_rectify_bit_exact(ctx, cfg):
    """GH_FLAG_ACT_RELU on the pooling commands: y = MaxPool2D(Rectify(z)) and its gradient with respect
    to z, each in one pass, with the bits of the separate operators (oracle: relu, pool, pool gradient,
    then dy * (z >= 0)).  Inputs with zeros of both signs and exact ties inside windows."""
    B, C, H, W, kernel, pad, stride = cfg
    rng = np.random.default_rng(2)
    zs = [synth.normal(17, (B, C, H, W)), rng.integers(-2, 3, (B, C, H, W)).astype(np.float32)]
    zs.append(np.where(rng.random((B, C, H, W)) < 0.3, np.float32(-0.0), zs[1]).astype(np.float32))
    for z in zs:
        oh, ow = O.maxpool_out_hw(H, W, kernel[0], kernel[1], pad, stride)
        dy = synth.normal(18, (B, C, oh, ow))
        a = O.relu(z).reshape(z.shape)
        want_y = O.maxpool2d(a, kernel, pad, stride)
        da = O.maxpool2d_bwd(a, dy, kernel, pad, stride)
        want_dz = (da * (z >= 0).astype(np.float32)).astype(np.float32)
        pz, pdy = ctx.upload(z), ctx.upload(dy)
        py, pdz = ctx.malloc(want_y.size * 4), ctx.malloc(z.size * 4)
        ctx.run([D.cmd_fill(py, want_y.size, np.nan), D.cmd_fill(pdz, z.size, np.nan)])
        fwd = D.cmd_maxpool2d(pz, py, B, C, H, W, kernel[0], kernel[1], pad, stride)
        bwd = D.cmd_maxpool2d_bwd(pz, pdy, pdz, B, C, H, W, kernel[0], kernel[1], pad, stride)
        fwd.flags |= _ffi.FLAG_ACT_RELU
        bwd.flags |= _ffi.FLAG_ACT_RELU
        ctx.run([fwd, bwd])
        got_y, got_dz = ctx.d2h(py, want_y.shape), ctx.d2h(pdz, z.shape)
        for p in (pz, pdy, py, pdz):
            ctx.free(p)
        assert_bits_equal(got_y, want_y, f"pool(relu(z)) {cfg}")
        assert_bits_equal(got_dz, want_dz, f"gradient of pool(relu(z)) {cfg}")


@pytest.mark.parametrize("shape", [(1, 1), (7, 10), (128, 10), (5, 64), (3, 65), (4, 1000)])
def test_softmax_backward(ctx, shape):
    x = synth.normal(3, shape)
    y = O.softmax(x)
    dy = synth.normal(4, shape)
    py, pg, pd = ctx.upload(y), ctx.upload(dy), ctx.malloc(y.size * 4)
    ctx.run(D.cmd_softmax_bwd(py, pg, pd, shape[0], shape[1]))
    got = ctx.d2h(pd, shape)
    for p in (py, pg, pd):
        ctx.free(p)
    want = O.softmax_bwd(y, dy)
    assert ulp_diff(got, want).max() <= 2
    assert np.allclose(got.sum(axis=1), 0, atol=1e-5)


CONV_BWD_CASES = [
    # B, C, H, W, F, kh, kw, pad, stride, dil
    (2, 3, 8, 9, 5, 3, 3, (1, 1), (1, 1), (1, 1)),
    (1, 4, 7, 7, 6, 1, 1, (0, 0), (1, 1), (1, 1)),
    (2, 2, 10, 11, 3, 3, 2, (2, 1), (2, 3), (1, 1)),       # strided: gather kernel for dx
    (1, 3, 12, 12, 4, 3, 3, (2, 2), (1, 1), (2, 2)),
    (2, 5, 9, 9, 7, 5, 5, (2, 2), (1, 1), (1, 1)),
    (2, 4, 9, 9, 3, 3, 3, (3, 3), (1, 1), (1, 1)),          # padding wider than the kernel reach: gather kernel
    (16, 1, 28, 28, 32, 3, 3, (1, 1), (1, 1), (1, 1)),      # convnet layers, batch trimmed
    (16, 32, 14, 14, 64, 3, 3, (1, 1), (1, 1), (1, 1)),
    (16, 64, 7, 7, 128, 3, 3, (1, 1), (1, 1), (1, 1)),
    (2, 16, 52, 52, 32, 3, 3, (1, 1), (1, 1), (1, 1)),
    (2, 256, 13, 13, 512, 3, 3, (1, 1), (1, 1), (1, 1)),
    # the small-image filter-gradient kernel (3x3, images up to 16x16, channels in sixteens, >= 16 filters):
    # a ragged filter tile, image groups that do not divide the batch, no padding, H != W, one slab with
    # many groups per workgroup (the tiles alone fill the device), the 16x16 limit, three-pixel images
    (7, 16, 7, 7, 40, 3, 3, (1, 1), (1, 1), (1, 1)),
    (9, 32, 6, 11, 80, 3, 3, (0, 0), (1, 1), (1, 1)),
    (5, 48, 16, 16, 17, 3, 3, (1, 1), (1, 1), (1, 1)),
    (3, 512, 5, 4, 1024, 3, 3, (1, 1), (1, 1), (1, 1)),
    (33, 16, 3, 3, 16, 3, 3, (1, 1), (1, 1), (1, 1)),
    (130, 16, 14, 14, 64, 3, 3, (1, 1), (1, 1), (1, 1)),
    # Conv1d shapes (ops/nn/api_cuda.go:18-20): H = 1, kernel {1,k}
    (3, 4, 1, 37, 6, 1, 3, (0, 1), (1, 1), (1, 1)),
    (2, 8, 1, 64, 16, 1, 5, (0, 2), (1, 2), (1, 1)),
    (2, 3, 1, 50, 5, 1, 3, (0, 2), (1, 1), (1, 2)),
]


def gpu_conv_bwd(ctx, x, w, dy, pad, stride, dil):
    B, C, H, W = x.shape
    F, _, kh, kw = w.shape
    px, pw, pg = ctx.upload(x), ctx.upload(w), ctx.upload(dy)
    pdx, pdw = ctx.malloc(x.size * 4), ctx.malloc(w.size * 4)
    ctx.run([D.cmd_fill(pdx, x.size, np.nan), D.cmd_fill(pdw, w.size, np.nan)])
    ctx.run([D.cmd_conv2d_bwd_data(pg, pw, pdx, B, C, H, W, F, kh, kw, pad, stride, dil),
             D.cmd_conv2d_bwd_filter(px, pg, pdw, B, C, H, W, F, kh, kw, pad, stride, dil)])
    dx, dw = ctx.d2h(pdx, x.shape), ctx.d2h(pdw, w.shape)
    for p in (px, pw, pg, pdx, pdw):
        ctx.free(p)
    return dx, dw


@pytest.mark.parametrize("cfg", CONV_BWD_CASES)
def test_conv_backward_vs_oracle(ctx, cfg):
    B, C, H, W, F, kh, kw, pad, stride, dil = cfg
    x = synth.uniform(300 + C, (B, C, H, W), -1, 1)
    w = synth.he_normal(400 + F, (F, C, kh, kw))
    oh, ow = O.conv_out_hw(H, W, kh, kw, pad, stride, dil)
    dy = synth.normal(500 + F, (B, F, oh, ow))
    dx, dw = gpu_conv_bwd(ctx, x, w, dy, pad, stride, dil)
    if B * C * H * W * F * kh * kw <= 4e8:
        rx, rw = O.conv2d_bwd_direct_f64(x, w, dy, pad, stride, dil)   # float64 definition
    else:
        rx, rw = O.conv2d_bwd(x, w, dy, pad, stride, dil)              # float32 port (pinned to the definition)
    assert rel_frobenius(dx, rx) <= TOL, f"dx {cfg}: {rel_frobenius(dx, rx):.3e}"
    assert rel_frobenius(dw, rw) <= TOL, f"dw {cfg}: {rel_frobenius(dw, rw):.3e}"
    # integer data: exact whatever the accumulation order
    rng = np.random.default_rng(7)
    xi = rng.integers(-3, 4, x.shape).astype(np.float32)
    wi = rng.integers(-3, 4, w.shape).astype(np.float32)
    di = rng.integers(-2, 3, dy.shape).astype(np.float32)
    dxi, dwi = gpu_conv_bwd(ctx, xi, wi, di, pad, stride, dil)
    oxi, owi = O.conv2d_bwd(xi, wi, di, pad, stride, dil)
    assert_bits_equal(dxi, oxi, f"integer dx {cfg}")
    assert_bits_equal(dwi, owi, f"integer dw {cfg}")


def test_small_image_filter_gradient_random_geometries(ctx):
    """Forty random geometries in the small-image filter-gradient kernel's domain (and just outside it:
    fewer than four output pixels, 15 filters) against the oracle: <= 1e-5 on real data, exact on integers."""
    rng = np.random.default_rng(2024)
    for it in range(40):
        B = int(rng.integers(1, 41)); C = int(rng.choice([16, 32, 48, 64])); F = int(rng.integers(15, 101))
        H = int(rng.integers(3, 17)); W = int(rng.integers(3, 17)); pad = int(rng.integers(0, 2))
        cfg = (B, C, H, W, F, pad)
        oh, ow = H + 2 * pad - 2, W + 2 * pad - 2
        x = synth.uniform(600 + it, (B, C, H, W), -1, 1)
        w = synth.he_normal(700 + it, (F, C, 3, 3))
        dy = synth.normal(800 + it, (B, F, oh, ow))
        _, dw = gpu_conv_bwd(ctx, x, w, dy, (pad, pad), (1, 1), (1, 1))
        _, rw = O.conv2d_bwd(x, w, dy, (pad, pad), (1, 1), (1, 1))
        assert rel_frobenius(dw, rw) <= TOL, f"dw {cfg}: {rel_frobenius(dw, rw):.3e}"
        xi = rng.integers(-3, 4, x.shape).astype(np.float32)
        di = rng.integers(-2, 3, dy.shape).astype(np.float32)
        _, dwi = gpu_conv_bwd(ctx, xi, w, di, (pad, pad), (1, 1), (1, 1))
        _, owi = O.conv2d_bwd(xi, w, di, (pad, pad), (1, 1), (1, 1))
        assert_bits_equal(dwi, owi, f"integer dw {cfg}")


@pytest.mark.parametrize("cfg", [(3, 16, 5, 5, 32, 1), (5, 32, 7, 7, 64, 1), (2, 16, 6, 5, 16, 0)])
def test_small_image_filter_gradient_keeps_infinities(ctx, cfg):
    """An infinite input value makes the filter-gradient entries it reaches infinite and leaves every
    other entry as it was (geometries whose pixel count per staged group is no multiple of four, so the
    last MFMA step has padding k: those must not multiply a zero gradient by the infinity)."""
    B, C, H, W, F, pad = cfg
    oh, ow = H + 2 * pad - 2, W + 2 * pad - 2
    x = synth.uniform(900, (B, C, H, W), -1, 1)
    w = synth.he_normal(901, (F, C, 3, 3))
    dy = np.abs(synth.normal(902, (B, F, oh, ow))) + 0.25     # positive: an infinite term stays +inf in the sum
    _, clean = gpu_conv_bwd(ctx, x, w, dy, (pad, pad), (1, 1), (1, 1))
    x[0, :, 0, 0] = np.inf
    _, dw = gpu_conv_bwd(ctx, x, w, dy, (pad, pad), (1, 1), (1, 1))
    with np.errstate(all="ignore"):
        _, rw = O.conv2d_bwd(x, w, dy, (pad, pad), (1, 1), (1, 1))
    assert not np.isnan(rw).any() and np.isinf(rw).any()
    assert np.array_equal(np.isnan(dw), np.isnan(rw)), f"{int(np.isnan(dw).sum())} NaN in the device's dW"
    assert np.array_equal(np.isposinf(dw), np.isposinf(rw)) and np.array_equal(np.isneginf(dw), np.isneginf(rw))
    fin = np.isfinite(rw)
    assert np.allclose(dw[fin], clean[fin], rtol=1e-4, atol=1e-5)


BN_CASES = [(3, 2, 1), (6, 4, 1), (2, 2, 4), (4, 3, 25), (8, 16, 26 * 26), (2, 32, 104 * 104), (128, 10, 1)]


@pytest.mark.parametrize("B,C,S", BN_CASES)
def test_batchnorm_training_forward_and_backward(ctx, B, C, S):
    x = synth.normal(21, (B, C, S), 0.5, 2.0)
    dy = synth.normal(22, (B, C, S))
    rm0, rv0 = synth.normal(23, (C,), 0.0, 0.1), synth.uniform(24, (C,), 0.5, 1.5)
    px, pg = ctx.upload(x), ctx.upload(dy)
    py, pdx = ctx.malloc(x.size * 4), ctx.malloc(x.size * 4)
    prm, prv = ctx.upload(rm0), ctx.upload(rv0)
    psm, psv = ctx.malloc(C * 4), ctx.malloc(C * 4)
    ctx.run(D.cmd_bn_train(px, py, prm, prv, psm, psv, B, C, S, 1e-5, 0.9))
    y, rm, rv = ctx.d2h(py, x.shape), ctx.d2h(prm, (C,)), ctx.d2h(prv, (C,))
    sm, sv = ctx.d2h(psm, (C,)), ctx.d2h(psv, (C,))
    wy, wrm, wrv, wsm, wsv = O.bn_train_stats(x, rm0, rv0, 0.9, 1e-5)
    assert np.allclose(sm, wsm, rtol=1e-5, atol=1e-6) and np.allclose(sv, wsv, rtol=1e-5)
    assert np.allclose(rm, wrm, rtol=1e-5, atol=1e-6) and np.allclose(rv, wrv, rtol=1e-5)
    assert rel_frobenius(y, wy) <= TOL
    # the reductions also agree with float64 sums of the same data
    x64 = x.astype(np.float64)
    assert np.allclose(sm, x64.mean(axis=(0, 2)), rtol=1e-5, atol=1e-6)
    assert np.allclose(sv, ((x64 - x64.mean(axis=(0, 2), keepdims=True)) ** 2).sum(axis=(0, 2)), rtol=1e-5)
    for training in (True, False):
        ctx.run(D.cmd_bn_bwd(px, pg, pdx, psm, psv, B, C, S, 1e-5, training=training))
        dx = ctx.d2h(pdx, x.shape)
        want = O.bn_bwd(x, dy, sm, sv, 1e-5, training=training)   # same saved statistics as the device used
        assert rel_frobenius(dx, want) <= TOL, f"bn backward training={training}: {rel_frobenius(dx, want):.3e}"
    for p in (px, pg, py, pdx, prm, prv, psm, psv):
        ctx.free(p)


@pytest.mark.parametrize("kind,kw", [
    ("vanilla", dict(eta=0.05)),
    ("vanilla", dict(eta=0.05, l1reg=0.01, l2reg=0.02, clip=0.5, batch=4.0)),
    ("rmsprop", dict(eta=0.01, l2reg=1e-6, clip=5.0, decay=0.999)),
    ("rmsprop", dict(eta=0.001)),
    ("adam", dict(eta=0.1, iteration=1)),
    ("adam", dict(eta=0.02, l1reg=0.001, l2reg=0.002, clip=1.0, batch=2.0, iteration=7)),
])
def test_solver_steps_bit_exact(ctx, kind, kw):
    """Three consecutive steps on the device against the oracle's (which is pinned by the
    reference's RMSProp closed form and Adam golden): weights and caches bit for bit."""
    n = 100003
    w = synth.normal(31, (n,))
    c1 = np.zeros(n, np.float32)
    c2 = np.zeros(n, np.float32)
    pw, pc1, pc2 = ctx.upload(w), ctx.upload(c1), ctx.upload(c2)
    for step in range(3):
        g = synth.normal(40 + step, (n,), 0.0, 3.0)
        if kind == "adam":
            kw = dict(kw, iteration=kw["iteration"] + (1 if step else 0))
        par, use = O.solver_params(kind=kind, **kw)
        pg = ctx.upload(g)
        ctx.run(D.cmd_solver_step(kind, pw, pg, n, par, use, pc1, pc2))
        ctx.free(pg)
        w, _, c1, c2 = O.solver_step(kind, w, g, c1, c2, **kw)
        assert_bits_equal(ctx.d2h(pw, (n,)), w, f"{kind} weights, step {step}")
        if kind != "vanilla":
            assert_bits_equal(ctx.d2h(pc1, (n,)), c1, f"{kind} cache, step {step}")
        if kind == "adam":
            assert_bits_equal(ctx.d2h(pc2, (n,)), c2, f"adam v, step {step}")
    for p in (pw, pc1, pc2):
        ctx.free(p)


@pytest.mark.parametrize("kind,kw", [("rmsprop", dict(eta=0.01, clip=2.0)), ("adam", dict(eta=0.001, iteration=3))])
def test_solver_steps_of_many_tensors_in_one_submit(ctx, kind, kw):
    """A run of solver steps with the same settings handed over in one submit is executed as
    one launch; weights and caches are those of one submit per tensor (eleven tensors: more
    than one launch holds; ragged and empty sizes; the first tensor stepped twice, in order)."""
    sizes = [1, 255, 256, 257, 1000, 0, 70001, 33, 4096, 5, 12345]
    par, use = O.solver_params(kind=kind, **kw)
    ws = [synth.normal(50 + i, (max(n, 1),))[:n] for i, n in enumerate(sizes)]
    gs = [synth.normal(80 + i, (max(n, 1),), 0.0, 3.0)[:n] for i, n in enumerate(sizes)]
    results = []
    for batched in (False, True):
        bufs = []
        cmds = []
        for w, g in zip(ws, gs):
            n = w.size
            pw, pg = ctx.upload(w if n else np.zeros(1, np.float32)), ctx.upload(g if n else np.zeros(1, np.float32))
            pc1, pc2 = ctx.upload(np.zeros(max(n, 1), np.float32)), ctx.upload(np.zeros(max(n, 1), np.float32))
            bufs.append((pw, pg, pc1, pc2, n))
            cmds.append(D.cmd_solver_step(kind, pw, pg, n, par, use, pc1, pc2))
        cmds.append(D.cmd_solver_step(kind, bufs[0][0], bufs[0][1], sizes[0], par, use, bufs[0][2], bufs[0][3]))
        if batched:
            ctx.run(cmds)
        else:
            for c in cmds:
                ctx.run(c)
        results.append([(ctx.d2h(pw, (max(n, 1),))[:n], ctx.d2h(pc1, (max(n, 1),))[:n], ctx.d2h(pc2, (max(n, 1),))[:n])
                        for pw, pg, pc1, pc2, n in bufs])
        for b in bufs:
            for q in b[:4]:
                ctx.free(q)
    for (w1, a1, b1), (w2, a2, b2) in zip(*results):
        assert_bits_equal(w1, w2, "weights: one submit == one submit per tensor")
        assert_bits_equal(a1, a2, "cache")
        assert_bits_equal(b1, b2, "second cache")
    w_ref, _, c_ref, v_ref = O.solver_step(kind, ws[4], gs[4], np.zeros(1000, np.float32), np.zeros(1000, np.float32), **kw)
    assert_bits_equal(results[1][4][0], w_ref, "batched step vs oracle")


@pytest.mark.parametrize("n", [1, 3, 4, 1000, 262147])
def test_relu_backward_is_gte_then_hadamard(ctx, n):
    """RELU_BWD stores the bits of Gte(x, 0) followed by HadamardProd with the gradient
    (special values included), also in place on the gradient."""
    x = synth.normal(61, (n,))
    dy = synth.normal(62, (n,))
    special = np.array([0.0, -0.0, np.nan, np.inf, -np.inf, 1e-45, -1e-45], np.float32)
    k = min(n, special.size)
    x[:k] = special[:k]
    dy[n - k:] = special[:k]
    mask = O.binop("gte", "vs", x, np.zeros(1, np.float32))
    want = O.binop("mul", "vv", dy, mask)
    px, pdy, pdx = ctx.upload(x), ctx.upload(dy), ctx.malloc(n * 4)
    ctx.run(D.cmd_relu_bwd(px, pdy, pdx, n))
    assert_bits_equal(ctx.d2h(pdx, (n,)), want, "relu backward")
    ctx.run(D.cmd_relu_bwd(px, pdy, pdy, n))
    assert_bits_equal(ctx.d2h(pdy, (n,)), want, "relu backward in place")
    for p in (px, pdy, pdx):
        ctx.free(p)


def test_backward_commands_validate(ctx):
    import ctypes as C
    buf = C.create_string_buffer(256)
    bad = D.cmd_conv2d_bwd_data(0x1000, 0x2000, 0x3000, 2, 8, 14, 14, 16, 3, 3, (1, 1))
    bad.flags |= 1 << 22
    assert ctx.lib.gh_validate(C.byref(bad), 1, buf, 256) != 0
    ok = D.cmd_conv2d_bwd_filter(0x1000, 0x2000, 0x3000, 2, 8, 14, 14, 16, 3, 3, (1, 1))
    assert ctx.lib.gh_validate(C.byref(ok), 1, buf, 256) == 0
    assert ctx.lib.gh_validate(C.byref(D.cmd_bn_train(1, 2, 3, 4, 5, 6, 1, 4, 1, 1e-5, 0.9)), 1, buf, 256) != 0
    assert ctx.lib.gh_validate(C.byref(D.cmd_softmax_bwd(1, 2, 0, 4, 4)), 1, buf, 256) != 0
