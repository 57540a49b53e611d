"""GPU parity: Conv2d (implicit GEMM), MaxPool2D, BatchNorm inference and
SoftMax through the C ABI against the CPU oracle and the reference's golden
vectors.  Bars: max pool bit-exact; conv <= 1e-5 relative Frobenius (exact on
integer data); batch norm bit-exact (contraction off); softmax <= 4 ulp
(<= 2 ulp per exp plus the reciprocal scaling)."""
import json
import os

import numpy as np
import pytest

from gorgonia_amd import device as D
from gorgonia_amd import synth
from oracle import binding as O
from tests.util import assert_bits_equal, rel_frobenius, ulp_diff

pytestmark = pytest.mark.gpu
G = os.path.join(os.path.dirname(__file__), "golden")
TOL = 1e-5


def load(name):
    with open(os.path.join(G, name)) as f:
        return json.load(f)


def gpu_conv(ctx, x, w, pad, stride, dil, act=None, alpha=0.0):
    B, C, H, W = x.shape
    F, _, kh, kw = w.shape
    oh, ow = O.conv_out_hw(H, W, kh, kw, pad, stride, dil)
    dx, dw = ctx.upload(x), ctx.upload(w)
    dy = ctx.malloc(B * F * oh * ow * 4)
    ctx.run(D.cmd_fill(dy, B * F * oh * ow, np.nan))
    ctx.run(D.cmd_conv2d(dx, dw, dy, B, C, H, W, F, kh, kw, pad, stride, dil, act=act, alpha=alpha))
    y = ctx.d2h(dy, (B, F, oh, ow))
    for p in (dx, dw, dy):
        ctx.free(p)
    return y


def test_conv_goldens(ctx):
    """known_issues_test.go:160-199, blas_test.go:426-460 (integer data: exact)."""
    for g in load("conv.json"):
        x = np.array(g["x"], dtype=np.float32).reshape(g["x_shape"])
        w = np.array(g["w"], dtype=np.float32).reshape(g["w_shape"])
        y = gpu_conv(ctx, x, w, g["pad"], g["stride"], g["dilation"])
        assert list(y.shape) == g["y_shape"]
        assert np.array_equal(y.reshape(-1), np.array(g["y"], dtype=np.float32)), g["source"]


CONV_CASES = [
    # B, C, H, W, F, kh, kw, pad, stride, dil
    (2, 3, 8, 9, 5, 3, 3, (1, 1), (1, 1), (1, 1)),
    (1, 4, 7, 7, 6, 1, 1, (0, 0), (1, 1), (1, 1)),
    (2, 2, 10, 11, 3, 3, 2, (2, 1), (2, 3), (1, 1)),
    (1, 3, 12, 12, 4, 3, 3, (2, 2), (1, 1), (2, 2)),
    (2, 5, 9, 9, 7, 5, 5, (2, 2), (1, 1), (1, 1)),
    # convnet layers (configuration 4), batch trimmed to keep the oracle quick
    (16, 1, 28, 28, 32, 3, 3, (1, 1), (1, 1), (1, 1)),
    (16, 32, 14, 14, 64, 3, 3, (1, 1), (1, 1), (1, 1)),
    (16, 64, 7, 7, 128, 3, 3, (1, 1), (1, 1), (1, 1)),
    # tiny-yolo-shaped layers (configuration 5) at reduced spatial size / batch
    (1, 3, 104, 104, 16, 3, 3, (1, 1), (1, 1), (1, 1)),
    (2, 16, 52, 52, 32, 3, 3, (1, 1), (1, 1), (1, 1)),
    (2, 256, 13, 13, 512, 3, 3, (1, 1), (1, 1), (1, 1)),
    (2, 1024, 13, 13, 425, 1, 1, (0, 0), (1, 1), (1, 1)),
]


@pytest.mark.parametrize("cfg", CONV_CASES)
def test_conv_vs_oracle(ctx, cfg):
    B, C, H, W, F, kh, kw, pad, stride, dil = cfg
    x = synth.uniform01(300 + C, (B, C, H, W))
    w = synth.he_normal(400 + F, (F, C, kh, kw))
    y = gpu_conv(ctx, x, w, pad, stride, dil)
    want = O.conv2d(x, w, pad, stride, dil)
    ref = O.conv2d_direct_f64(x, w, pad, stride, dil)
    assert y.shape == want.shape
    err = rel_frobenius(y, ref)
    assert err <= TOL, f"conv {cfg}: rel frobenius {err:.3e}"
    assert rel_frobenius(want, ref) <= TOL
    # integer data: exact whatever the accumulation order
    rng = np.random.default_rng(7)
    xi = rng.integers(-3, 4, (B, C, H, W)).astype(np.float32)
    wi = rng.integers(-3, 4, (F, C, kh, kw)).astype(np.float32)
    assert_bits_equal(gpu_conv(ctx, xi, wi, pad, stride, dil), O.conv2d(xi, wi, pad, stride, dil),
                      f"integer conv {cfg}")


def test_conv_fused_activation_epilogue(ctx):
    x = synth.uniform(1, (4, 8, 14, 14), -1, 1)
    w = synth.he_normal(2, (16, 8, 3, 3))
    plain = gpu_conv(ctx, x, w, (1, 1), (1, 1), (1, 1))
    assert_bits_equal(gpu_conv(ctx, x, w, (1, 1), (1, 1), (1, 1), act="relu"),
                      O.relu(plain).reshape(plain.shape), "conv+relu")
    assert_bits_equal(gpu_conv(ctx, x, w, (1, 1), (1, 1), (1, 1), act="leaky", alpha=0.1),
                      O.leaky_relu(plain, 0.1).reshape(plain.shape), "conv+leaky")


def gpu_pool(ctx, x, kernel, pad, stride):
    B, C, H, W = x.shape
    oh, ow = O.maxpool_out_hw(H, W, kernel[0], kernel[1], pad, stride)
    dx = ctx.upload(x)
    dy = ctx.malloc(B * C * oh * ow * 4)
    ctx.run(D.cmd_maxpool2d(dx, dy, B, C, H, W, kernel[0], kernel[1], pad, stride))
    y = ctx.d2h(dy, (B, C, oh, ow))
    ctx.free(dx); ctx.free(dy)
    return y


def test_maxpool_asymmetric_golden(ctx):
    """nn_test.go:91-138: the reference's own 3072-float input/output pair."""
    g = load("maxpool_asym.json")
    x = np.array(g["x"], dtype=np.float32).reshape(g["shape"])
    y = gpu_pool(ctx, x, g["kernel"], g["pad"], g["stride"])
    assert_bits_equal(y.reshape(-1), np.array(g["y"], dtype=np.float32), "maxpool golden")


@pytest.mark.parametrize("cfg", [
    ((2, 3, 28, 28), (2, 2), (0, 0), (2, 2)),
    ((4, 32, 14, 14), (2, 2), (0, 0), (2, 2)),
    ((4, 128, 7, 7), (2, 2), (0, 0), (2, 2)),       # odd size: last row/col dropped
    ((1, 16, 416, 416), (2, 2), (0, 0), (2, 2)),
    ((2, 512, 13, 13), (2, 2), (1, 0, 1, 0), (1, 1)),  # stride-1 pool of the yolo config
    ((2, 3, 9, 11), (3, 3), (1, 1), (1, 1)),
    ((2, 3, 9, 11), (3, 2), (1, 0), (2, 1)),
    ((1, 1, 4, 4), (4, 4), (0, 0), (1, 1)),
    ((1, 2, 6, 10), (2, 2), (0, 1, 0, 1), (2, 2)),
])
def test_maxpool_bit_exact(ctx, cfg):
    shape, kernel, pad, stride = cfg
    x = synth.normal(500, shape)
    x.reshape(-1)[::7] = 0.0
    x.reshape(-1)[3::11] = -0.0   # which zero wins depends on the scan order
    y = gpu_pool(ctx, x, kernel, pad, stride)
    assert_bits_equal(y, O.maxpool2d(x, kernel, pad, stride), f"maxpool {cfg}")


@pytest.mark.parametrize("shape", [(8, 16, 52, 52), (2, 1024, 13, 13), (3, 2), (256, 300), (2, 3, 5, 7),
                                   (1, 1, 1, 1)])
@pytest.mark.parametrize("affine", [False, True])
def test_batchnorm_infer_bit_exact(ctx, shape, affine):
    Cn = shape[1]
    x = synth.normal(600, shape)
    mean = synth.normal(601, (Cn,), 0.0, 0.1)
    var = synth.uniform(602, (Cn,), 0.5, 1.5)
    gamma = synth.uniform(603, (Cn,), 0.5, 1.5) if affine else None
    beta = synth.normal(604, (Cn,), 0.0, 0.1) if affine else None
    B = shape[0]
    S = int(np.prod(shape)) // (B * Cn)
    dx, dm, dv = ctx.upload(x), ctx.upload(mean), ctx.upload(var)
    dg = ctx.upload(gamma) if affine else 0
    db = ctx.upload(beta) if affine else 0
    dy = ctx.malloc(x.nbytes)
    ctx.run(D.cmd_bn_infer(dx, dy, dm, dv, B, Cn, S, 1e-5, dg, db))
    y = ctx.d2h(dy, shape)
    assert_bits_equal(y, O.bn_infer(x, mean, var, 1e-5, gamma, beta), f"bn {shape}")
    # in place (the reference's op overwrites its output buffer, op_nn.go:1628)
    ctx.run(D.cmd_bn_infer(dx, dx, dm, dv, B, Cn, S, 1e-5, dg, db))
    assert_bits_equal(ctx.d2h(dx, shape), y, "bn in place")
    for p in (dx, dm, dv, dy, dg, db):
        if p:
            ctx.free(p)


def test_batchnorm_eval_goldens(ctx):
    """nn_amd64_test.go ExpectedEvalResult via the same steps the oracle pin
    uses: running stats from one training step (CPU side, not on this path),
    then the GPU eval kernel, then the fully-connected product of the test."""
    from tests.test_oracle_pins import _init, _ranged
    for c in load("batchnorm.json")["cases"]:
        shp = c["x_shape"]
        n = int(np.prod(shp))
        x = (_ranged(*c["x_ranged"], n) if "x_ranged" in c else np.array(c["x"], np.float32)).reshape(shp)
        B, Cn = shp[0], shp[1]
        S = n // (B * Cn)
        gamma, beta = _init(c["scale_init"], Cn), _init(c["bias_init"], Cn)
        _, rm, rv = O.bn_train(x, np.zeros(Cn, np.float32), np.ones(Cn, np.float32), 0.9, 1e-5)
        dx, dm, dv, dg, db = (ctx.upload(a) for a in (x, rm, rv, gamma, beta))
        dy = ctx.malloc(x.nbytes)
        ctx.run(D.cmd_bn_infer(dx, dy, dm, dv, B, Cn, S, 1e-5, dg, db))
        assert_bits_equal(ctx.d2h(dy, shp), O.bn_infer(x, rm, rv, 1e-5, gamma, beta), c["desc"])
        for p in (dx, dm, dv, dg, db, dy):
            ctx.free(p)


@pytest.mark.parametrize("shape", [(256, 10), (128, 10), (1, 1), (5, 64), (7, 65), (33, 1000), (3, 5000)])
def test_softmax(ctx, shape):
    x = synth.normal(700, shape, 0.0, 3.0)
    dx = ctx.upload(x)
    dy = ctx.malloc(x.nbytes)
    ctx.run(D.cmd_softmax(dx, dy, shape[0], shape[1]))
    y = ctx.d2h(dy, shape)
    want = O.softmax(x)
    u = ulp_diff(y, want)
    assert u.max() <= 2, f"softmax {shape}: {u.max()} ulp"
    assert np.allclose(y.sum(axis=1, dtype=np.float64), 1.0, atol=1e-5)
    ctx.free(dx); ctx.free(dy)


def test_softmax_goldens(ctx):
    """op_softmax_test.go:13-100 (float64 goldens, checked at the float32
    tolerance of op_softmax_test.go:110-137)."""
    for c in load("softmax_do.json")["cases"]:
        x = np.array(c["input"], dtype=np.float32).reshape(c["shape"])
        rows = int(np.prod(c["shape"][:-1])) if len(c["shape"]) > 1 else 1
        cols = c["shape"][-1]
        dx = ctx.upload(x)
        dy = ctx.malloc(x.nbytes)
        ctx.run(D.cmd_softmax(dx, dy, rows, cols))
        y = ctx.d2h(dy, x.shape)
        assert np.allclose(y.reshape(-1), c["expected"], rtol=1e-5, atol=1e-7)
        ctx.free(dx); ctx.free(dy)
