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
    # small images with 16 and 128 channels (the K-split small-image kernel)
    (9, 16, 12, 12, 33, 3, 3, (1, 1), (1, 1), (1, 1)),
    (4, 128, 6, 6, 24, 3, 3, (0, 0), (1, 1), (1, 1)),
    # tiny-yolo-shaped layers (configuration 5) at reduced spatial size / batch
    (1, 3, 104, 104, 16, 3, 3, (1, 1), (1, 1), (1, 1)),
    (2, 16, 52, 52, 32, 3, 3, (1, 1), (1, 1), (1, 1)),
    (2, 256, 13, 13, 512, 3, 3, (1, 1), (1, 1), (1, 1)),
    (2, 1024, 13, 13, 425, 1, 1, (0, 0), (1, 1), (1, 1)),
    # wide rows: the LDS kernel's rectangular-tile layout, partial tiles on both axes
    (1, 8, 71, 75, 16, 3, 3, (1, 1), (1, 1), (1, 1)),
    (2, 16, 66, 68, 40, 3, 3, (0, 0), (1, 1), (1, 1)),
    (1, 8, 104, 104, 64, 3, 3, (1, 1), (1, 1), (1, 1)),
    (1, 16, 70, 130, 96, 3, 3, (1, 1), (1, 1), (1, 1)),
    # Conv1d (ops/nn/api_cuda.go:18-20): H = 1, kernel {1,k}, pad {0,p}, stride {1,s}, dilation {1,d}
    (3, 4, 1, 37, 6, 1, 3, (0, 1), (1, 1), (1, 1)),
    (2, 8, 1, 64, 16, 1, 5, (0, 2), (1, 2), (1, 1)),
    (2, 3, 1, 50, 5, 1, 3, (0, 2), (1, 1), (1, 2)),
    (4, 16, 1, 128, 32, 1, 7, (0, 0), (1, 3), (1, 2)),
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


def gpu_conv_tail(ctx, x, w, pad, bn=None, act=None, alpha=0.0, pool2=False, eps=1e-5):
    """Conv2d with followers in its epilogue: bn = (mean, var, gamma|None, beta|None) host arrays."""
    B, C, H, W = x.shape
    F, _, kh, kw = w.shape
    oh, ow = O.conv_out_hw(H, W, kh, kw, pad, (1, 1), (1, 1))
    yh, yw = (oh // 2, ow // 2) if pool2 else (oh, ow)
    held = [ctx.upload(x), ctx.upload(w)]
    dbn = None
    if bn is not None:
        dbn = tuple(0 if a is None else ctx.upload(a) for a in bn)
        held += [p for p in dbn if p]
    dy = ctx.malloc(B * F * yh * yw * 4)
    held.append(dy)
    ctx.run(D.cmd_fill(dy, B * F * yh * yw, np.nan))
    ctx.run(D.cmd_conv2d(held[0], held[1], dy, B, C, H, W, F, kh, kw, pad, act=act, alpha=alpha, bn=dbn,
                         eps=eps, pool2=pool2))
    y = ctx.d2h(dy, (B, F, yh, yw))
    for p in held:
        ctx.free(p)
    return y


def gpu_bn(ctx, x, mean, var, gamma, beta, eps):
    B, C = x.shape[:2]
    S = x.size // (B * C)
    dx, dm, dv = ctx.upload(x), ctx.upload(mean), ctx.upload(var)
    dg = ctx.upload(gamma) if gamma is not None else 0
    db = ctx.upload(beta) if beta is not None else 0
    ctx.run(D.cmd_bn_infer(dx, dx, dm, dv, B, C, S, eps, gamma=dg, beta=db))
    y = ctx.d2h(dx, x.shape)
    for p in (dx, dm, dv, dg, db):
        if p:
            ctx.free(p)
    return y


# shapes that reach each convolution kernel: the direct one (C <= 4), the
# LDS-staged 3x3 one with and without split-K, the gather one (1x1)
TAIL_CASES = [(2, 3, 20, 22, 16, 3, 1), (3, 1, 28, 28, 32, 3, 1), (2, 4, 9, 9, 5, 3, 0),
              (2, 16, 26, 26, 32, 3, 1), (2, 256, 13, 13, 64, 3, 1), (2, 64, 13, 13, 40, 1, 0),
              (1, 16, 60, 72, 32, 3, 1), (1, 64, 52, 80, 72, 3, 1)]


@pytest.mark.parametrize("cfg", TAIL_CASES)
def test_conv_epilogue_batchnorm_activation_bit_exact(ctx, cfg):
    """conv -> BatchNorm(eval) -> LeakyReLU as one command stores the bits of the three separate commands."""
    B, C, H, W, F, k, pad = cfg
    x = synth.uniform(11, (B, C, H, W), -1, 1)
    w = synth.he_normal(12, (F, C, k, k))
    mean, var = synth.normal(13, (F,), 0.0, 0.1), synth.uniform(14, (F,), 0.5, 1.5)
    gamma, beta = synth.uniform(15, (F,), 0.5, 1.5), synth.normal(16, (F,), 0.0, 0.1)
    plain = gpu_conv(ctx, x, w, (pad, pad), (1, 1), (1, 1))
    for g, b in ((gamma, beta), (None, None)):
        bn = gpu_bn(ctx, plain.copy(), mean, var, g, b, 1e-5)
        assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), bn=(mean, var, g, b)), bn, f"conv+bn {cfg}")
        assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), bn=(mean, var, g, b), act="leaky", alpha=0.1),
                          O.leaky_relu(bn, 0.1).reshape(bn.shape), f"conv+bn+leaky {cfg}")
    # and against the oracle's own batch norm of the same convolution result
    want = O.bn_infer(plain, mean, var, 1e-5, gamma, beta)
    assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), bn=(mean, var, gamma, beta)), want, "vs oracle bn")


@pytest.mark.parametrize("cfg", [(3, 1, 28, 28, 32, 1), (2, 3, 21, 19, 16, 1), (2, 4, 10, 12, 6, 0),
                                 (1, 2, 7, 7, 9, 1), (2, 2, 9, 8, 7, 2), (1, 4, 6, 11, 5, 2),   # padding wider than one
                                 # the matrix-core kernel: blocks of whole rows (even height, blocks crossing
                                 # images), whole images (odd height), 128-pixel blocks, rectangular tiles
                                 (5, 32, 14, 14, 64, 1), (3, 16, 7, 7, 40, 1), (130, 8, 7, 7, 8, 1),
                                 (2, 8, 26, 26, 16, 1), (2, 8, 16, 16, 70, 0), (2, 8, 52, 52, 8, 1),
                                 (1, 8, 70, 66, 24, 1), (1, 16, 64, 66, 48, 0), (2, 8, 9, 5, 16, 1)])
def test_conv_epilogue_pool_bit_exact(ctx, cfg):
    """conv -> ReLU -> MaxPool 2x2/2 as one command (odd sizes drop the last row/column)."""
    B, C, H, W, F, pad = cfg
    x = synth.uniform(21, (B, C, H, W), -1, 1)
    w = synth.he_normal(22, (F, C, 3, 3))
    cmd = D.cmd_conv2d(1, 1, 1, B, C, H, W, F, 3, 3, (pad, pad))
    assert ctx.lib.gh_conv2d_can_pool(cmd) == 1
    act = gpu_conv(ctx, x, w, (pad, pad), (1, 1), (1, 1), act="relu")
    want = gpu_pool(ctx, act, (2, 2), (0, 0), (2, 2))
    got = gpu_conv_tail(ctx, x, w, (pad, pad), act="relu", pool2=True)
    assert_bits_equal(got, want, f"conv+relu+pool {cfg}")
    assert_bits_equal(want, O.maxpool2d(O.relu(act).reshape(act.shape), (2, 2), (0, 0), (2, 2)), "pool vs oracle")
    mean, var = synth.normal(23, (F,), 0.0, 0.1), synth.uniform(24, (F,), 0.5, 1.5)
    plain = gpu_conv(ctx, x, w, (pad, pad), (1, 1), (1, 1))
    chain = gpu_pool(ctx, O.leaky_relu(gpu_bn(ctx, plain.copy(), mean, var, None, None, 1e-5), 0.1).reshape(plain.shape),
                     (2, 2), (0, 0), (2, 2))
    assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), bn=(mean, var, None, None), act="leaky", alpha=0.1,
                                    pool2=True), chain, f"conv+bn+leaky+pool {cfg}")


# one shape per convolution kernel that carries an epilogue: direct (C <= 4), small images, patches of
# deep layers, wide images, the LDS-tiled 3x3 one, and the gather kernel (1x1)
SPECIAL_VALUE_CASES = [(3, 1, 28, 28, 32, 3, 1), (5, 32, 14, 14, 64, 3, 1), (2, 256, 13, 13, 64, 3, 1),
                       (2, 16, 130, 131, 32, 3, 1), (1, 64, 52, 80, 72, 3, 1), (2, 64, 13, 13, 40, 1, 0)]


@pytest.mark.parametrize("cfg", SPECIAL_VALUE_CASES)
def test_conv_epilogue_special_values_bit_exact(ctx, cfg):
    """Epilogues on results that are +0, -0, infinite, NaN, tiny and huge: images with blank (+0) and -0
    regions, a few infinities and NaNs, values near overflow, filters with zeroed taps.  The activations'
    short forms must store what the reference's arithmetic (pos + neg * alpha on the plain result) stores
    for every such value and every alpha sign, and pooling must keep the first of a tie between zeros."""
    B, C, H, W, F, k, pad = cfg
    rng = np.random.default_rng(77)
    x = synth.uniform(71, (B, C, H, W), -1, 1)
    x[:, :, : H // 3, :] = 0.0                       # blank rows: results exactly +0
    x[:, :, H // 3: H // 2, : W // 2] = -0.0
    x[0, 0, H - 2, W - 2] = np.inf
    x[B - 1, C - 1, H // 2 + 1, 1] = -np.inf
    x[0, C // 2, H - 3, W // 2] = np.nan
    x[B - 1, 0, H - 1, :] *= 3e38                    # products overflow for some filters
    x[0, 0, H // 2 + 2, :] *= 1e-38                  # denormal products
    w = synth.he_normal(72, (F, C, k, k))
    w[rng.integers(0, F, 8), rng.integers(0, C, 8)] = 0.0
    w[1 % F] = -np.abs(w[1 % F])
    plain = gpu_conv(ctx, x, w, (pad, pad), (1, 1), (1, 1))
    assert np.isnan(plain).any() and np.isinf(plain).any() and (plain == 0).any()
    mean, var = synth.normal(73, (F,), 0.0, 0.1), synth.uniform(74, (F,), 0.5, 1.5)
    gamma, beta = synth.uniform(75, (F,), 0.5, 1.5), synth.normal(76, (F,), 0.0, 0.1)
    cmd = D.cmd_conv2d(1, 1, 1, B, C, H, W, F, k, k, (pad, pad))
    can_pool = ctx.lib.gh_conv2d_can_pool(cmd) == 1
    relu = O.relu(plain).reshape(plain.shape)
    assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), act="relu"), relu, f"conv+relu {cfg}")
    if can_pool:
        assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), act="relu", pool2=True),
                          O.maxpool2d(relu, (2, 2), (0, 0), (2, 2)), f"conv+relu+pool {cfg}")
        assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), pool2=True),
                          O.maxpool2d(plain, (2, 2), (0, 0), (2, 2)), f"conv+pool {cfg}")
    for alpha in (0.1, 0.0, -0.5, 2.0, np.inf):
        leaky = O.leaky_relu(plain, alpha).reshape(plain.shape)
        assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), act="leaky", alpha=alpha), leaky,
                          f"conv+leaky({alpha}) {cfg}")
        for g, b in ((gamma, beta), (None, beta), (gamma, None), (None, None)):
            bn = O.bn_infer(plain, mean, var, 1e-5, g, b)
            want = O.leaky_relu(bn, alpha).reshape(plain.shape)
            assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), bn=(mean, var, g, b), act="leaky", alpha=alpha),
                              want, f"conv+bn+leaky({alpha}) gamma={g is not None} beta={b is not None} {cfg}")
            if can_pool and alpha in (0.1, -0.5):
                assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), bn=(mean, var, g, b), act="leaky",
                                                alpha=alpha, pool2=True),
                                  O.maxpool2d(want, (2, 2), (0, 0), (2, 2)), f"conv+bn+leaky({alpha})+pool {cfg}")


# shapes the K-split small-image kernel takes (3x3, images up to 16x16, 16 or 128 channels): ragged filter
# tiles, batches that do not fill the last workgroup, no padding, odd and even extents, H != W
SMALL_IMAGE_CASES = [(7, 16, 7, 7, 10, 1), (3, 128, 5, 6, 20, 1), (1, 16, 4, 4, 5, 1), (4, 128, 6, 6, 24, 0),
                     (9, 16, 8, 15, 33, 1), (6, 16, 10, 9, 17, 0)]
# and those of the kernel with the pixels on the MFMA rows (32 or 64 channels, 4 to 16 pixels wide): the
# same kinds, plus the smallest and largest images it takes, odd output extents on either axis (the
# pixels outside every pooling window), more filters than one round of workgroups, and a batch that
# leaves the last workgroup's image slots partly empty
ROWS_CASES = [(5, 32, 14, 14, 50, 1), (9, 64, 7, 7, 33, 1), (6, 32, 16, 16, 16, 0), (2, 64, 9, 13, 17, 0),
              (11, 32, 6, 11, 64, 1), (130, 64, 7, 7, 8, 1), (3, 32, 4, 4, 20, 1), (2, 64, 16, 16, 40, 1),
              (1, 32, 3, 5, 7, 1), (17, 64, 2, 16, 130, 1), (4, 32, 5, 4, 33, 0), (35, 64, 8, 5, 300, 1)]


# single-channel images on the matrix cores (even output extents, 16 to 256 filters): the smallest and the
# largest image, ragged filter tiles, a last pixel tile that is partly empty, no padding, H != W
ROWS1_CASES = [(3, 1, 28, 28, 32, 1), (2, 1, 6, 6, 16, 0), (5, 1, 64, 64, 40, 1), (1, 1, 2, 2, 16, 1),
               (4, 1, 10, 30, 256, 1), (7, 1, 8, 12, 17, 1), (2, 1, 6, 8, 20, 0), (130, 1, 4, 6, 33, 1)]


@pytest.mark.parametrize("cfg", SMALL_IMAGE_CASES + ROWS_CASES + ROWS1_CASES)
def test_conv_small_images(ctx, cfg):
    """The two small-image convolution kernels against the oracle (<= 1e-5, exact on integers), and every
    epilogue they can carry against the separate commands bit for bit."""
    B, C, H, W, F, pad = cfg
    x = synth.uniform(31, (B, C, H, W), -1, 1)
    w = synth.he_normal(32, (F, C, 3, 3))
    plain = gpu_conv(ctx, x, w, (pad, pad), (1, 1), (1, 1))
    ref = O.conv2d_direct_f64(x, w, (pad, pad), (1, 1), (1, 1))
    err = rel_frobenius(plain, ref)
    assert err <= TOL, f"small conv {cfg}: rel frobenius {err:.3e}"
    rng = np.random.default_rng(9)
    xi = rng.integers(-3, 4, (B, C, H, W)).astype(np.float32)
    wi = rng.integers(-3, 4, (F, C, 3, 3)).astype(np.float32)
    assert_bits_equal(gpu_conv(ctx, xi, wi, (pad, pad), (1, 1), (1, 1)), O.conv2d(xi, wi, (pad, pad), (1, 1), (1, 1)),
                      f"integer small conv {cfg}")
    mean, var = synth.normal(33, (F,), 0.0, 0.1), synth.uniform(34, (F,), 0.5, 1.5)
    gamma, beta = synth.uniform(35, (F,), 0.5, 1.5), synth.normal(36, (F,), 0.0, 0.1)
    bn = O.bn_infer(plain, mean, var, 1e-5, gamma, beta)
    leaky = O.leaky_relu(bn, 0.1).reshape(bn.shape)
    assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), bn=(mean, var, gamma, beta), act="leaky", alpha=0.1), leaky,
                      f"small conv+bn+leaky {cfg}")
    cmd = D.cmd_conv2d(1, 1, 1, B, C, H, W, F, 3, 3, (pad, pad))
    if plain.shape[2] >= 2 and plain.shape[3] >= 2:
        assert ctx.lib.gh_conv2d_can_pool(cmd) == 1
        relu = O.relu(plain).reshape(plain.shape)
        assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), act="relu", pool2=True),
                          O.maxpool2d(relu, (2, 2), (0, 0), (2, 2)), f"small conv+relu+pool {cfg}")
        assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), bn=(mean, var, gamma, beta), act="leaky", alpha=0.1,
                                        pool2=True),
                          O.maxpool2d(leaky, (2, 2), (0, 0), (2, 2)), f"small conv+bn+leaky+pool {cfg}")


# (B, H, W, F, pad) of the second convolution of a folded first layer: its input has 32 channels and is
# Conv2d 3x3 pad 1 -> Rectify -> MaxPool2D 2x2 of single-channel images of 2H x 2W.  The convnet's own
# layer, ragged filter counts, several images per workgroup, no padding, the smallest and the largest
# images, H != W, a batch that leaves the last workgroup partly empty
PRE_CASES = [(5, 14, 14, 64, 1), (3, 7, 7, 33, 1), (9, 4, 4, 16, 1), (2, 16, 16, 40, 1), (6, 6, 11, 50, 0),
             (130, 5, 8, 20, 1), (1, 14, 14, 64, 1), (4, 9, 13, 130, 0)]


@pytest.mark.parametrize("cfg", PRE_CASES)
def test_conv_folded_first_layer_bit_exact(ctx, cfg):
    """GH_FLAG_CONV_PRE: one command stores the bits of the three it stands for (single-channel
    convolution + Rectify + pool, then the convolution), with and without followers of its own, and
    special values in the image and the first filters travel as they do through the separate commands."""
    B, H, W, F, pad = cfg
    C = 32
    x0 = synth.uniform(71, (B, 1, 2 * H, 2 * W), -1, 1)
    w0 = synth.he_normal(72, (C, 1, 3, 3))
    w1 = synth.he_normal(73, (F, C, 3, 3))
    probe = D.cmd_conv2d(1, 1, 1, B, C, H, W, F, 3, 3, (pad, pad))
    assert ctx.lib.gh_conv2d_can_pre(probe) == 1, cfg
    mean, var = synth.normal(74, (F,), 0.0, 0.1), synth.uniform(75, (F,), 0.5, 1.5)
    gamma, beta = synth.uniform(76, (F,), 0.5, 1.5), synth.normal(77, (F,), 0.0, 0.1)

    def folded(x0, w0, w1=w1, **kw):
        oh, ow = H + 2 * pad - 2, W + 2 * pad - 2
        yh, yw = (oh // 2, ow // 2) if kw.get("pool2") else (oh, ow)
        held = [ctx.upload(x0), ctx.upload(w1), ctx.upload(w0)]
        dbn = None
        if kw.get("bn") is not None:
            dbn = tuple(ctx.upload(a) for a in kw["bn"])
            held += list(dbn)
        dy = ctx.malloc(B * F * yh * yw * 4)
        held.append(dy)
        ctx.run(D.cmd_fill(dy, B * F * yh * yw, np.nan))
        ctx.run(D.cmd_conv2d(held[0], held[1], dy, B, C, H, W, F, 3, 3, (pad, pad), act=kw.get("act"),
                             alpha=kw.get("alpha", 0.0), bn=dbn, pool2=bool(kw.get("pool2")), pre=held[2]))
        y = ctx.d2h(dy, (B, F, yh, yw))
        for p in held:
            ctx.free(p)
        return y

    mid = gpu_conv_tail(ctx, x0, w0, (1, 1), act="relu", pool2=True)
    assert mid.shape == (B, C, H, W)
    ref = O.maxpool2d(O.relu(O.conv2d(x0, w0, (1, 1), (1, 1), (1, 1))).reshape(B, C, 2 * H, 2 * W), (2, 2), (0, 0), (2, 2))
    assert rel_frobenius(mid, ref) <= TOL
    assert_bits_equal(folded(x0, w0), gpu_conv(ctx, mid, w1, (pad, pad), (1, 1), (1, 1)), f"folded {cfg}")
    if H + 2 * pad - 2 >= 2 and W + 2 * pad - 2 >= 2:
        assert_bits_equal(folded(x0, w0, act="relu", pool2=True),
                          gpu_conv_tail(ctx, mid, w1, (pad, pad), act="relu", pool2=True), f"folded+relu+pool {cfg}")
        assert_bits_equal(folded(x0, w0, bn=(mean, var, gamma, beta), act="leaky", alpha=0.1, pool2=True),
                          gpu_conv_tail(ctx, mid, w1, (pad, pad), bn=(mean, var, gamma, beta), act="leaky", alpha=0.1,
                                        pool2=True), f"folded+bn+leaky+pool {cfg}")
    # integers: exact against the oracle's chain
    rng = np.random.default_rng(5)
    xi = rng.integers(-3, 4, x0.shape).astype(np.float32)
    w0i = rng.integers(-2, 3, w0.shape).astype(np.float32)
    w1i = rng.integers(-2, 3, w1.shape).astype(np.float32)
    midi = O.maxpool2d(O.relu(O.conv2d(xi, w0i, (1, 1), (1, 1), (1, 1))).reshape(B, C, 2 * H, 2 * W), (2, 2), (0, 0), (2, 2))
    assert_bits_equal(folded(xi, w0i, w1i), O.conv2d(midi.reshape(B, C, H, W), w1i, (pad, pad), (1, 1), (1, 1)), f"folded integers {cfg}")
    # special values in the image and in the first filters
    xs = x0.copy()
    flat = xs.reshape(-1)
    flat[::37] = np.inf; flat[5::41] = -np.inf; flat[11::43] = np.nan; flat[3::29] = -0.0; flat[7::31] = 0.0
    ws = w0.copy()
    ws.reshape(-1)[4::19] = -0.0
    ws.reshape(-1)[9::23] = np.inf
    mids = gpu_conv_tail(ctx, xs, ws, (1, 1), act="relu", pool2=True)
    assert_bits_equal(folded(xs, ws), gpu_conv(ctx, mids, w1, (pad, pad), (1, 1), (1, 1)), f"folded special values {cfg}")


@pytest.mark.parametrize("cfg", ROWS_CASES + ROWS1_CASES)
def test_conv_keeps_unpooled_result_bit_exact(ctx, cfg):
    """GH_FLAG_CONV_KEEP: one command stores the pooled activation and the convolution's own result, each with
    the bits of the separate commands (what a training step keeps for its backward pass)."""
    B, C, H, W, F, pad = cfg
    oh, ow = H + 2 * pad - 2, W + 2 * pad - 2
    probe = D.cmd_conv2d(1, 1, 1, B, C, H, W, F, 3, 3, (pad, pad))
    if not ctx.lib.gh_conv2d_can_pool(probe):
        assert ctx.lib.gh_conv2d_can_keep(probe) == 0
        return
    assert ctx.lib.gh_conv2d_can_keep(probe) == 1
    x = synth.uniform(81, (B, C, H, W), -1, 1)
    w = synth.he_normal(82, (F, C, 3, 3))
    x.reshape(-1)[::53] = np.inf; x.reshape(-1)[7::59] = np.nan; x.reshape(-1)[3::31] = -0.0
    mean, var = synth.normal(83, (F,), 0.0, 0.1), synth.uniform(84, (F,), 0.5, 1.5)
    gamma, beta = synth.uniform(85, (F,), 0.5, 1.5), synth.normal(86, (F,), 0.0, 0.1)
    for bn, act in ((None, "relu"), ((mean, var, gamma, beta), "leaky"), (None, None)):
        held = [ctx.upload(x), ctx.upload(w)]
        dbn = None
        if bn is not None:
            dbn = tuple(ctx.upload(a) for a in bn)
            held += list(dbn)
        dp = ctx.malloc(B * F * (oh // 2) * (ow // 2) * 4)
        dz = ctx.malloc(B * F * oh * ow * 4)
        held += [dp, dz]
        ctx.run(D.cmd_fill(dp, B * F * (oh // 2) * (ow // 2), np.nan))
        ctx.run(D.cmd_fill(dz, B * F * oh * ow, np.nan))
        ctx.run(D.cmd_conv2d(held[0], held[1], dp, B, C, H, W, F, 3, 3, (pad, pad), act=act, alpha=0.1, bn=dbn,
                             pool2=True, keep=dz))
        p = ctx.d2h(dp, (B, F, oh // 2, ow // 2))
        z = ctx.d2h(dz, (B, F, oh, ow))
        for q in held:
            ctx.free(q)
        assert_bits_equal(z, gpu_conv_tail(ctx, x, w, (pad, pad), bn=bn), f"kept result {cfg} bn={bn is not None}")
        assert_bits_equal(p, gpu_conv_tail(ctx, x, w, (pad, pad), bn=bn, act=act, alpha=0.1, pool2=True),
                          f"pooled result next to a kept one {cfg} act={act}")


# shapes the patch kernel takes (3x3, 64 channels or more, K split over eight wavefronts): partial
# patches on both axes, ragged filter tiles, no padding, pooled extents odd and even
PATCH_CASES = [(2, 64, 20, 17, 40, 1), (2, 64, 28, 28, 32, 1), (1, 64, 24, 14, 20, 0), (1, 96, 26, 26, 48, 1), (3, 128, 13, 13, 70, 1), (1, 64, 31, 18, 16, 0),
               (2, 256, 13, 13, 33, 1), (1, 64, 52, 52, 32, 1), (2, 64, 9, 40, 24, 1)]


@pytest.mark.parametrize("cfg", PATCH_CASES)
def test_conv_patch_kernel(ctx, cfg):
    """The patch convolution kernel against the oracle (<= 1e-5, exact on integers), and every epilogue
    it can carry against the oracle's operators applied to its own plain result, bit for bit."""
    B, C, H, W, F, pad = cfg
    x = synth.uniform(41, (B, C, H, W), -1, 1)
    w = synth.he_normal(42, (F, C, 3, 3))
    plain = gpu_conv(ctx, x, w, (pad, pad), (1, 1), (1, 1))
    ref = O.conv2d_direct_f64(x, w, (pad, pad), (1, 1), (1, 1))
    err = rel_frobenius(plain, ref)
    assert err <= TOL, f"patch conv {cfg}: rel frobenius {err:.3e}"
    rng = np.random.default_rng(10)
    xi = rng.integers(-3, 4, (B, C, H, W)).astype(np.float32)
    wi = rng.integers(-3, 4, (F, C, 3, 3)).astype(np.float32)
    assert_bits_equal(gpu_conv(ctx, xi, wi, (pad, pad), (1, 1), (1, 1)), O.conv2d(xi, wi, (pad, pad), (1, 1), (1, 1)),
                      f"integer patch conv {cfg}")
    mean, var = synth.normal(43, (F,), 0.0, 0.1), synth.uniform(44, (F,), 0.5, 1.5)
    gamma, beta = synth.uniform(45, (F,), 0.5, 1.5), synth.normal(46, (F,), 0.0, 0.1)
    leaky = O.leaky_relu(O.bn_infer(plain, mean, var, 1e-5, gamma, beta), 0.1).reshape(plain.shape)
    assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), bn=(mean, var, gamma, beta), act="leaky", alpha=0.1), leaky,
                      f"patch conv+bn+leaky {cfg}")
    cmd = D.cmd_conv2d(1, 1, 1, B, C, H, W, F, 3, 3, (pad, pad))
    if ctx.lib.gh_conv2d_can_pool(cmd) == 1:
        assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), bn=(mean, var, gamma, beta), act="leaky", alpha=0.1,
                                        pool2=True),
                          O.maxpool2d(leaky, (2, 2), (0, 0), (2, 2)), f"patch conv+bn+leaky+pool {cfg}")


# shapes the 1x1 kernel takes (stride 1, no padding, channels a multiple of 256, four pixels or more per image, too
# few 64x64 tiles to fill the device): ragged filter and pixel tiles, tiles crossing images, image sizes of every
# remainder mod 4 (the last quad of an image overlaps the one before), two and four channel groups in flight,
# every filter-tile height; and two the tiled kernel keeps (one pixel per image, 384 channels)
POINTWISE_CASES = [(2, 1024, 13, 13, 425), (8, 256, 13, 13, 40), (3, 512, 7, 9, 33), (1, 512, 26, 26, 255),
                   (5, 768, 5, 3, 17), (2, 256, 31, 29, 96), (9, 256, 2, 3, 150), (3, 1024, 2, 2, 48), (4, 512, 5, 5, 300), (2, 256, 104, 100, 24),
                   (70, 256, 1, 1, 64), (3, 384, 7, 9, 33)]


@pytest.mark.parametrize("cfg", POINTWISE_CASES)
def test_conv_pointwise_kernel(ctx, cfg):
    """The 1x1 convolution kernel against the oracle (<= 1e-5, exact on integers), and its epilogues against the
    oracle's operators applied to its own plain result, bit for bit."""
    B, C, H, W, F = cfg
    x = synth.uniform(51, (B, C, H, W), -1, 1)
    w = synth.he_normal(52, (F, C, 1, 1))
    plain = gpu_conv(ctx, x, w, (0, 0), (1, 1), (1, 1))
    ref = O.conv2d_direct_f64(x, w, (0, 0), (1, 1), (1, 1))
    err = rel_frobenius(plain, ref)
    assert err <= TOL, f"1x1 conv {cfg}: rel frobenius {err:.3e}"
    rng = np.random.default_rng(11)
    xi = rng.integers(-3, 4, (B, C, H, W)).astype(np.float32)
    wi = rng.integers(-3, 4, (F, C, 1, 1)).astype(np.float32)
    assert_bits_equal(gpu_conv(ctx, xi, wi, (0, 0), (1, 1), (1, 1)), O.conv2d(xi, wi, (0, 0), (1, 1), (1, 1)),
                      f"integer 1x1 conv {cfg}")
    mean, var = synth.normal(53, (F,), 0.0, 0.1), synth.uniform(54, (F,), 0.5, 1.5)
    gamma, beta = synth.uniform(55, (F,), 0.5, 1.5), synth.normal(56, (F,), 0.0, 0.1)
    bn = O.bn_infer(plain, mean, var, 1e-5, gamma, beta)
    assert_bits_equal(gpu_conv_tail(ctx, x, w, (0, 0), bn=(mean, var, gamma, beta)), bn, f"1x1 conv+bn {cfg}")
    assert_bits_equal(gpu_conv_tail(ctx, x, w, (0, 0), bn=(mean, var, gamma, beta), act="leaky", alpha=0.1),
                      O.leaky_relu(bn, 0.1).reshape(plain.shape), f"1x1 conv+bn+leaky {cfg}")
    assert_bits_equal(gpu_conv_tail(ctx, x, w, (0, 0), act="relu"), O.relu(plain).reshape(plain.shape), f"1x1 conv+relu {cfg}")
    assert ctx.lib.gh_conv2d_can_pool(D.cmd_conv2d(1, 1, 1, B, C, H, W, F, 1, 1, (0, 0))) == 0


# shapes the wide-image kernel takes (3x3, at most 64 channels, enough pixels that patches alone fill the
# device; whole K per wavefront): channel counts that are not multiples of four, ragged filter tiles,
# partial patches on both axes, no padding, pooled extents odd and even
WIDE_CASES = [(2, 16, 130, 131, 32, 1), (4, 32, 104, 104, 64, 1), (3, 3, 120, 96, 16, 1), (8, 5, 64, 66, 32, 1),
              (2, 8, 129, 140, 5, 0), (1, 24, 181, 190, 40, 1), (1, 48, 190, 181, 21, 1), (3, 12, 150, 111, 70, 0),
              (1, 6, 200, 170, 33, 1),
              # three and four channels (one quad of planes, the last one padding for C = 3), taken from the direct kernel
              (2, 4, 140, 130, 20, 1), (1, 3, 260, 270, 16, 0)]


@pytest.mark.parametrize("cfg", WIDE_CASES)
def test_conv_wide_kernel(ctx, cfg):
    """The wide-image convolution kernel against the oracle (<= 1e-5, exact on integers), and every
    epilogue it can carry against the oracle's operators applied to its own plain result, bit for bit."""
    B, C, H, W, F, pad = cfg
    x = synth.uniform(51, (B, C, H, W), -1, 1)
    w = synth.he_normal(52, (F, C, 3, 3))
    plain = gpu_conv(ctx, x, w, (pad, pad), (1, 1), (1, 1))
    ref = O.conv2d_direct_f64(x, w, (pad, pad), (1, 1), (1, 1))
    err = rel_frobenius(plain, ref)
    assert err <= TOL, f"wide conv {cfg}: rel frobenius {err:.3e}"
    rng = np.random.default_rng(11)
    xi = rng.integers(-3, 4, (B, C, H, W)).astype(np.float32)
    wi = rng.integers(-3, 4, (F, C, 3, 3)).astype(np.float32)
    assert_bits_equal(gpu_conv(ctx, xi, wi, (pad, pad), (1, 1), (1, 1)), O.conv2d(xi, wi, (pad, pad), (1, 1), (1, 1)),
                      f"integer wide conv {cfg}")
    mean, var = synth.normal(53, (F,), 0.0, 0.1), synth.uniform(54, (F,), 0.5, 1.5)
    gamma, beta = synth.uniform(55, (F,), 0.5, 1.5), synth.normal(56, (F,), 0.0, 0.1)
    leaky = O.leaky_relu(O.bn_infer(plain, mean, var, 1e-5, gamma, beta), 0.1).reshape(plain.shape)
    assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), bn=(mean, var, gamma, beta), act="leaky", alpha=0.1), leaky,
                      f"wide conv+bn+leaky {cfg}")
    relu = O.relu(plain).reshape(plain.shape)
    assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), act="relu"), relu, f"wide conv+relu {cfg}")
    cmd = D.cmd_conv2d(1, 1, 1, B, C, H, W, F, 3, 3, (pad, pad))
    if ctx.lib.gh_conv2d_can_pool(cmd) == 1:
        assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), bn=(mean, var, gamma, beta), act="leaky", alpha=0.1,
                                        pool2=True),
                          O.maxpool2d(leaky, (2, 2), (0, 0), (2, 2)), f"wide conv+bn+leaky+pool {cfg}")
        assert_bits_equal(gpu_conv_tail(ctx, x, w, (pad, pad), act="relu", pool2=True),
                          O.maxpool2d(relu, (2, 2), (0, 0), (2, 2)), f"wide conv+relu+pool {cfg}")


def test_conv_random_geometry_sweep(ctx):
    """Seeded sweep over geometries nobody picked by hand - 3x3 / stride 1 on small and large images, 1x1 over
    many channels, and kernels, strides, dilations and paddings of every kind - whichever kernel each one
    reaches: the plain convolution against the oracle (as a norm, and value by value), BatchNorm and an
    activation in the epilogue against the separate commands bit for bit, and the pool on top wherever
    gh_conv2d_can_pool allows it."""
    routes, pooled, tails = set(), 0, 0
    for case in range(160):
        rng = np.random.default_rng(case)
        B = int(rng.integers(1, 9))
        C = int(rng.choice([1, 2, 3, 4, 7, 8, 16, 24, 32, 48, 64, 96, 128, 256]))
        large = rng.random() < 0.25 and C <= 64
        H, W = (int(rng.integers(20, 120)), int(rng.integers(20, 120))) if large else \
               (int(rng.integers(1, 34)), int(rng.integers(1, 34)))
        F = int(rng.choice([1, 3, 8, 15, 16, 17, 31, 32, 33, 48, 64, 65, 100, 128, 130, 256]))
        if case % 4 == 3:
            kh, kw = int(rng.choice([1, 2, 3, 5])), int(rng.choice([1, 2, 3, 4]))
            pad = (int(rng.integers(0, kh)), int(rng.integers(0, kw)))
            stride = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
            dil = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        elif case % 4 == 2 and C >= 64:
            kh = kw = 1; pad = (0, 0); stride = dil = (1, 1)
        else:
            kh = kw = 3; pad = (int(rng.integers(0, 2)),) * 2; stride = dil = (1, 1)
        oh, ow = O.conv_out_hw(H, W, kh, kw, pad, stride, dil)
        if oh < 1 or ow < 1 or B * C * H * W > 6_000_000 or B * F * oh * ow > 6_000_000:
            continue
        tag = f"case {case}: B{B} C{C} {H}x{W} F{F} k{kh}x{kw} pad{pad} stride{stride} dilation{dil}"
        x = synth.uniform(3000 + case, (B, C, H, W), -1, 1)
        w = synth.he_normal(4000 + case, (F, C, kh, kw))
        routes.add(ctx.lib.gh_conv2d_route(D.cmd_conv2d(1, 1, 1, B, C, H, W, F, kh, kw, pad, stride, dil)))
        got = gpu_conv(ctx, x, w, pad, stride, dil)
        ref = O.conv2d(x, w, pad, stride, dil)
        err = rel_frobenius(got, ref)
        assert err <= TOL, f"{tag}: {err:.3e}"
        assert np.abs(got.astype(np.float64) - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max()), f"{tag}: a value is off"
        if stride != (1, 1) or dil != (1, 1) or pad[0] != pad[1] or kh != kw:
            continue
        use_bn = rng.random() < 0.5
        act = [None, "relu", "leaky"][int(rng.integers(0, 3))]
        bn = None
        h = got
        if use_bn:
            bn = (synth.normal(13 + case, (F,), 0.0, 0.1), synth.uniform(14 + case, (F,), 0.5, 1.5),
                  synth.uniform(15 + case, (F,), 0.5, 1.5), synth.normal(16 + case, (F,), 0.0, 0.1))
            h = gpu_bn(ctx, h.copy(), bn[0], bn[1], bn[2], bn[3], 1e-5)
        if act == "relu":
            h = O.relu(h).reshape(h.shape)
        elif act == "leaky":
            h = O.leaky_relu(h, 0.1).reshape(h.shape)
        if use_bn or act:
            tails += 1
            assert_bits_equal(gpu_conv_tail(ctx, x, w, pad, bn=bn, act=act, alpha=0.1), h, f"{tag}: bn {use_bn}, {act}")
        if ctx.lib.gh_conv2d_can_pool(D.cmd_conv2d(1, 1, 1, B, C, H, W, F, kh, kw, pad, pool2=True)) == 1:
            pooled += 1
            assert_bits_equal(gpu_conv_tail(ctx, x, w, pad, bn=bn, act=act, alpha=0.1, pool2=True),
                              gpu_pool(ctx, h, (2, 2), (0, 0), (2, 2)), f"{tag}: bn {use_bn}, {act}, pool")
    assert pooled >= 40 and tails >= 40 and len(routes) >= 6, (pooled, tails, routes)


def test_conv_pointwise_random_geometries(ctx):
    """Seeded sweep over 1x1 convolutions with 256-1024 channels (the K-split 1x1 kernel, every filter-tile height,
    images of every size mod 4): against the float64 sum, exact on small integers, and conv+LeakyReLU against the
    oracle's LeakyReLU of the plain result bit for bit."""
    rng = np.random.default_rng(78)
    for case in range(14):
        B = int(rng.integers(1, 10))
        C = int(rng.choice([256, 512, 768, 1024]))
        H, W = int(rng.integers(1, 20)), int(rng.integers(2, 20))
        F = int(rng.integers(1, 200))
        x = synth.uniform(5000 + case, (B, C, H, W), -1, 1)
        w = synth.he_normal(6000 + case, (F, C, 1, 1))
        got = gpu_conv(ctx, x, w, (0, 0), (1, 1), (1, 1))
        ref = np.einsum("fc,bchw->bfhw", w[:, :, 0, 0].astype(np.float64), x.astype(np.float64))
        err = rel_frobenius(got, ref)
        assert err <= TOL, f"case {case}: B{B} C{C} {H}x{W} F{F}: {err:.3e}"
        xi = rng.integers(-3, 4, (B, C, H, W)).astype(np.float32)
        wi = rng.integers(-3, 4, (F, C, 1, 1)).astype(np.float32)
        want = np.einsum("fc,bchw->bfhw", wi[:, :, 0, 0].astype(np.float64), xi.astype(np.float64)).astype(np.float32)
        assert_bits_equal(gpu_conv(ctx, xi, wi, (0, 0), (1, 1), (1, 1)), want, f"case {case}: integer 1x1 conv")
        assert_bits_equal(gpu_conv_tail(ctx, x, w, (0, 0), act="leaky", alpha=0.1), O.leaky_relu(got, 0.1).reshape(got.shape),
                          f"case {case}: 1x1 conv+leaky")


def test_conv_pool_flag_needs_a_pooling_kernel(ctx):
    # 13 rows of 13: no block of at most 128 pixels holds a whole image
    cmd = D.cmd_conv2d(0x1000, 0x2000, 0x3000, 2, 8, 13, 13, 16, 3, 3, (1, 1), pool2=True)
    assert ctx.lib.gh_conv2d_can_pool(cmd) == 0
    import ctypes as C
    buf = C.create_string_buffer(256)
    assert ctx.lib.gh_validate(C.byref(cmd), 1, buf, 256) != 0
    assert b"pooling" in buf.value


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
