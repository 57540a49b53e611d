"""GPU parity of the float64 forward neural-network operators (Conv2d, MaxPool2D,
BatchNorm eval, Rectify, LeakyRelu, SoftMax) through the C ABI and the tape
machine against the CPU oracle's float64 twins.  Bars: bit-exact for everything
but SoftMax (same operation order, one rounding per step); SoftMax <= 4 float64
ulp: the exponentials come from two libraries (each within 1 ulp), and their
differences pass through the row sum and the quotient."""
import numpy as np
import pytest

from gorgonia_amd import _ffi
from gorgonia_amd import device as D
from gorgonia_amd import graph as G
from oracle import binding as O
from tests.util import assert_bits_equal

pytestmark = pytest.mark.gpu
F64 = _ffi.F64


def _rand(seed, shape, scale=1.0):
    return np.random.default_rng(seed).standard_normal(shape) * scale


def _ulp64(a, b):
    ia = a.view(np.int64).astype(np.int64)
    ib = b.view(np.int64).astype(np.int64)
    ia = np.where(ia < 0, np.int64(-2**63) - ia, ia)
    ib = np.where(ib < 0, np.int64(-2**63) - ib, ib)
    return np.abs(ia - ib)


CONV_CASES = [
    # B, C, H, W, F, kh, kw, pad, stride, dil
    (2, 3, 9, 8, 5, 3, 3, (1, 1), (1, 1), (1, 1)),
    (1, 8, 14, 14, 16, 3, 3, (1, 1), (1, 1), (1, 1)),
    (2, 4, 10, 11, 6, 1, 1, (0, 0), (1, 1), (1, 1)),
    (2, 2, 12, 9, 3, 5, 3, (2, 1), (2, 1), (1, 1)),
    (1, 3, 13, 13, 4, 3, 3, (2, 2), (1, 2), (2, 2)),
]


@pytest.mark.parametrize("cfg", CONV_CASES)
def test_conv2d_float64_bit_exact(ctx, cfg):
    B, C, H, W, F, kh, kw, pad, stride, dil = cfg
    x, w = _rand(1, (B, C, H, W)), _rand(2, (F, C, kh, kw), 0.3)
    want = O.conv2d(x, w, pad, stride, dil)
    dx, dw, dy = ctx.upload(x), ctx.upload(w), ctx.malloc(want.size * 8)
    ctx.run(D.cmd_conv2d(dx, dw, dy, B, C, H, W, F, kh, kw, pad, stride, dil, dtype=F64))
    got = ctx.d2h(dy, want.shape, np.float64)
    for p in (dx, dw, dy):
        ctx.free(p)
    assert_bits_equal(got, want, f"float64 conv {cfg}")
    ref = O.conv2d(x.astype(np.float32), w.astype(np.float32), pad, stride, dil)
    assert np.allclose(got, ref, rtol=1e-4, atol=1e-4)   # and it is the same convolution as the float32 one


CONV_MFMA_CASES = [
    # enough filters and pixels for the matrix-core kernel: each of its three tile shapes, odd and even
    # C*kh*kw, ragged edges in filters and pixels, stride / dilation / rectangular kernels
    (4, 1, 28, 28, 32, 3, 3, (1, 1), (1, 1), (1, 1)),      # 32-filter tiles, K = 9
    (3, 5, 17, 19, 24, 3, 3, (1, 1), (1, 1), (1, 1)),      # 32-filter tiles, ragged, K = 45
    (8, 32, 14, 14, 64, 3, 3, (1, 1), (1, 1), (1, 1)),     # 64x64 tiles
    (2, 7, 21, 20, 70, 5, 3, (2, 1), (2, 1), (1, 1)),      # 64x64 tiles, ragged, strided
    (2, 6, 23, 23, 40, 3, 3, (2, 2), (1, 2), (2, 2)),      # dilated
    (40, 8, 30, 30, 130, 3, 3, (1, 1), (1, 1), (1, 1)),    # 128x128 tiles, ragged filters
    (36, 16, 30, 31, 128, 1, 1, (0, 0), (1, 1), (1, 1)),   # 128x128 tiles, 1x1
]


@pytest.mark.parametrize("cfg", CONV_MFMA_CASES)
def test_conv2d_float64_matrix_cores(ctx, cfg):
    """The float64 implicit-GEMM kernel: the matrix cores sum each group of four products in
    their own order, so against the oracle's sequential float64 sum the bar is 1e-13 relative
    (far inside the 1e-5 of the float32 path), and equality on small-integer data, where
    every partial sum is exact."""
    B, C, H, W, F, kh, kw, pad, stride, dil = cfg
    rng = np.random.default_rng(5)
    for integer in (False, True):
        x = rng.integers(-4, 5, (B, C, H, W)).astype(np.float64) if integer else rng.standard_normal((B, C, H, W))
        w = rng.integers(-4, 5, (F, C, kh, kw)).astype(np.float64) if integer else rng.standard_normal((F, C, kh, kw)) * 0.3
        want = O.conv2d(x, w, pad, stride, dil)
        dx, dw, dy = ctx.upload(x), ctx.upload(w), ctx.malloc(want.size * 8)
        ctx.run(D.cmd_conv2d(dx, dw, dy, B, C, H, W, F, kh, kw, pad, stride, dil, dtype=F64))
        got = ctx.d2h(dy, want.shape, np.float64)
        for p in (dx, dw, dy):
            ctx.free(p)
        if integer:
            assert np.array_equal(got, want), f"integer float64 conv {cfg}"
        else:
            assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 1e-13, f"float64 conv {cfg}"


@pytest.mark.parametrize("cfg", [(2, 3, 8, 10, (2, 2), (0, 0), (2, 2)), (1, 2, 7, 8, (3, 2), (1, 1), (1, 2)),
                                 (2, 4, 13, 13, (2, 2), (1, 0, 1, 0), (1, 1)), (2, 3, 9, 11, (2, 2), (0, 0), (2, 2))])
def test_maxpool_float64_bit_exact(ctx, cfg):
    B, C, H, W, kernel, pad, stride = cfg
    x = _rand(3, (B, C, H, W))
    x.reshape(-1)[::7] = 0.0
    x.reshape(-1)[3::11] = -0.0
    want = O.maxpool2d(x, kernel, pad, stride)
    dx, dy = ctx.upload(x), ctx.malloc(want.size * 8)
    ctx.run(D.cmd_maxpool2d(dx, dy, B, C, H, W, kernel[0], kernel[1], pad, stride, dtype=F64))
    got = ctx.d2h(dy, want.shape, np.float64)
    ctx.free(dx); ctx.free(dy)
    assert_bits_equal(got, want, f"float64 maxpool {cfg}")
    # the same pool reading its input through Rectify: the bits of the two operators, the activation never stored
    xs = x.copy()
    xs.reshape(-1)[5::13] = np.inf; xs.reshape(-1)[9::17] = -np.inf; xs.reshape(-1)[1::19] = np.nan
    want = O.maxpool2d(O.relu(xs).reshape(xs.shape), kernel, pad, stride)
    dx, dy = ctx.upload(xs), ctx.malloc(want.size * 8)
    cmd = D.cmd_maxpool2d(dx, dy, B, C, H, W, kernel[0], kernel[1], pad, stride, dtype=F64)
    cmd.flags |= _ffi.FLAG_ACT_RELU
    ctx.run(cmd)
    got = ctx.d2h(dy, want.shape, np.float64)
    ctx.free(dx); ctx.free(dy)
    assert_bits_equal(got, want, f"float64 rectify+maxpool {cfg}")


@pytest.mark.parametrize("shape", [(4, 6), (2, 5, 7, 3)])
@pytest.mark.parametrize("affine", [False, True])
def test_batchnorm_float64_bit_exact(ctx, shape, affine):
    x = _rand(4, shape)
    Cn = shape[1]
    mean, var = _rand(5, (Cn,)), np.random.default_rng(6).uniform(0.5, 2.0, Cn)
    g, b = (_rand(7, (Cn,)), _rand(8, (Cn,))) if affine else (None, None)
    want = O.bn_infer(x, mean, var, 1e-5, g, b)
    held = [ctx.upload(a) for a in (x, mean, var)] + ([ctx.upload(g), ctx.upload(b)] if affine else [0, 0])
    dy = ctx.malloc(x.size * 8)
    B = shape[0]
    ctx.run(D.cmd_bn_infer(held[0], dy, held[1], held[2], B, Cn, x.size // (B * Cn), 1e-5, held[3], held[4], dtype=F64))
    got = ctx.d2h(dy, shape, np.float64)
    for p in held + [dy]:
        if p:
            ctx.free(p)
    assert_bits_equal(got, want, "float64 batchnorm")


def test_activations_float64_bit_exact(ctx):
    x = _rand(9, (100_003,))
    x[:6] = [0.0, -0.0, np.inf, -np.inf, np.nan, 1e-320]
    dx, dy = ctx.upload(x), ctx.malloc(x.size * 8)
    ctx.run(D.cmd_relu(dx, dy, x.size, dtype=F64))
    assert_bits_equal(ctx.d2h(dy, x.shape, np.float64), O.relu(x), "float64 relu")
    ctx.run(D.cmd_leaky_relu(dx, dy, x.size, 0.1, dtype=F64))   # 0.1 is not a float32: the full double must arrive
    assert_bits_equal(ctx.d2h(dy, x.shape, np.float64), O.leaky_relu(x, 0.1), "float64 leaky relu")
    ctx.free(dx); ctx.free(dy)


@pytest.mark.parametrize("shape", [(1, 1), (7, 10), (128, 10), (5, 64), (3, 65), (4, 1000)])
def test_softmax_float64(ctx, shape):
    x = _rand(10, shape, 3.0)
    dx, dy = ctx.upload(x), ctx.malloc(x.size * 8)
    ctx.run(D.cmd_softmax(dx, dy, shape[0], shape[1], dtype=F64))
    got = ctx.d2h(dy, shape, np.float64)
    ctx.free(dx); ctx.free(dy)
    assert _ulp64(got, O.softmax(x)).max() <= 4
    assert np.allclose(got.sum(axis=1), 1.0, atol=1e-14)


def test_float64_commands_validate(ctx):
    import ctypes as C
    buf = C.create_string_buffer(256)
    bad = D.cmd_conv2d(1, 2, 3, 1, 8, 8, 8, 8, 3, 3, (1, 1), act="relu", dtype=F64)
    assert ctx.lib.gh_validate(C.byref(bad), 1, buf, 256) != 0 and b"float64" in buf.value
    assert ctx.lib.gh_conv2d_can_pool(D.cmd_conv2d(1, 2, 3, 2, 8, 14, 14, 16, 3, 3, (1, 1), dtype=F64)) == 0
    bwd = D.cmd_conv2d_bwd_data(1, 2, 3, 1, 8, 8, 8, 8, 3, 3, (1, 1), dtype=F64)
    assert ctx.lib.gh_validate(C.byref(bwd), 1, buf, 256) == 0   # the gradients have float64 twins


def test_tape_float64_network(ctx):
    """conv -> batchnorm -> leakyrelu -> maxpool -> reshape -> matmul -> softmax in float64 on the
    tape machine, with activation folding requested (it must leave float64 nodes alone)."""
    x, w = _rand(11, (2, 3, 8, 8)), _rand(12, (4, 3, 3, 3), 0.3)
    mean, var = _rand(13, (4,)), np.random.default_rng(14).uniform(0.5, 2.0, 4)
    gam, bet = _rand(15, (4,)), _rand(16, (4,))
    w2 = _rand(17, (64, 5), 0.2)
    g = G.NewGraph()
    xn, wn = G.NewTensor(g, x), G.NewTensor(g, w)
    h = G.Conv2d(xn, wn, (3, 3), (1, 1), (1, 1), (1, 1))
    h = G.BatchNorm(h, G.NewTensor(g, gam), G.NewTensor(g, bet), G.NewTensor(g, mean), G.NewTensor(g, var), 1e-5)
    h = G.MaxPool2D(G.LeakyRelu(h, 0.1), (2, 2), (0, 0), (2, 2))
    out = G.Read(G.SoftMax(G.Mul(G.Reshape(h, (2, 64)), G.NewTensor(g, w2))), np.float64)
    m = G.NewTapeMachine(g, fuse_activations=True)
    assert m.fused == 0
    m.RunAll()
    ref = O.conv2d(x, w, (1, 1), (1, 1), (1, 1))
    ref = O.maxpool2d(O.leaky_relu(O.bn_infer(ref, mean, var, 1e-5, gam, bet), 0.1).reshape(ref.shape), (2, 2), (0, 0), (2, 2))
    want = O.softmax(ref.reshape(2, 64) @ w2)
    assert np.allclose(out, want, rtol=1e-12, atol=1e-15)
    m.Close()


def test_tape_float64_convnet_folds_rectify_into_pool(ctx):
    """The convnet in float64 (the reference example's default dtype, examples/convnet/main.go:28): the
    convolutions have no epilogue there, so FuseActivations lets each pool read through the Rectify in front
    of it; the output keeps the bits of the unfolded machine."""
    from gorgonia_amd import configs
    inp = {k: v.astype(np.float64) for k, v in configs.convnet_inputs(8).items()}
    outs = []
    for fuse in (False, True):
        g, o = configs.build_convnet(inp)
        m = G.NewTapeMachine(g, fuse_activations=fuse)
        if fuse:
            assert m.fused == 3 and m.program().count("rectify+maxpool2d") == 3, m.program()
        m.RunAll()
        outs.append(o["out"].copy())
        m.Close()
    assert outs[0].dtype == np.float64
    assert_bits_equal(outs[1], outs[0], "float64 convnet, Rectify folded into the pools")


def test_conv2d_float64_seeded_geometry_sweep(ctx):
    """Forward, image gradient and filter gradient in float64 over seeded geometries large
    enough for the matrix-core kernels (kernel 1..5, stride 1..2, dilation 1..2, any padding
    that keeps the output non-empty), integer data: all three must be exact."""
    rng = np.random.default_rng(31)
    done = 0
    while done < 12:
        B, C, F = int(rng.integers(2, 7)), int(rng.integers(1, 40)), int(rng.integers(16, 90))
        H, W = int(rng.integers(9, 26)), int(rng.integers(9, 26))
        kh, kw = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        stride = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        dil = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        pad = (int(rng.integers(0, dil[0] * (kh - 1) + 1)), int(rng.integers(0, dil[1] * (kw - 1) + 1)))
        if dil[0] * (kh - 1) + 1 > H + 2 * pad[0] or dil[1] * (kw - 1) + 1 > W + 2 * pad[1]:
            continue
        x = rng.integers(-3, 4, (B, C, H, W)).astype(np.float64)
        w = rng.integers(-3, 4, (F, C, kh, kw)).astype(np.float64)
        want = O.conv2d(x, w, pad, stride, dil)
        dyv = rng.integers(-3, 4, want.shape).astype(np.float64)
        dx_ref, dw_ref = O.conv2d_bwd(x, w, dyv, pad, stride, dil)
        px, pw, pdy = ctx.upload(x), ctx.upload(w), ctx.upload(dyv)
        py, pdx, pdw = ctx.malloc(want.size * 8), ctx.malloc(x.size * 8), ctx.malloc(w.size * 8)
        ctx.run([D.cmd_conv2d(px, pw, py, B, C, H, W, F, kh, kw, pad, stride, dil, dtype=F64),
                 D.cmd_conv2d_bwd_data(pdy, pw, pdx, B, C, H, W, F, kh, kw, pad, stride, dil, dtype=F64),
                 D.cmd_conv2d_bwd_filter(px, pdy, pdw, B, C, H, W, F, kh, kw, pad, stride, dil, dtype=F64)])
        got = ctx.d2h(py, want.shape, np.float64)
        dx, dw = ctx.d2h(pdx, x.shape, np.float64), ctx.d2h(pdw, w.shape, np.float64)
        for p in (px, pw, pdy, py, pdx, pdw):
            ctx.free(p)
        tag = f"B{B} C{C} F{F} {H}x{W} k{kh}x{kw} pad{pad} stride{stride} dil{dil}"
        assert np.array_equal(got, want), "forward " + tag
        assert np.array_equal(dx, dx_ref), "image gradient " + tag
        assert np.array_equal(dw, dw_ref), "filter gradient " + tag
        done += 1
