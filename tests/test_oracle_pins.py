"""Pins the CPU oracle (oracle/oracle.c) before anything is compared to it:
the reference's own golden vectors (tests/golden/*.json, extracted as data from
the Go test files), closed forms, and brute force on small inputs.  No GPU."""
import json
import os

import numpy as np
import pytest

from oracle import binding as O
from tests.util import ulp_diff

G = os.path.join(os.path.dirname(__file__), "golden")


def load(name):
    with open(os.path.join(G, name)) as f:
        return json.load(f)


# ---- elementwise ---------------------------------------------------------------

GO_OP = {"Add": "add", "Sub": "sub", "Mul": "mul", "HadamardProd": "mul", "Div": "div",
         "HadamardDiv": "div"}


def test_binop_table():
    """op_math_test.go:23-360 binOpTests (the table op_math_cuda_test.go:44-99
    replays on the GPU engine): vv / vs / sv / ss forms, f64 and f32."""
    for i, c in enumerate(load("binop.json")["cases"]):
        dt = np.float32 if c["a"]["bits"] == 32 else np.float64
        a = np.array(c["a"]["v"], dtype=dt)
        b = np.array(c["b"]["v"], dtype=dt)
        want = np.array(c["correct"]["v"], dtype=dt)
        sa, sb = c["a"]["scalar"], c["b"]["scalar"]
        if c["op"] == "Mul" and not (sa or sb):
            continue  # Mul on two tensors is a matrix/vector product, pinned in the linalg tests
        if a.size != b.size and not (sa or sb):
            continue  # broadcast rows of the table (pinned by the broadcast tests)
        mode = "ss" if sa and sb else "sv" if sa else "vs" if sb else "vv"
        got = O.binop(GO_OP[c["op"]], mode, a, b)
        assert np.array_equal(got, want), f"case {i} {c['op']} {mode}: {got} vs {want}"


def test_gt_table():
    """operations_test.go:158-233 gtTests, the same-dtype (retSame) rows."""
    assert O.binop("gt", "ss", np.array([1.0]), np.array([0.0]))[0] == 1.0
    assert O.binop("gt", "ss", np.array([0.0]), np.array([1.0]))[0] == 0.0
    assert np.array_equal(O.binop("gt", "sv", np.array([1.0]), np.array([0.0, 2.0])), [1.0, 0.0])
    assert np.array_equal(O.binop("gt", "vs", np.array([0.0, 2.0]), np.array([1.0])), [0.0, 1.0])
    a = np.arange(6, dtype=np.float64)
    assert np.array_equal(O.binop("gt", "vv", a, a[::-1].copy()), [0, 0, 0, 1, 1, 1])
    a32 = np.array([0, 2], dtype=np.float32)
    assert np.array_equal(O.binop("gt", "vs", a32, np.array([1], np.float32)), np.array([0, 1], np.float32))


def test_cmp_and_arith_against_numpy_ieee():
    rng = np.random.default_rng(1)
    a = rng.standard_normal(10001).astype(np.float32)
    b = rng.standard_normal(10001).astype(np.float32)
    a[:6] = [0.0, -0.0, np.inf, -np.inf, np.nan, 1e-42]
    b[:6] = [-0.0, 0.0, np.inf, np.inf, 1.0, 0.5]
    with np.errstate(all="ignore"):
        ref = {"add": a + b, "sub": a - b, "mul": a * b, "div": a / b,
               "lt": (a < b), "lte": (a <= b), "gt": (a > b), "gte": (a >= b), "eq": (a == b),
               "ne": (a != b)}
    for fn, want in ref.items():
        got = O.binop(fn, "vv", a, b)
        want = want.astype(np.float32)
        same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
        assert same.all(), fn


def test_cube_table():
    """op_math_cuda_test.go:16-42 TestCUDACube: cube of Range(0..32)."""
    x = np.arange(32, dtype=np.float32)
    assert np.array_equal(O.unary("cube", x), x * x * x)
    assert np.array_equal(O.unary("cube", x.astype(np.float64)), (x.astype(np.float64)) ** 3)


def test_sigmoid_closed_form():
    """math_nooptim.go:36-44: cut-offs at -88 and 15, float64 exp, one rounding."""
    x = np.array([-89, -88.0001, -88, -1, 0, 1, 15, 15.0001, 16], dtype=np.float32)
    s = O.unary("sigmoid", x)
    assert s[0] == 0 and s[1] == 0 and s[2] > 0 and s[4] == 0.5 and s[6] < 1 and s[7] == 1 and s[8] == 1
    xs = np.linspace(-30, 14, 20001).astype(np.float32)
    want = (1.0 / (1.0 + np.exp(-xs.astype(np.float64)))).astype(np.float32)
    assert ulp_diff(O.unary("sigmoid", xs), want).max() == 0
    # symmetry s(x) + s(-x) = 1 up to one rounding of each term
    xs = xs[np.abs(xs) <= 14]  # beyond 15 the cut-off returns exactly 1
    s1, s2 = O.unary("sigmoid", xs), O.unary("sigmoid", -xs)
    assert np.max(np.abs(s1.astype(np.float64) + s2 - 1.0)) <= 2 ** -23


def test_tanh_exp_against_identities():
    """tanh/exp are unpinned bit-for-bit (math32 is not vendored); these check
    the float64-rounded-once form the oracle states: odd symmetry, tanh(0)=0,
    exp(0)=1, exp(x)*exp(-x)=1 and agreement with numpy's float64 libm."""
    x = np.linspace(-12, 12, 24001).astype(np.float32)
    t = O.unary("tanh", x)
    assert np.array_equal(t, -O.unary("tanh", -x))
    assert ulp_diff(t, np.tanh(x.astype(np.float64)).astype(np.float32)).max() <= 1
    e = O.unary("exp", x)
    assert ulp_diff(e, np.exp(x.astype(np.float64)).astype(np.float32)).max() <= 1
    assert np.max(np.abs(e.astype(np.float64) * O.unary("exp", -x) - 1.0)) < 3e-7
    assert O.unary("exp", np.zeros(1, np.float32))[0] == 1.0
    assert O.unary("tanh", np.zeros(1, np.float32))[0] == 0.0


def test_pow_two_is_square():
    x = np.random.default_rng(2).standard_normal(5000).astype(np.float32)
    assert np.array_equal(O.binop("pow", "vs", x, np.array([2.0], np.float32)), x * x)


def test_leaky_relu_golden():
    g = load("leaky_relu.json")
    x = np.array(g["x"], dtype=np.float32)
    y = O.leaky_relu(x, g["alpha"])
    assert np.max(np.abs(y - np.array(g["y"], dtype=np.float32))) <= g["tolerance"]
    # composed form: +-Inf -> NaN (Inf * 0), negative -> alpha*x, relu of negatives is -0.0
    sp = O.leaky_relu(np.array([np.inf, -np.inf, -2.0, 3.0], np.float32), 0.1)
    assert np.isnan(sp[0]) and np.isnan(sp[1]) and sp[2] == np.float32(-2.0) * np.float32(0.1) and sp[3] == 3.0
    r = O.relu(np.array([-1.0, 0.0, 2.0], np.float32))
    assert np.signbit(r[0]) and r[0] == 0 and r[2] == 2


def test_broadcast_matches_repeat_then_op():
    """operations_broadcast_test.go:167-293 pattern: (2,3)+(2,1)/(1,3) style
    broadcasts equal numpy broadcasting of the same IEEE op."""
    big = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    small = np.array([10, 20, 30], dtype=np.float32)
    got = O.bcast_binop("add", big.reshape(-1), small, 2, 3, 4).reshape(2, 3, 4)
    assert np.array_equal(got, big + small[None, :, None])
    got = O.bcast_binop("sub", big.reshape(-1), small, 2, 3, 4, small_left=True).reshape(2, 3, 4)
    assert np.array_equal(got, small[None, :, None] - big)
    row = np.array([1, 2, 3, 4], dtype=np.float32)
    got = O.bcast_binop("mul", big.reshape(-1), row, 6, 4, 1).reshape(6, 4)
    assert np.array_equal(got, big.reshape(6, 4) * row[None, :])


# ---- max pool --------------------------------------------------------------------

def test_maxpool_asymmetric_golden():
    """nn_test.go:91-138: 2x2 stride 1 pad [1,0,1,0] on (1,3,32,32) - the
    darknet "stride-1 pool" of the Tiny-YOLO configuration. Exact equality."""
    g = load("maxpool_asym.json")
    x = np.array(g["x"], dtype=np.float32).reshape(g["shape"])
    y = O.maxpool2d(x, g["kernel"], g["pad"], g["stride"])
    assert list(y.shape) == g["shape"]
    assert np.array_equal(y.reshape(-1), np.array(g["y"], dtype=np.float32))


def test_maxpool_small_cases():
    """nn_test.go:195-266 TestMaxPool example 1 and brute force windows."""
    x = np.arange(16, dtype=np.float32).reshape(1, 1, 4, 4)
    assert O.maxpool2d(x, (4, 4), (0, 0), (1, 1)).reshape(-1).tolist() == [15.0]
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 3, 9, 11)).astype(np.float32)
    for k, p, s in [((2, 2), (0, 0), (2, 2)), ((3, 3), (1, 1), (1, 1)), ((3, 2), (1, 0), (2, 1))]:
        y = O.maxpool2d(x, k, p, s)
        xp = np.full((2, 3, 9 + 2 * p[0], 11 + 2 * p[1]), -np.inf, np.float32)
        xp[:, :, p[0]:p[0] + 9, p[1]:p[1] + 11] = x
        oh = (9 + 2 * p[0] - k[0]) // s[0] + 1
        ow = (11 + 2 * p[1] - k[1]) // s[1] + 1
        assert y.shape == (2, 3, oh, ow)
        for i in range(oh):
            for j in range(ow):
                win = xp[:, :, i * s[0]:i * s[0] + k[0], j * s[1]:j * s[1] + k[1]]
                assert np.array_equal(y[:, :, i, j], win.max(axis=(2, 3)))


# ---- conv ---------------------------------------------------------------------------

def test_conv_goldens():
    for g in load("conv.json"):
        x = np.array(g["x"], dtype=np.float32).reshape(g["x_shape"])
        w = np.array(g["w"], dtype=np.float32).reshape(g["w_shape"])
        y = O.conv2d(x, w, g["pad"], g["stride"], g["dilation"])
        assert list(y.shape) == g["y_shape"], g["source"]
        assert np.array_equal(y.reshape(-1), np.array(g["y"], dtype=np.float32)), g["source"]


@pytest.mark.parametrize("cfg", [
    (2, 3, 8, 9, 5, 3, 3, (1, 1), (1, 1), (1, 1)),
    (1, 4, 7, 7, 6, 1, 1, (0, 0), (1, 1), (1, 1)),
    (2, 2, 10, 11, 3, 3, 2, (2, 1), (2, 3), (1, 1)),
    (1, 3, 12, 12, 4, 3, 3, (2, 2), (1, 1), (2, 2)),
    (3, 1, 28, 28, 8, 3, 3, (1, 1), (1, 1), (1, 1)),
])
def test_conv_im2col_path_equals_direct_definition(cfg):
    """The im2col+GEMM+transpose restatement against a brute-force float64
    cross-correlation: a wrong index, a transposed operand or a dropped pad
    would fail here."""
    B, C, H, W, F, kh, kw, pad, stride, dil = cfg
    rng = np.random.default_rng(4)
    x = rng.standard_normal((B, C, H, W)).astype(np.float32)
    w = rng.standard_normal((F, C, kh, kw)).astype(np.float32)
    y = O.conv2d(x, w, pad, stride, dil)
    ref = O.conv2d_direct_f64(x, w, pad, stride, dil)
    assert y.shape == ref.shape
    assert np.linalg.norm(y - ref) / np.linalg.norm(ref) < 1e-6
    # integer data: exact
    xi = rng.integers(-4, 5, (B, C, H, W)).astype(np.float32)
    wi = rng.integers(-4, 5, (F, C, kh, kw)).astype(np.float32)
    assert np.array_equal(O.conv2d(xi, wi, pad, stride, dil), O.conv2d_direct_f64(xi, wi, pad, stride, dil))


# ---- linalg ---------------------------------------------------------------------------

def test_gemm_against_numpy_float64():
    rng = np.random.default_rng(5)
    for (m, k, n) in [(1, 1, 1), (7, 5, 3), (64, 100, 33)]:
        A = rng.standard_normal((m, k)).astype(np.float32)
        B = rng.standard_normal((k, n)).astype(np.float32)
        ref = A.astype(np.float64) @ B.astype(np.float64)
        for ta, tb in [(0, 0), (0, 1), (1, 0), (1, 1)]:
            As = A.T.copy() if ta else A
            Bs = B.T.copy() if tb else B
            assert np.allclose(O.gemm_f64acc(As, Bs, ta, tb), ref, rtol=1e-12, atol=1e-12)
            got = O.gemm(As, Bs, ta, tb)
            assert np.linalg.norm(got - ref) / np.linalg.norm(ref) < 1e-6
    Ai = rng.integers(-9, 10, (20, 30)).astype(np.float32)
    Bi = rng.integers(-9, 10, (30, 10)).astype(np.float32)
    assert np.array_equal(O.gemm(Ai, Bi), Ai @ Bi)


def test_mul_table():
    """operations_test.go:43-54 mulTests: matrix x vector and vector x vector on
    Range inputs (forward values)."""
    A = np.arange(6, dtype=np.float32).reshape(2, 3)
    v = np.arange(3, dtype=np.float32)
    assert np.array_equal(O.gemv(A, v), [5, 14])
    assert np.array_equal(O.gemv(A, np.arange(2, dtype=np.float32), trans=True), [3, 4, 5])
    assert np.array_equal(O.outer(v, v), np.outer(v, v))
    a = np.arange(12, dtype=np.float32).reshape(2, 3, 2)
    b = np.arange(12, dtype=np.float32).reshape(2, 2, 3)
    assert np.array_equal(O.bmm(a, b), np.matmul(a, b))  # example_linalg_test.go:11-92


# ---- softmax ----------------------------------------------------------------------------

def test_softmax_goldens():
    for c in load("softmax_do.json")["cases"]:
        x = np.array(c["input"], dtype=np.float64).reshape(c["shape"])
        want = np.array(c["expected"], dtype=np.float64).reshape(c["shape"])
        assert np.allclose(O.softmax(x), want, rtol=1e-12, atol=1e-15)
        got32 = O.softmax(x.astype(np.float32))
        assert np.allclose(got32, want, rtol=1e-5, atol=1e-7)  # op_softmax_test.go:110-137 tolerance


# ---- batch norm ----------------------------------------------------------------------------

def _ranged(start, step, n):
    out = np.empty(n, dtype=np.float32)
    st, inc = np.float32(start), np.float32(step)
    for i in range(n):
        out[i] = st
        st = np.float32(st + inc)
    return out


def _init(spec, n):
    if spec.startswith("RangedFromWithStep"):
        a, b = spec[spec.index("(") + 1:spec.index(")")].split(",")
        return _ranged(float(a), float(b), n)
    if spec.startswith("Ones"):
        return np.ones(n, np.float32)
    if spec.startswith("Zeroes"):
        return np.zeros(n, np.float32)
    raise ValueError(spec)


@pytest.mark.parametrize("idx", range(6))
def test_batchnorm_goldens(idx):
    """nn_amd64_test.go bnAllCases through the test body of nn_test.go:319-440:
    one training-mode run from running stats (0, 1) with momentum 0.9, eps 1e-5,
    y = gamma*BN(x) + beta, then y . fcWeight^T.  Checks the running statistics,
    the training output, and the eval-mode output (after the reference's one Adam
    step on scale/bias/fcWeight, whose update is lr*g/(|g|+eps) on the first step)."""
    c = load("batchnorm.json")["cases"][idx]
    shp = c["x_shape"]
    n = int(np.prod(shp))
    x = (_ranged(*c["x_ranged"], n) if "x_ranged" in c else np.array(c["x"], np.float32)).reshape(shp)
    B, Cn = shp[0], shp[1]
    feat = n // B
    gamma = _init(c["scale_init"], Cn)
    beta = _init(c["bias_init"], Cn)
    fcw = _init(c["scale_init"], B * feat).reshape(B, feat)

    y, rm, rv = O.bn_train(x, np.zeros(Cn, np.float32), np.ones(Cn, np.float32), 0.9, 1e-5)
    assert np.allclose(rm, c["expected_mean"], rtol=1e-5, atol=1e-6)
    assert np.allclose(rv, c["expected_variance"], rtol=1e-5, atol=1e-6)

    S = feat // Cn
    def affine(t, g, b):
        t3 = t.reshape(B, Cn, S)
        return (g[None, :, None] * t3 + b[None, :, None]).astype(np.float32).reshape(B, feat)

    out = affine(y, gamma, beta) @ fcw.T
    assert np.allclose(out.reshape(-1), c["expected_train_result"], rtol=2e-4, atol=2e-5)

    # one Adam step (first step: update = lr * g / (|g| + eps), lr 0.02, eps 1e-8)
    def adam(p, g):
        g = np.asarray(g, np.float64)
        return (p - 0.02 * g / (np.abs(g) + 1e-8)).astype(np.float32)

    yfull = affine(y, gamma, beta)
    g_fcw = np.tile(yfull.sum(axis=0, dtype=np.float64) / (B * B), (B, 1))
    if np.min(np.abs(g_fcw)) < 1e-6 or min(map(abs, c["expected_scale_grad"])) < 1e-6:
        # gradients at rounding-noise level make the Adam step (and with it the
        # reference's eval golden) depend on summation order: eval is then pinned
        # by the closed form below only
        ye = O.bn_infer(x, rm, rv, 1e-5, gamma, beta)
        a = 1.0 / np.sqrt(rv.astype(np.float64) + 1e-5)
        ref = (x.reshape(B, Cn, S).astype(np.float64) - rm[None, :, None]) * a[None, :, None]
        ref = ref * gamma[None, :, None] + beta[None, :, None]
        assert np.allclose(ye.reshape(B, Cn, S), ref, rtol=1e-5, atol=1e-5)
        return
    gamma2 = adam(gamma, c["expected_scale_grad"])
    beta2 = adam(beta, c["expected_bias_grad"])
    fcw2 = adam(fcw, g_fcw)
    ye = O.bn_infer(x, rm, rv, 1e-5, gamma2, beta2).reshape(B, feat)
    oute = ye @ fcw2.T
    assert np.allclose(oute.reshape(-1), c["expected_eval_result"], rtol=2e-4, atol=2e-5)


def test_has_nan_inf():
    a = np.zeros(100, np.float32)
    assert not O.has_nan(a) and not O.has_inf(a)
    a[7] = np.nan
    assert O.has_nan(a) and not O.has_inf(a)
    a[7] = -np.inf
    assert O.has_inf(a) and not O.has_nan(a)


def test_mod_is_go_math_mod():
    """math.Mod's documented special cases (Go standard library, math/mod.go: Mod(±Inf, y) = NaN,
    Mod(NaN, y) = NaN, Mod(x, 0) = NaN, Mod(x, ±Inf) = x, Mod(x, NaN) = NaN; the result takes
    the sign of x) and exactness: x - trunc(x/y)*y evaluated in integers."""
    from oracle import binding as O
    f = np.float32
    a = np.array([7.5, -7.5, 7.5, -7.5, 5.0, np.inf, -np.inf, np.nan, 3.0, 3.0, -3.0, 3.0, 0.0, -0.0], f)
    b = np.array([2.0, 2.0, -2.0, -2.0, 0.0, 2.0, 2.0, 2.0, np.inf, -np.inf, np.inf, np.nan, 3.0, 3.0], f)
    got = O.binop("mod", "vv", a, b)
    want = np.array([1.5, -1.5, 1.5, -1.5, np.nan, np.nan, np.nan, np.nan, 3.0, 3.0, -3.0, np.nan, 0.0, -0.0], f)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
    # exact remainders on integers scaled by powers of two
    rng = np.random.default_rng(5)
    x = rng.integers(-10**6, 10**6, 5000)
    y = rng.integers(1, 5000, 5000) * rng.choice([-1, 1], 5000)
    for dt, scale in ((np.float32, 0.25), (np.float64, 2.0 ** -20)):
        r = O.binop("mod", "vv", (x * scale).astype(dt), (y * scale).astype(dt))
        exact = np.sign(x) * (np.abs(x) % np.abs(y)) * scale
        assert np.array_equal(r, exact.astype(dt))


# ---- float64 twins of the forward neural-network operators -----------------------------

def test_float64_nn_twins_equal_the_pinned_float32_functions_where_both_are_exact():
    """Data on which float32 and float64 arithmetic are both exact (small integers, powers of
    two): the float64 twins must reproduce the float32 functions pinned above."""
    from oracle import binding as O
    rng = np.random.default_rng(11)
    x = rng.integers(-6, 7, (3, 4, 9, 8)).astype(np.float64)
    w = rng.integers(-3, 4, (5, 4, 3, 3)).astype(np.float64)
    f32 = lambda a: a.astype(np.float32)
    for pad, stride, dil in [((1, 1), (1, 1), (1, 1)), ((0, 2), (2, 1), (1, 1)), ((2, 2), (1, 2), (2, 1))]:
        a = O.conv2d(x, w, pad, stride, dil)
        assert a.dtype == np.float64 and np.array_equal(a, O.conv2d(f32(x), f32(w), pad, stride, dil))
    for kernel, pad, stride in [((2, 2), (0, 0), (2, 2)), ((3, 2), (1, 1), (1, 2)), ((2, 2), (1, 0, 1, 0), (1, 1))]:
        a = O.maxpool2d(x, kernel, pad, stride)
        assert a.dtype == np.float64 and np.array_equal(a, O.maxpool2d(f32(x), kernel, pad, stride))
    assert np.array_equal(O.relu(x), O.relu(f32(x))) and np.array_equal(O.leaky_relu(x, 0.25), O.leaky_relu(f32(x), 0.25))
    mean, var = np.array([1.0, -2.0, 0.5, 4.0]), np.array([3.0, 15.0, 0.0, 63.0])   # var + 1 is a square
    g, b = np.array([2.0, -1.0, 0.5, 4.0]), np.array([1.0, 0.0, -3.0, 8.0])
    assert np.array_equal(O.bn_infer(x, mean, var, 1.0, g, b), O.bn_infer(f32(x), mean, var, 1.0, g, b))


def test_float64_nn_twins_against_their_definitions():
    """General float64 data against independent numpy restatements: the documented per-step
    roundings of batch norm and the activations, a sequential-order sum for the convolution."""
    from oracle import binding as O
    rng = np.random.default_rng(12)
    x = rng.standard_normal((2, 3, 6, 5))
    w = rng.standard_normal((4, 3, 3, 3))
    got = O.conv2d(x, w, (1, 1), (1, 1), (1, 1))
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
    want = np.zeros_like(got)
    for c in range(3):
        for kr in range(3):
            for kc in range(3):   # k ascending, one rounded product and one rounded add per tap
                want = want + xp[:, None, c, kr:kr + 6, kc:kc + 5] * w[None, :, c, kr, kc, None, None]
    assert np.array_equal(got, want)
    mean, var, g, b = rng.standard_normal(3), rng.uniform(0.5, 2, 3), rng.standard_normal(3), rng.standard_normal(3)
    a = 1.0 / np.sqrt(var + 1e-5)
    sh = (1, 3, 1, 1)
    want = g.reshape(sh) * ((x * a.reshape(sh)) + (-mean * a).reshape(sh)) + b.reshape(sh)
    assert np.array_equal(O.bn_infer(x, mean, var, 1e-5, g, b), want)
    assert np.array_equal(O.relu(x), x * (x >= 0))
    assert np.array_equal(O.leaky_relu(x, 0.1), x * (x >= 0) + (x * (x < 0)) * 0.1)
    pooled = O.maxpool2d(x, (2, 2), (0, 0), (2, 2))
    assert np.array_equal(pooled, x[:, :, :6, :4].reshape(2, 3, 3, 2, 2, 2).max(axis=(3, 5)))
