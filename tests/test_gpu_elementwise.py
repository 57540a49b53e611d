"""GPU parity: elementwise binary / unary / broadcast / relu kernels against the
CPU oracle on the same seeded inputs, called through the C ABI (gh_submit).

Bars: add/sub/mul/div/compare/relu/leaky/broadcast bit-exact; exp/tanh/sigmoid
(and the other transcendentals) within 2 float32 ulp; pow(x, 2) bit-exact."""
import numpy as np
import pytest

from gorgonia_amd import _ffi
from gorgonia_amd import device as D
from gorgonia_amd import synth
from oracle import binding as O
from tests.util import assert_bits_equal, ulp_diff

pytestmark = pytest.mark.gpu

EXACT_BIN = ["add", "sub", "mul", "div", "lt", "lte", "gt", "gte", "eq", "ne"]
SIZES = [0, 1, 3, 4, 5, 255, 1024, 4099, 1 << 20, (1 << 20) + 7]


def _special(n, seed):
    """Seeded values salted with signed zeros, denormals, infinities, NaN, ties."""
    a = synth.uniform(seed, (n,), -4.0, 4.0)
    sp = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-42, -1e-42, 3.4e38, -3.4e38,
                   1.17549435e-38, 2.0, 0.5], dtype=np.float32)
    k = min(n, sp.size)
    a[:k] = sp[:k]
    return a


def _operands(mode, n):
    if mode == "vv":
        return _special(n, 11), _special(n, 23)[::-1].copy()
    if mode == "vs":
        return _special(n, 11), np.array([1.5], dtype=np.float32)
    if mode == "sv":
        return np.array([-2.25], dtype=np.float32), _special(n, 23)
    return np.array([3.0], dtype=np.float32), np.array([-0.75], dtype=np.float32)


@pytest.mark.parametrize("fn", EXACT_BIN)
@pytest.mark.parametrize("mode", ["vv", "vs", "sv", "ss"])
def test_binary_bit_exact(ctx, fn, mode):
    for n in ([1] if mode == "ss" else SIZES):
        a, b = _operands(mode, n)
        da, db = ctx.upload(a), ctx.upload(b)
        ctx.run(D.cmd_bin(fn, mode, da, db, n))
        dst, dst_host, src, src_host = (db, b, da, a) if mode == "sv" else (da, a, db, b)
        got = ctx.d2h(dst, dst_host.shape)
        assert_bits_equal(got, O.binop(fn, mode, a, b), f"{fn}_{mode} n={n}")
        # the operand that is not the destination is left untouched
        assert_bits_equal(ctx.d2h(src, src_host.shape), src_host, f"{fn}_{mode} source operand")
        ctx.free(da)
        ctx.free(db)


def test_binary_unaligned_operands(ctx):
    n = 1000
    a = synth.uniform(5, (n + 3,), -4, 4)
    b = synth.uniform(6, (n + 3,), -4, 4)
    da, db = ctx.upload(a), ctx.upload(b)
    ctx.run(D.cmd_bin("mul", "vv", da + 4, db + 8, n))  # 4- and 8-byte offsets
    got = ctx.d2h(da, (n + 3,))
    want = a.copy()
    want[1:n + 1] = O.binop("mul", "vv", a[1:n + 1], b[2:n + 2])
    assert_bits_equal(got, want, "unaligned mul")
    ctx.free(da); ctx.free(db)


def test_binary_f64(ctx):
    n = 4099
    rng = np.random.default_rng(3)
    a = rng.uniform(-4, 4, n)
    b = rng.uniform(-4, 4, n)
    for fn in ["add", "sub", "mul", "div", "gte"]:
        da, db = ctx.upload(a), ctx.upload(b)
        ctx.run(D.cmd_bin(fn, "vv", da, db, n, dtype=1))
        got = ctx.d2h(da, (n,), np.float64)
        assert_bits_equal(got, O.binop(fn, "vv", a, b), f"{fn}_vv_f64")
        ctx.free(da); ctx.free(db)


def test_pow_scalar_two_is_exact_square(ctx):
    n = (1 << 18) + 3
    a = synth.uniform(7, (n,), 0.0, 1.0)
    two = np.array([2.0], dtype=np.float32)
    da, db = ctx.upload(a), ctx.upload(two)
    ctx.run(D.cmd_bin("pow", "vs", da, db, n))
    got = ctx.d2h(da, (n,))
    assert_bits_equal(got, O.binop("pow", "vs", a, two), "pow(x,2) vs oracle")
    assert_bits_equal(got, a * a, "pow(x,2) == x*x")
    ctx.free(da); ctx.free(db)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_mod_bit_exact(ctx, dtype):
    """Engine.Mod (cuda/arith.go:589-640): math.Mod semantics, exact in both widths."""
    n = 100_003
    a = (synth.uniform(31, (n,), -50, 50)).astype(dtype)
    b = (synth.uniform(32, (n,), -7, 7)).astype(dtype)
    special = np.array([0.0, -0.0, 5.5, -5.5, np.inf, -np.inf, np.nan, 1e30, 3.0], dtype=dtype)
    a[:81] = np.repeat(special, 9)
    b[:81] = np.tile(special, 9)
    dt = _ffi.F32 if dtype == np.float32 else _ffi.F64
    for mode in ("vv", "vs", "sv"):
        A = a.copy() if mode != "sv" else a[:1].copy()
        B = b.copy() if mode != "vs" else b[3:4].copy()
        da, db = ctx.upload(A), ctx.upload(B)
        ctx.run(D.cmd_bin("mod", mode, da, db, n, dtype=dt))
        got = ctx.d2h(db if mode == "sv" else da, (n,), dtype)
        ctx.free(da); ctx.free(db)
        want = O.binop("mod", mode, A, B)
        assert_bits_equal(got, want, f"mod {mode} {dtype.__name__}")
        with np.errstate(invalid="ignore", divide="ignore"):
            ref = np.fmod(A if mode != "sv" else np.full(n, A[0], dtype), B if mode != "vs" else np.full(n, B[0], dtype))
        assert_bits_equal(got, ref.astype(dtype), f"mod {mode} against fmod")


def test_pow_general(ctx):
    n = 50000
    a = synth.uniform(8, (n,), 0.01, 4.0)
    b = synth.uniform(9, (n,), -3.0, 3.0)
    da, db = ctx.upload(a), ctx.upload(b)
    ctx.run(D.cmd_bin("pow", "vv", da, db, n))
    got = ctx.d2h(da, (n,))
    assert ulp_diff(got, O.binop("pow", "vv", a, b)).max() <= 2
    ctx.free(da); ctx.free(db)


ULP2 = ["exp", "tanh", "sigmoid", "ln", "log2", "sin", "cos", "log1p", "expm1", "softplus"]
EXACT_UNARY = ["abs", "sign", "ceil", "floor", "neg", "square", "sqrt", "inverse", "invsqrt", "cube"]


def _unary_input(fn, n, seed):
    if fn in ("ln", "log2", "sqrt", "invsqrt"):
        x = synth.uniform(seed, (n,), 1e-3, 50.0)
    elif fn == "log1p":
        x = synth.uniform(seed, (n,), -0.99, 50.0)
    elif fn in ("exp", "expm1"):
        x = synth.uniform(seed, (n,), -80.0, 80.0)
    elif fn in ("sigmoid", "softplus"):
        x = synth.uniform(seed, (n,), -110.0, 30.0)
    elif fn == "tanh":
        x = np.concatenate([synth.uniform(seed, (n // 2,), -12.0, 12.0),
                            synth.uniform(seed + 1, (n - n // 2,), -0.01, 0.01)])
    else:
        x = synth.uniform(seed, (n,), -4.0, 4.0)
    sp = np.array([0.0, -0.0, 1.0, -1.0, 0.5, -0.5, 1e-30, -1e-30, 15.0, 15.000001, -88.0,
                   -88.00001, 14.0, -103.0, 20.0, -20.0], dtype=np.float32)
    if fn not in ("ln", "log2", "sqrt", "invsqrt", "log1p", "inverse"):
        x[:sp.size] = sp
    return x.astype(np.float32)


@pytest.mark.parametrize("fn", ULP2)
def test_unary_within_2ulp(ctx, fn):
    for n in [5, 4099, (1 << 20) + 3]:
        x = _unary_input(fn, max(n, 32), 31)[:n] if n < 32 else _unary_input(fn, n, 31)
        d = ctx.upload(x)
        ctx.run(D.cmd_unary(fn, d, x.size))
        got = ctx.d2h(d, (x.size,))
        want = O.unary(fn, x)
        u = ulp_diff(got, want)
        assert u.max() <= 2, f"{fn}: max ulp {u.max()} at x={x[int(u.argmax())]!r}"
        ctx.free(d)


@pytest.mark.parametrize("fn", EXACT_UNARY)
def test_unary_bit_exact(ctx, fn):
    for n in [5, 4099, (1 << 20) + 3]:
        x = _unary_input(fn, max(n, 32), 41)[:n]
        d = ctx.upload(x)
        ctx.run(D.cmd_unary(fn, d, x.size))
        got = ctx.d2h(d, (x.size,))
        assert_bits_equal(got, O.unary(fn, x), fn)
        ctx.free(d)


UNARY_SPECIALS = [0.0, -0.0, np.nan, np.inf, -np.inf, 1e-42, -1e-42, 1.0, -1.0, 2.5, -2.5, 0.5, -0.5,
                  3.0e38, -3.0e38, 16777216.0]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("fn", EXACT_UNARY)
def test_unary_special_values_bit_exact(ctx, fn, dtype):
    """Signed zeros, NaN, infinities and denormals through the single-operation codes, both
    widths.  sign follows the device kernel form (x > 0) - (x < 0) of
    "cuda modules/src/elemunaryop.cu":125-131: +0 for +0, -0 and NaN."""
    x = np.array(UNARY_SPECIALS, dtype=dtype)
    d = ctx.upload(x)
    ctx.run(D.cmd_unary(fn, d, x.size, dtype=_ffi.F32 if dtype == np.float32 else _ffi.F64))
    got = ctx.d2h(d, (x.size,), dtype)
    ctx.free(d)
    with np.errstate(all="ignore"):
        want = O.unary(fn, x)
    assert_bits_equal(got, want, f"{fn} {dtype.__name__}")
    if fn == "sign":
        z = got[:3].view(np.uint32 if dtype == np.float32 else np.uint64)
        assert (z == 0).all(), "sign(+0), sign(-0), sign(NaN) must be +0"


@pytest.mark.parametrize("fn", ULP2 + EXACT_UNARY)
def test_unary_float64(ctx, fn):
    """The float64 twins: single-operation codes bit-exact, the transcendental ones within
    2 float64 ulp of the oracle (float64 libm), cut-offs of the reference's scalar forms
    (math.go:50-58, math_nooptim.go:25-34) included in the inputs."""
    n = 20011
    x = _unary_input(fn, n, 53).astype(np.float64)
    x[16:] += np.random.default_rng(54).uniform(-1e-9, 1e-9, n - 16) * np.abs(x[16:])  # use the low mantissa bits
    if fn == "sigmoid":
        x[16:32] = [-709.0, -709.5, np.nextafter(-709.0, -800.0), -708.9, 19.0, 19.5, np.nextafter(19.0, 20.0), 16.0,
                    -100.0, -88.5, 15.5, 18.99, -700.0, 0.0, 40.0, -800.0]
    if fn == "softplus":
        x[16:32] = [-708.0, -708.5, np.nextafter(-708.0, -800.0), -707.9, 16.0, 16.5, np.nextafter(16.0, 17.0), 15.0,
                    -200.0, -103.5, 14.5, 15.99, -700.0, 0.0, 40.0, -800.0]
    d = ctx.upload(x)
    ctx.run(D.cmd_unary(fn, d, n, dtype=_ffi.F64))
    got = ctx.d2h(d, (n,), np.float64)
    ctx.free(d)
    with np.errstate(all="ignore"):
        want = O.unary(fn, x)
    if fn in EXACT_UNARY:
        assert_bits_equal(got, want, f"{fn} float64")
        return
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    gi, wi = got[ok].view(np.int64), want[ok].view(np.int64)
    gi = np.where(gi < 0, -(gi & 0x7FFFFFFFFFFFFFFF), gi)
    wi = np.where(wi < 0, -(wi & 0x7FFFFFFFFFFFFFFF), wi)
    u = np.abs(gi - wi)
    assert u.max() <= 2, f"{fn}: {u.max()} ulp at x={x[ok][int(u.argmax())]!r}"
    if fn in ("sigmoid", "softplus"):   # the cut-offs store exact values
        assert_bits_equal(got[16:32][[1, 2, 5, 6, 15]], want[16:32][[1, 2, 5, 6, 15]], f"{fn} cut-offs")


@pytest.mark.parametrize("fn", ["sigmoid", "tanh"])
def test_sigmoid_tanh_dense_sweep(ctx, fn):
    """Every 61st float32 bit pattern of both signs (70 million values, NaNs and infinities
    included) against the oracle (float64 libm rounded once): at most 2 ulp anywhere."""
    chunk = 1 << 24
    d = ctx.malloc(chunk * 4)
    worst = 0
    for start in range(0, 1 << 32, 61 * chunk):
        bits = (np.arange(chunk, dtype=np.uint64) * 61 + start)
        bits = bits[bits < (1 << 32)].astype(np.uint32)
        x = bits.view(np.float32)
        ctx.h2d(d, x)
        ctx.run(D.cmd_unary(fn, d, x.size))
        got = ctx.d2h(d, (x.size,))
        want = O.unary(fn, x)
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(got), nan)
        diff = ulp_diff(got[~nan], want[~nan])
        worst = max(worst, int(diff.max()))
        assert worst <= 2, (fn, x[~nan][np.argmax(diff)], got[~nan][np.argmax(diff)], want[~nan][np.argmax(diff)])
    ctx.free(d)
    print(f"{fn}: worst error over the sweep {worst} ulp")


def test_sigmoid_identities(ctx):
    """Closed-form pins of the sigmoid kernel itself: s(0)=1/2, cut-offs
    (math_nooptim.go:36-44), monotone, s(x)+s(-x)=1 within rounding."""
    x = np.linspace(-20, 15, 70001).astype(np.float32)
    xs = np.concatenate([x, -x, np.array([0.0, -88.5, 15.5, -88.0, 15.0], np.float32)])
    d = ctx.upload(xs)
    ctx.run(D.cmd_unary("sigmoid", d, xs.size))
    s = ctx.d2h(d, (xs.size,))
    n = x.size
    assert s[2 * n] == 0.5 and s[2 * n + 1] == 0.0 and s[2 * n + 2] == 1.0
    assert s[2 * n + 3] > 0.0 and s[2 * n + 4] < 1.0
    assert np.all(np.diff(s[:n]) >= 0)
    ok = np.abs(x) <= 15
    assert np.max(np.abs(s[:n][ok].astype(np.float64) + s[n:2 * n][ok] - 1.0)) <= 2 ** -23
    ctx.free(d)


@pytest.mark.parametrize("fn", ["add", "mul", "sub", "div"])
@pytest.mark.parametrize("shape", [(64, 4096, 1), (7, 12, 1), (8, 16, 169), (3, 5, 64), (1, 4096, 1),
                                   (4096, 8, 1)])
@pytest.mark.parametrize("left", [False, True])
def test_broadcast_bit_exact(ctx, fn, shape, left):
    outer, mid, inner = shape
    big = synth.uniform(51, (outer * mid * inner,), -4, 4)
    small = synth.uniform(52, (mid,), -4, 4)
    db, ds = ctx.upload(big), ctx.upload(small)
    dd = ctx.malloc(big.nbytes)
    ctx.run(D.cmd_bcast(fn, dd, db, ds, outer, mid, inner, small_left=left))
    got = ctx.d2h(dd, big.shape)
    assert_bits_equal(got, O.bcast_binop(fn, big, small, outer, mid, inner, left), f"bcast {fn}")
    ctx.free(db); ctx.free(ds); ctx.free(dd)


@pytest.mark.parametrize("fn", ["add", "mul", "sub", "div", "lt", "gte"])
@pytest.mark.parametrize("shape", [(64, 4096, 1), (7, 13, 1), (8, 16, 169), (1, 4098, 1), (4097, 2, 1)])
@pytest.mark.parametrize("left", [False, True])
def test_broadcast_float64_bit_exact(ctx, fn, shape, left):
    """The float64 twin: the same repeat-then-operate result (broadcast.go:69-129), one IEEE operation per element."""
    outer, mid, inner = shape
    big = synth.uniform(53, (outer * mid * inner,), -4, 4).astype(np.float64) + 2.0 ** -40
    small = synth.uniform(54, (mid,), -4, 4).astype(np.float64) - 2.0 ** -41
    db, ds = ctx.upload(big), ctx.upload(small)
    dd = ctx.malloc(big.nbytes)
    ctx.run(D.cmd_bcast(fn, dd, db, ds, outer, mid, inner, small_left=left, dtype=_ffi.F64))
    got = ctx.d2h(dd, big.shape, np.float64)
    assert_bits_equal(got, O.bcast_binop(fn, big, small, outer, mid, inner, left), f"bcast f64 {fn}")
    ctx.free(db); ctx.free(ds); ctx.free(dd)


def test_large_operands_cold_then_warm_same_bits(ctx):
    """Tensors of 32 MiB: the first launch finds them nowhere in the library's account of the
    last-level cache and streams them (non-temporal accesses), the repeat finds them there and
    uses plain accesses, and a launch behind 400 MiB of other traffic streams again.  Every one
    stores the oracle's bits, in place and into a separate destination."""
    n = 8 << 20
    a, b = _special(n, 61), _special(n, 62)[::-1].copy()
    row = synth.uniform(63, (4096,), -4, 4)
    want_mul = O.binop("mul", "vv", a, b)
    want_tanh = O.unary("tanh", a)
    want_vs = O.binop("add", "vs", a, np.array([1.5], np.float32))
    want_bc = O.bcast_binop("add", a, row, n // 4096, 4096, 1, False)
    da, db, dd, dr = ctx.upload(a), ctx.upload(b), ctx.malloc(4 * n), ctx.upload(row)
    ds = ctx.upload(np.array([1.5], np.float32))
    filler = [ctx.malloc(64 << 20) for _ in range(3)]

    def check(tag):
        ctx.run(D.cmd_bin("mul", "vv", da, db, n, dst=dd))
        assert_bits_equal(ctx.d2h(dd, (n,)), want_mul, f"mul vv, {tag}")
        ctx.run(D.cmd_unary("tanh", da, n, dst=dd))
        assert ulp_diff(ctx.d2h(dd, (n,)), want_tanh).max() <= 2, f"tanh, {tag}"
        ctx.run(D.cmd_bin("add", "vs", da, ds, n, dst=dd))
        assert_bits_equal(ctx.d2h(dd, (n,)), want_vs, f"add vs, {tag}")
        ctx.run(D.cmd_bcast("add", dd, da, dr, n // 4096, 4096, 1))
        assert_bits_equal(ctx.d2h(dd, (n,)), want_bc, f"broadcast add, {tag}")

    check("never seen")
    check("just used")
    for rep in range(3):               # 3 x 3 x 64 MiB through the streaming kernels
        for f in filler:
            ctx.run(D.cmd_unary("neg", f, 16 << 20))
    check("long unused")
    # in place, cold then warm
    for tag in ("cold", "warm"):
        ctx.run(D.cmd_copy(dd, da, 4 * n))
        if tag == "cold":
            for f in filler:
                ctx.run(D.cmd_unary("neg", f, 16 << 20))
            for f in filler:
                ctx.run(D.cmd_unary("neg", f, 16 << 20))
        ctx.run(D.cmd_bin("mul", "vv", dd, db, n))
        assert_bits_equal(ctx.d2h(dd, (n,)), want_mul, f"mul vv in place, {tag}")
    for p in [da, db, dd, dr, ds] + filler:
        ctx.free(p)


def test_copy_command_from_pinned_host_memory(ctx):
    """GH_OP_MEMCPY_D2D with pinned host memory on the source side, as the tape machine's uploads use it:
    the small sizes go through the copy kernels (128-bit, word and odd-tail forms), the large one through
    the copy engine; every one lands byte for byte."""
    import ctypes as C
    rng = np.random.default_rng(5)
    for nbytes in (64, 4096 + 8, 401408, (4 << 20) - 4, 4 << 20, (6 << 20) + 12, 17 << 20):
        host = C.c_void_p()
        assert ctx.lib.gh_host_alloc(ctx.h, C.c_int64(nbytes), C.byref(host)) == 0
        src = rng.integers(0, 2 ** 32, nbytes // 4, dtype=np.uint32)
        C.memmove(host, src.ctypes.data, nbytes)
        dev = ctx.malloc(nbytes)
        ctx.run(D.cmd_fill(dev, nbytes // 4, 0.0))
        ctx.run(D.cmd_copy(dev, host.value, nbytes))
        got = ctx.d2h(dev, (nbytes // 4,), np.uint32)
        assert np.array_equal(got, src), f"{nbytes} bytes"
        ctx.free(dev)
        assert ctx.lib.gh_host_free(ctx.h, host) == 0


def test_relu_and_leaky_bit_exact(ctx):
    for n in [1, 7, 4099, (1 << 20) + 1]:
        x = _special(n, 61)
        dx = ctx.upload(x)
        dy = ctx.malloc(x.nbytes)
        ctx.run(D.cmd_relu(dx, dy, n))
        got = ctx.d2h(dy, (n,))
        assert_bits_equal(got, O.relu(x), "relu")
        ctx.run(D.cmd_leaky_relu(dx, dy, n, 0.1))
        assert_bits_equal(ctx.d2h(dy, (n,)), O.leaky_relu(x, 0.1), "leaky")
        ctx.free(dx); ctx.free(dy)
    # negative inputs give -0.0 (x * 0), the CPU engine's form (nn.go:154-162)
    x = np.array([-1.0, -0.0, 0.0, 2.0], np.float32)
    dx = ctx.upload(x); dy = ctx.malloc(16)
    ctx.run(D.cmd_relu(dx, dy, 4))
    got = ctx.d2h(dy, (4,))
    assert np.signbit(got[0]) and got[0] == 0.0 and got[3] == 2.0
    ctx.free(dx); ctx.free(dy)


def test_has_nan_inf(ctx):
    n = 100003
    x = synth.uniform(71, (n,), -4, 4)
    flag = ctx.malloc(4)
    for kind, val in [("nan", np.nan), ("inf", np.inf), ("inf", -np.inf)]:
        d = ctx.upload(x)
        ctx.run(D.cmd_has(kind, d, flag, n))
        assert ctx.d2h(flag, (1,), np.int32)[0] == 0
        y = x.copy(); y[n - 2] = val
        ctx.h2d(d, y)
        ctx.run(D.cmd_has(kind, d, flag, n))
        assert ctx.d2h(flag, (1,), np.int32)[0] == 1
        other = "inf" if kind == "nan" else "nan"
        ctx.run(D.cmd_has(other, d, flag, n))
        assert ctx.d2h(flag, (1,), np.int32)[0] == 0
        ctx.free(d)
    ctx.free(flag)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_has_nan_inf_finds_one_value_anywhere(ctx, dt):
    """One NaN / Inf at the first element, the last, in the unaligned elements in front of the 16-byte vectors,
    behind them and in the middle, of tensors at every 4- or 8-byte offset: found; absent: not found; values next
    to the tensor never looked at."""
    code = _ffi.F32 if dt == np.float32 else _ffi.F64
    size = np.dtype(dt).itemsize
    flag = ctx.malloc(4)
    rng = np.random.default_rng(5)
    for n in (1, 3, 4100, 65537, 1 << 20):
        for off in range(0, 16 // size + 1):
            host = synth.uniform(80 + off, (n + 8,), -4, 4).astype(dt)
            host[:off] = np.nan                  # outside the tensor: must not be seen
            host[off + n:] = np.inf
            d = ctx.upload(host)
            a = d + off * size
            for kind in ("nan", "inf"):
                ctx.run(D.cmd_has(kind, a, flag, n, dtype=code))
                assert ctx.d2h(flag, (1,), np.int32)[0] == 0, (n, off, kind)
            for pos in sorted({0, n - 1, min(n - 1, 2), max(0, n - 3), int(rng.integers(n))}):
                for kind, val in (("nan", np.nan), ("inf", -np.inf)):
                    y = host.copy()
                    y[off + pos] = val
                    ctx.h2d(d, y)
                    ctx.run(D.cmd_has(kind, a, flag, n, dtype=code))
                    assert ctx.d2h(flag, (1,), np.int32)[0] == 1, (n, off, pos, kind)
                    ctx.run(D.cmd_has("inf" if kind == "nan" else "nan", a, flag, n, dtype=code))
                    assert ctx.d2h(flag, (1,), np.int32)[0] == 0, (n, off, pos, kind, "other")
            ctx.free(d)
    ctx.free(flag)


def test_denormals_and_division_are_ieee(ctx):
    """No flush-to-zero, correctly rounded division (the reference builds its
    kernels with -ftz=false -prec-div=true, cmd/cudagen/main.go:41-43)."""
    a = np.array([1e-40, 2e-45, 1.0, 1.0, 7.0, 1e-38], np.float32)
    b = np.array([0.5, 1.0, 3.0, 7.0, 3.0, 0.1], np.float32)
    for fn in ("mul", "div", "add"):
        da, db = ctx.upload(a), ctx.upload(b)
        ctx.run(D.cmd_bin(fn, "vv", da, db, a.size))
        got = ctx.d2h(da, a.shape)
        want = {"mul": a * b, "div": a / b, "add": a + b}[fn]
        assert_bits_equal(got, want, f"ieee {fn}")
        ctx.free(da); ctx.free(db)
