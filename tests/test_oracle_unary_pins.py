"""Pins the rest of the oracle's unary family, the float64 cut-offs and general pow
(oracle/oracle.c unary_f32 / unary_f64 / binop pow) against what the mathematics
fixes: IEEE-754 single operations (numpy), arbitrary-precision values rounded once
(mpmath), known values that tell one function code from another, and the cut-off
constants of the reference's scalar forms (math.go:50-68, math_nooptim.go:19-52).
No GPU."""
import numpy as np
import mpmath
import pytest

from oracle import binding as O

mpmath.mp.prec = 200

F32, F64 = np.float32, np.float64


def bits(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint32 if a.dtype == np.float32 else np.uint64)


def same_bits(got, want):
    got, want = np.ascontiguousarray(got), np.ascontiguousarray(want)
    assert got.dtype == want.dtype
    nan = np.isnan(got) & np.isnan(want)
    return ((bits(got) == bits(want)) | nan).all()


def ulps(got, want):
    """Distance in units in the last place of the array's own type (both finite)."""
    it = np.int32 if got.dtype == np.float32 else np.int64
    a = got.view(it).astype(np.int64)
    b = np.ascontiguousarray(want, dtype=got.dtype).view(it).astype(np.int64)
    top = np.int64(0x7FFFFFFF if got.dtype == np.float32 else 0x7FFFFFFFFFFFFFFF)
    a = np.where(a < 0, -(a & top), a)
    b = np.where(b < 0, -(b & top), b)
    return np.abs(a - b)


def samples(dt, lo, hi, n, seed):
    rng = np.random.default_rng(seed)
    return rng.uniform(lo, hi, n).astype(dt)


def rounded(fn, xs, dt):
    """fn evaluated with 200 bits on the exact value of each x and rounded once to dt."""
    out = np.empty(len(xs), dtype=dt)
    for i, x in enumerate(xs):
        v = fn(mpmath.mpf(float(x)))
        out[i] = _round_to(v, dt)
    return out


def _round_to(v, dt):
    if dt is F64:
        return F64(float(v))               # mpmath -> float is correctly rounded
    # float32: round the 200-bit value directly (going through float64 could round twice)
    if v == 0:
        return F32(0.0)
    m, e = mpmath.frexp(v)                 # v = m * 2**e, 0.5 <= |m| < 1
    e = int(e)
    emin = -149                            # the smallest float32 subnormal is 2**-149
    q = max(e - 24, emin)                  # exponent of the last kept bit
    scaled = v / mpmath.mpf(2) ** q
    n = int(mpmath.nint(scaled))           # nint rounds half to even
    return F32(np.ldexp(float(n), q))


SPECIALS32 = np.array([0.0, -0.0, 1.0, -1.0, 0.5, -0.5, 2.5, -2.5, 1e-40, -1e-40, 3.4e38, -3.4e38,
                       np.inf, -np.inf, np.nan, 16777216.0, 8388607.5, -8388607.5, 1.5, -1.5], F32)


# ---- single IEEE operations: any conforming implementation has the same bits ----------------

@pytest.mark.parametrize("dt", [F32, F64])
def test_exact_unary_codes_against_numpy_ieee(dt):
    x = np.concatenate([samples(dt, -50, 50, 4000, 3), SPECIALS32.astype(dt),
                        samples(dt, -1e-3, 1e-3, 200, 4)])
    one = dt(1)
    with np.errstate(all="ignore"):
        want = {
            "abs": np.abs(x), "neg": -x, "square": x * x, "cube": (x * x) * x,
            "ceil": np.ceil(x), "floor": np.floor(x), "sqrt": np.sqrt(x),
            "inverse": one / x, "invsqrt": one / np.sqrt(x),
        }
        for fn, w in want.items():
            got = O.unary(fn, x)
            assert got.dtype == dt
            assert same_bits(got, w.astype(dt)), fn
    # one value per code that no other code of the family produces
    v = dt(-2.25)
    assert O.unary("abs", np.array([v]))[0] == 2.25
    assert O.unary("neg", np.array([v]))[0] == 2.25 and O.unary("neg", np.array([dt(2.25)]))[0] == -2.25
    assert O.unary("square", np.array([v]))[0] == 5.0625
    assert O.unary("cube", np.array([dt(-1.5)]))[0] == -3.375
    assert O.unary("ceil", np.array([v]))[0] == -2 and O.unary("floor", np.array([v]))[0] == -3
    assert O.unary("sqrt", np.array([dt(6.25)]))[0] == 2.5
    assert O.unary("inverse", np.array([dt(-8)]))[0] == -0.125
    assert O.unary("invsqrt", np.array([dt(16)]))[0] == 0.25
    # neg flips the sign bit of zero, abs clears it, ceil of (-1, 0) is -0
    z = O.unary("neg", np.array([dt(0.0)]))
    assert np.signbit(z[0]) and not np.signbit(O.unary("abs", z)[0])
    assert np.signbit(O.unary("ceil", np.array([dt(-0.5)]))[0])


@pytest.mark.parametrize("dt", [F32, F64])
def test_sign_follows_the_device_kernel_form(dt):
    """(x > 0) - (x < 0), "cuda modules/src/elemunaryop.cu":125-131 - the one form of sign the
    reference's sources hold for the device path.  gorgonia's scalar fallback (math.go:13-25)
    and the tensor package's StdEng.Sign (not vendored) agree with it on every non-zero
    number; they differ at zero and NaN, where this form gives +0."""
    x = np.concatenate([samples(dt, -50, 50, 2000, 5), np.array([1e-40, -1e-40, np.inf, -np.inf], dt)])
    got = O.unary("sign", x)
    assert same_bits(got, np.sign(x).astype(dt))
    assert set(np.unique(got)) == {-1.0, 1.0}
    z = O.unary("sign", np.array([0.0, -0.0, np.nan], dt))
    assert (bits(z) == 0).all(), "sign(+0), sign(-0) and sign(NaN) are +0 in the device form"


# ---- transcendental codes: 200-bit value rounded once, plus known values ---------------------

TRANS = {
    "sin": (mpmath.sin, -20.0, 20.0),
    "cos": (mpmath.cos, -20.0, 20.0),
    "exp": (mpmath.exp, -80.0, 80.0),
    "ln": (mpmath.log, 1e-6, 1e6),
    "log2": (lambda v: mpmath.log(v, 2), 1e-6, 1e6),
    "log1p": (mpmath.log1p, -0.999, 50.0),
    "expm1": (mpmath.expm1, -30.0, 30.0),
    "tanh": (mpmath.tanh, -12.0, 12.0),
}


@pytest.mark.parametrize("fn", sorted(TRANS))
def test_transcendental_f32_is_the_exact_value_rounded_once(fn):
    """The float32 forms go through float64 libm and round once (math_nooptim.go:22 for tanh,
    the same shape for the others): at most 1 ulp from the correctly rounded value, and equal
    to it except in the rare double-rounding case."""
    f, lo, hi = TRANS[fn]
    x = np.concatenate([samples(F32, lo, hi, 600, 7), samples(F32, max(lo, -1e-3), min(hi, 1e-3) if lo < 0 else lo * 2, 100, 8)])
    got = O.unary(fn, x)
    want = rounded(f, x, F32)
    d = ulps(got, want)
    assert d.max() <= 1, (fn, x[d.argmax()])
    assert (d == 0).mean() > 0.999, fn


@pytest.mark.parametrize("fn", sorted(TRANS))
def test_transcendental_f64_within_one_ulp_of_the_exact_value(fn):
    f, lo, hi = TRANS[fn]
    x = samples(F64, lo, hi, 400, 9)
    got = O.unary(fn, x)
    want = rounded(f, x, F64)
    d = ulps(got, want)
    assert d.max() <= 1, (fn, x[d.argmax()], got[d.argmax()], want[d.argmax()])


@pytest.mark.parametrize("dt", [F32, F64])
def test_transcendental_known_values_tell_the_codes_apart(dt):
    u = lambda fn, v: O.unary(fn, np.array([v], dt))[0]
    eps = 2 * np.finfo(dt).eps
    assert abs(u("sin", np.pi / 6) - 0.5) <= eps and u("sin", 0.0) == 0
    assert abs(u("cos", np.pi / 3) - 0.5) <= eps and u("cos", 0.0) == 1
    assert u("exp", 0.0) == 1 and abs(u("exp", 1.0) - np.e) <= 2 * eps
    assert u("ln", 1.0) == 0 and abs(u("ln", np.e) - 1) <= eps
    assert u("log2", 8.0) == 3 and u("log2", 0.25) == -2 and u("log2", 1.0) == 0
    for k in range(-20, 21):
        assert u("log2", 2.0 ** k) == k
    # log1p and expm1 at an argument where ln(1+x) and exp(x)-1 lose every digit
    t = dt(2.0) ** (-40 if dt is F32 else -60)
    assert u("log1p", t) == t and u("expm1", t) == t
    assert abs(u("log1p", np.e - 1) - 1) <= eps and abs(u("expm1", 1.0) - (np.e - 1)) <= 2 * eps
    assert u("tanh", 0.0) == 0 and u("tanh", 40.0) == 1 and u("tanh", -40.0) == -1
    # domain edges
    with np.errstate(all="ignore"):
        assert np.isnan(u("ln", -1.0)) and u("ln", 0.0) == -np.inf
        assert np.isnan(u("log2", -1.0)) and u("log1p", -1.0) == -np.inf and np.isnan(u("log1p", -2.0))
        assert u("expm1", -np.inf) == -1 and u("exp", -np.inf) == 0


# ---- the cut-offs of the reference's scalar forms --------------------------------------------

def test_softplus_f32_cutoffs_and_values():
    """math.go:60-68: 0 below -103, x above 14, float32(log1p(exp(float64(x)))) between."""
    sp = lambda v: O.unary("softplus", np.array([v], F32))[0]
    below, above = np.nextafter(F32(-103), F32(-200)), np.nextafter(F32(14), F32(20))
    assert sp(below) == 0 and sp(-150.0) == 0
    assert sp(-103.0) == F32(1e-45), "at the cut-off itself the formula runs: the smallest subnormal"
    assert sp(-103.5) == 0, "without the cut-off this would be the smallest subnormal too"
    assert sp(above) == above and sp(14.5) == F32(14.5) and sp(1e30) == F32(1e30)
    assert sp(14.0) == _round_to(mpmath.log1p(mpmath.exp(14)), F32) and sp(14.0) > 14
    # 14.5 tells the cut-off from the formula: log1p(exp(14.5)) rounds to the float32 above 14.5
    assert _round_to(mpmath.log1p(mpmath.exp(mpmath.mpf(14.5))), F32) > F32(14.5)
    x = samples(F32, -103, 14, 800, 11)
    want = rounded(lambda v: mpmath.log1p(mpmath.exp(v)), x, F32)
    assert ulps(O.unary("softplus", x), want).max() <= 1
    assert sp(0.0) == F32(np.log(2.0))


def test_softplus_f64_cutoffs_and_values():
    """math.go:50-58: 0 below -708, x above 16."""
    sp = lambda v: O.unary("softplus", np.array([v], F64))[0]
    assert sp(np.nextafter(-708.0, -800.0)) == 0 and sp(-708.5) == 0 and sp(-1000.0) == 0
    assert sp(-708.0) > 0 and abs(sp(-708.0) / float(mpmath.exp(-708)) - 1) < 1e-15
    assert float(mpmath.exp(mpmath.mpf(-708.5))) > 0, "so the zero at -708.5 is the cut-off, not underflow"
    assert sp(16.5) == 16.5 and sp(np.nextafter(16.0, 17.0)) == np.nextafter(16.0, 17.0) and sp(1e300) == 1e300
    assert float(mpmath.log1p(mpmath.exp(mpmath.mpf(16.5)))) > 16.5, "the formula would not return x at 16.5"
    assert sp(16.0) == float(mpmath.log1p(mpmath.exp(16))) and sp(16.0) > 16
    # float32's cut-offs (-103, 14) must not be the ones in force here
    assert sp(15.0) > 15.0 and sp(-200.0) > 0
    x = samples(F64, -700, 16, 500, 12)
    want = rounded(lambda v: mpmath.log1p(mpmath.exp(v)), x, F64)
    assert ulps(O.unary("softplus", x), want).max() <= 2
    assert sp(0.0) == np.log(2.0)


def test_sigmoid_f64_cutoffs_and_values():
    """math_nooptim.go:25-34: 0 below -709, 1 above 19, 1/(1+exp(-x)) between."""
    sg = lambda v: O.unary("sigmoid", np.array([v], F64))[0]
    assert sg(np.nextafter(-709.0, -800.0)) == 0 and sg(-709.5) == 0 and sg(-1e4) == 0
    assert sg(-709.0) > 0
    assert float(1 / (1 + mpmath.exp(mpmath.mpf(709.5)))) > 0, "so the zero at -709.5 is the cut-off"
    assert sg(19.5) == 1 and sg(np.nextafter(19.0, 20.0)) == 1
    assert sg(19.0) < 1 and float(1 / (1 + mpmath.exp(mpmath.mpf(-19.5)))) < 1
    # float32's cut-offs (-88, 15) must not be the ones in force here
    assert sg(16.0) < 1 and abs(sg(16.0) - float(1 / (1 + mpmath.exp(-16)))) < 1e-16
    assert sg(-100.0) > 0 and abs(sg(-100.0) / float(mpmath.exp(-100)) - 1) < 1e-15
    assert sg(0.0) == 0.5
    x = samples(F64, -700, 19, 500, 13)
    want = rounded(lambda v: 1 / (1 + mpmath.exp(-v)), x, F64)
    assert ulps(O.unary("sigmoid", x), want).max() <= 2
    # symmetry s(x) + s(-x) = 1
    x = samples(F64, -18, 18, 500, 14)
    assert np.max(np.abs(O.unary("sigmoid", x) + O.unary("sigmoid", -x) - 1)) <= 2.3e-16


def test_sigmoid_f32_cutoffs_exactly():
    """math_nooptim.go:36-44 at the neighbours of -88 and 15."""
    sg = lambda v: O.unary("sigmoid", np.array([v], F32))[0]
    assert sg(np.nextafter(F32(-88), F32(-90))) == 0 and sg(-88.0) == _round_to(1 / (1 + mpmath.exp(88)), F32) > 0
    assert sg(np.nextafter(F32(15), F32(16))) == 1 and sg(15.0) == _round_to(1 / (1 + mpmath.exp(-15)), F32) < 1
    # the formula alone would give a subnormal, not 0, at -100
    assert _round_to(1 / (1 + mpmath.exp(100)), F32) > 0 and sg(-100.0) == 0


# ---- general pow ---------------------------------------------------------------------------

@pytest.mark.parametrize("dt", [F32, F64])
def test_pow_exact_cases(dt):
    p = lambda a, b, mode="vv": O.binop("pow", mode, np.asarray(a, dt).reshape(-1), np.asarray(b, dt).reshape(-1))
    # integer powers whose value is representable: exact in any faithful pow
    a = np.array([2, 3, 5, 7, 10, -2, -3, 1.5, -1.5, 0.5, 12, 2, 2, 4, 9], dt)
    b = np.array([10, 5, 3, 2, 4, 3, 4, 3, 3, 7, 2, -3, 0.5 * 2, 0.5, 0.5], dt)
    want = np.array([1024, 243, 125, 49, 10000, -8, 81, 3.375, -3.375, 0.0078125, 144, 0.125, 2, 2, 3], dt)
    assert same_bits(p(a, b), want)
    # square roots of perfect squares and reciprocals of powers of two through pow
    n = np.arange(1, 200, dtype=dt)
    assert same_bits(p(n * n, np.full_like(n, 0.5)), n)
    k = np.arange(-30, 31)
    assert same_bits(p(np.full(k.size, 2, dt), k.astype(dt)), (2.0 ** k).astype(dt))
    assert same_bits(p((2.0 ** k).astype(dt), np.full(k.size, -1, dt)), (2.0 ** -k).astype(dt))
    # operand order: vs is tensor ** scalar, sv is scalar ** tensor
    assert same_bits(p([1, 2, 3], [2], "vs"), np.array([1, 4, 9], dt))
    assert same_bits(p([2], [1, 2, 3], "sv"), np.array([2, 4, 8], dt))
    assert same_bits(p([3], [2], "ss"), np.array([9], dt))
    # special cases every pow shares (C99 F.9.4.4, Go math.Pow)
    with np.errstate(all="ignore"):
        a = np.array([5, 0, -0.0, 0, -8, -8, np.inf, 2, 2, np.nan, 1, -1], dt)
        b = np.array([0, 3, 3, -1, 1 / 3, 3, -1, np.inf, -np.inf, 0, np.nan, np.inf], dt)
        want = np.array([1, 0, -0.0, np.inf, np.nan, -512, 0, np.inf, 0, 1, 1, 1], dt)
        assert same_bits(p(a, b), want)


@pytest.mark.parametrize("dt", [F32, F64])
def test_pow_general_is_the_exact_value_rounded_once(dt):
    a = samples(dt, 0.05, 30, 500, 21)
    b = samples(dt, -6, 6, 500, 22)
    got = O.binop("pow", "vv", a, b)
    want = np.array([_round_to(mpmath.power(mpmath.mpf(float(x)), mpmath.mpf(float(y))), dt)
                     for x, y in zip(a, b)], dt)
    d = ulps(got, want)
    assert d.max() <= 1, (a[d.argmax()], b[d.argmax()])
    if dt is F32:
        assert (d == 0).mean() > 0.999
    # large integer powers beyond the mantissa, against exact integer arithmetic
    base = np.arange(3, 40, 2)
    for e in (9, 14, 23):
        want = np.array([dt(int(v) ** e) if dt is F64 else _round_to(mpmath.mpf(int(v) ** e), F32) for v in base], dt)
        got = O.binop("pow", "vs", base.astype(dt), np.array([e], dt))
        assert ulps(got, want).max() <= (0 if dt is F32 else 1)
