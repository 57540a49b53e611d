"""GPU parity: MatMul / BatchedMatMul / MatVecMul / Outer through the C ABI
against the CPU oracle.  Bar: relative Frobenius error <= 1e-5 against the
float64 product (the oracle's own float32 sequential-k result is held to the
same bar), and exact equality on integer-valued inputs where every summation
order is exact."""
import numpy as np
import pytest

from gorgonia_amd import device as D
from gorgonia_amd import synth
from oracle import binding as O
from tests.util import assert_bits_equal, rel_frobenius

pytestmark = pytest.mark.gpu
TOL = 1e-5


def _run_gemm(ctx, A, B, ta=False, tb=False, act=None, alpha=0.0, softmax=False, bias=None):
    m, k = (A.shape[1], A.shape[0]) if ta else A.shape
    n = B.shape[0] if tb else B.shape[1]
    dA, dB = ctx.upload(A), ctx.upload(B)
    dbias = ctx.upload(bias) if bias is not None else 0
    dC = ctx.malloc(m * n * 4)
    ctx.run(D.cmd_fill(dC, m * n, np.nan))
    ctx.run(D.cmd_gemm(dA, dB, dC, m, n, k, trans_a=ta, trans_b=tb, act=act, alpha=alpha, softmax=softmax,
                       bias=dbias))
    out = ctx.d2h(dC, (m, n))
    for p in (dA, dB, dC) + ((dbias,) if dbias else ()):
        ctx.free(p)
    return out


SHAPES = [(1, 1, 1), (3, 5, 7), (32, 32, 2), (64, 64, 16), (65, 129, 33), (128, 128, 128),
          (256, 784, 300), (256, 300, 100), (256, 100, 10), (128, 1152, 625), (130, 10, 625),
          (512, 512, 512), (1000, 37, 259),
          # 16x16-tile small-output kernel: ragged edges, K not a multiple of 4 or 16
          (100, 333, 37), (17, 1001, 48), (16, 35, 33), (64, 4096, 1000)]  # (m, k, n)


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
def test_matmul_vs_oracle(ctx, ta, tb):
    for (m, k, n) in SHAPES:
        A = synth.normal(100 + m, (k, m) if ta else (m, k))
        B = synth.normal(200 + n, (n, k) if tb else (k, n))
        got = _run_gemm(ctx, A, B, ta, tb)
        ref = O.gemm_f64acc(A, B, ta, tb)
        err = rel_frobenius(got, ref)
        assert err <= TOL, f"gemm {m}x{k}x{n} ta={ta} tb={tb}: rel frobenius {err:.3e}"
        assert rel_frobenius(O.gemm(A, B, ta, tb), ref) <= TOL


def test_matmul_small_output_shapes_sweep(ctx):
    """Seeded sweep over the shapes the small-output kernels take (few output tiles, K from 32
    up, ragged everything, transposed views): every product against the float64 one, and on
    integer-valued operands exactly."""
    rng = np.random.default_rng(2024)
    for case in range(60):
        m = int(rng.integers(1, 200))
        n = int(rng.integers(1, 200))
        k = int(rng.integers(32, 700))
        ta, tb = [(False, False), (True, False), (False, True), (True, True)][case % 4]
        integer = case % 3 == 0
        if integer:
            A = rng.integers(-4, 5, (k, m) if ta else (m, k)).astype(np.float32)
            B = rng.integers(-4, 5, (n, k) if tb else (k, n)).astype(np.float32)
        else:
            A = synth.normal(1000 + case, (k, m) if ta else (m, k))
            B = synth.normal(2000 + case, (n, k) if tb else (k, n))
        got = _run_gemm(ctx, A, B, ta, tb)
        ref = O.gemm_f64acc(A, B, ta, tb)
        if integer:
            assert np.array_equal(got, ref.astype(np.float32)), f"case {case}: {m}x{k}x{n} ta={ta} tb={tb}"
        else:
            err = rel_frobenius(got, ref)
            assert err <= TOL, f"case {case}: {m}x{k}x{n} ta={ta} tb={tb}: {err:.3e}"


def test_matmul_integer_exact(ctx):
    """Small-integer inputs: every partial sum is exactly representable, so any
    accumulation order must give the oracle's bits."""
    rng = np.random.default_rng(0)
    for (m, k, n) in [(64, 64, 64), (100, 50, 30), (256, 300, 100), (7, 1, 5), (100, 50, 36), (40, 77, 50)]:
        A = rng.integers(-8, 9, (m, k)).astype(np.float32)
        B = rng.integers(-8, 9, (k, n)).astype(np.float32)
        for ta, tb in [(False, False), (False, True), (True, False), (True, True)]:
            As = A.T.copy() if ta else A
            Bs = B.T.copy() if tb else B
            got = _run_gemm(ctx, As, Bs, ta, tb)
            assert_bits_equal(got, O.gemm(As, Bs, ta, tb), f"int gemm ta={ta} tb={tb}")
            assert np.array_equal(got, (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32))


def test_matmul_fused_relu_epilogue(ctx):
    A = synth.normal(1, (256, 784))
    B = synth.normal(2, (784, 300))
    plain = _run_gemm(ctx, A, B)
    fused = _run_gemm(ctx, A, B, act="relu")
    assert_bits_equal(fused, O.relu(plain).reshape(plain.shape), "gemm+relu epilogue")
    fusedl = _run_gemm(ctx, A, B, act="leaky", alpha=0.1)
    assert_bits_equal(fusedl, O.leaky_relu(plain, 0.1).reshape(plain.shape), "gemm+leaky epilogue")


@pytest.mark.parametrize("m,k,n,ta,tb", [
    (256, 784, 300, False, False),    # 16x32 tiles of the small-output kernel
    (64, 512, 1000, False, False),    # 16x16 tiles
    (256, 100, 10, False, False),     # 32x32 tiles
    (512, 512, 512, False, False),    # tiled kernel
    (1024, 4096, 64, False, False),   # tiled kernel with a split K range and the reduction pass
])
def test_matmul_fused_bias_epilogue(ctx, m, k, n, ta, tb):
    """Mul -> BroadcastAdd(row bias) [-> Rectify] as one command stores the bits of the separate commands."""
    A = synth.normal(5, (k, m) if ta else (m, k))
    B = synth.normal(6, (n, k) if tb else (k, n))
    bias = synth.normal(7, (n,))
    plain = _run_gemm(ctx, A, B, ta, tb)
    want = O.bcast_binop("add", plain.reshape(-1), bias, m, n, 1).reshape(m, n)
    assert_bits_equal(_run_gemm(ctx, A, B, ta, tb, bias=bias), want, "gemm+bias epilogue")
    assert_bits_equal(_run_gemm(ctx, A, B, ta, tb, bias=bias, act="relu"), O.relu(want).reshape(m, n),
                      "gemm+bias+relu epilogue")
    if n <= 32 and not (ta or tb):
        assert_bits_equal(_run_gemm(ctx, A, B, bias=bias, softmax=True), O.softmax(want), "gemm+bias+softmax epilogue")


def test_matmul_bias_flag_checks(ctx):
    import ctypes as C
    buf = C.create_string_buffer(256)
    for cmd in (D.cmd_gemm(1, 1, 1, 64, 64, 64, bias=1, dtype=1), D.cmd_gemm(1, 1, 1, 64, 64, 64, bias=1, trans_a=True),
                D.cmd_gemm(1, 1, 1, 64, 64, 64, bias=1, trans_b=True)):
        assert ctx.lib.gh_validate(C.byref(cmd), 1, buf, 256) != 0 and b"bias" in buf.value
    cmd = D.cmd_gemm(1, 1, 1, 64, 64, 64, bias=1)
    cmd.ptr[3] = 0
    assert ctx.lib.gh_validate(C.byref(cmd), 1, buf, 256) != 0 and b"bias" in buf.value


@pytest.mark.parametrize("m,k,n", [(128, 625, 10), (1, 32, 1), (33, 100, 32), (2048, 64, 7), (50, 48, 31)])
def test_matmul_fused_softmax_epilogue(ctx, m, k, n):
    """MatMul -> SoftMax as one command stores the bits of the two commands."""
    A = synth.normal(3, (m, k))
    B = synth.normal(4, (k, n), 0.0, 0.3)
    assert ctx.lib.gh_gemm_can_softmax(D.cmd_gemm(1, 1, 1, m, n, k)) == 1
    plain = _run_gemm(ctx, A, B)
    dx, dy = ctx.upload(plain), ctx.malloc(m * n * 4)
    ctx.run(D.cmd_softmax(dx, dy, m, n))
    want = ctx.d2h(dy, (m, n))
    ctx.free(dx); ctx.free(dy)
    assert_bits_equal(_run_gemm(ctx, A, B, softmax=True), want, "gemm+softmax epilogue")
    assert_bits_equal(want, O.softmax(plain), "softmax kernel vs oracle")
    relu = _run_gemm(ctx, A, B, act="relu", softmax=True)
    assert_bits_equal(relu, O.softmax(O.relu(plain).reshape(plain.shape)), "gemm+relu+softmax epilogue")


def test_matmul_softmax_flag_needs_whole_rows_in_a_tile(ctx):
    import ctypes as C
    buf = C.create_string_buffer(256)
    for cmd in (D.cmd_gemm(1, 1, 1, 64, 33, 64, softmax=True), D.cmd_gemm(1, 1, 1, 64, 10, 16, softmax=True),
                D.cmd_gemm(1, 1, 1, 64, 10, 64, trans_b=True, softmax=True), D.cmd_gemm(1, 1, 1, 4096, 10, 64, softmax=True)):
        assert ctx.lib.gh_gemm_can_softmax(cmd) == 0
        assert ctx.lib.gh_validate(C.byref(cmd), 1, buf, 256) != 0 and b"softmax" in buf.value


def test_matmul_strided_ld(ctx):
    """Leading dimensions larger than the logical width (sub-matrix views)."""
    m, k, n = 70, 52, 44
    Abig = synth.normal(3, (m, k + 12))
    Bbig = synth.normal(4, (k, n + 8))
    dA, dB = ctx.upload(Abig), ctx.upload(Bbig)
    dC = ctx.malloc(m * (n + 4) * 4)
    ctx.run(D.cmd_fill(dC, m * (n + 4), -7.0))
    ctx.run(D.cmd_gemm(dA, dB, dC, m, n, k, lda=k + 12, ldb=n + 8, ldc=n + 4))
    out = ctx.d2h(dC, (m, n + 4))
    ref = O.gemm_f64acc(Abig[:, :k].copy(), Bbig[:, :n].copy())
    assert rel_frobenius(out[:, :n], ref) <= TOL
    assert np.all(out[:, n:] == -7.0)  # padding columns untouched
    for p in (dA, dB, dC):
        ctx.free(p)


@pytest.mark.parametrize("shape", [(4, 32, 48, 40), (64, 64, 64, 64), (3, 130, 70, 50), (6, 2, 3, 2)])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False)])
def test_batched_matmul(ctx, shape, ta, tb):
    batch, m, k, n = shape
    A = synth.normal(5, (batch, k, m) if ta else (batch, m, k))
    B = synth.normal(6, (batch, n, k) if tb else (batch, k, n))
    dA, dB = ctx.upload(A), ctx.upload(B)
    dC = ctx.malloc(batch * m * n * 4)
    ctx.run(D.cmd_gemm(dA, dB, dC, m, n, k, trans_a=ta, trans_b=tb, batch=batch, stride_a=m * k,
                       stride_b=k * n, stride_c=m * n))
    got = ctx.d2h(dC, (batch, m, n))
    want = O.bmm(A, B, ta, tb)
    for b in range(batch):
        ref = O.gemm_f64acc(A[b], B[b], ta, tb)
        assert rel_frobenius(got[b], ref) <= TOL
        assert rel_frobenius(want[b], ref) <= TOL
    for p in (dA, dB, dC):
        ctx.free(p)


def test_batched_matmul_reference_example(ctx):
    """example_linalg_test.go:11-92: BatchedMatMul of Range tensors."""
    a = np.arange(2 * 3 * 2, dtype=np.float32).reshape(2, 3, 2)
    b = np.arange(2 * 2 * 3, dtype=np.float32).reshape(2, 2, 3)
    dA, dB = ctx.upload(a), ctx.upload(b)
    dC = ctx.malloc(2 * 3 * 3 * 4)
    ctx.run(D.cmd_gemm(dA, dB, dC, 3, 3, 2, batch=2, stride_a=6, stride_b=6, stride_c=9))
    got = ctx.d2h(dC, (2, 3, 3))
    assert np.array_equal(got, np.matmul(a, b))
    for p in (dA, dB, dC):
        ctx.free(p)


@pytest.mark.parametrize("m,n", [(1, 1), (5, 3), (64, 64), (300, 784), (1000, 1001), (2048, 4096), (4099, 260),
                                 (33, 8192), (7, 1028)])
@pytest.mark.parametrize("trans", [False, True])
def test_matvec(ctx, m, n, trans):
    A = synth.normal(7, (m, n))
    x = synth.normal(8, (m if trans else n,))
    dA, dx = ctx.upload(A), ctx.upload(x)
    dy = ctx.malloc((n if trans else m) * 4)
    ctx.run(D.cmd_gemv(dA, dx, dy, m, n, trans=trans))
    got = ctx.d2h(dy, (n if trans else m,))
    ref = (A.T if trans else A).astype(np.float64) @ x.astype(np.float64)
    assert rel_frobenius(got, ref) <= TOL
    assert rel_frobenius(O.gemv(A, x, trans), ref) <= TOL
    # integer data: exact in any order of summation; a second launch repeats the bits
    rng = np.random.default_rng(3)
    Ai = rng.integers(-3, 4, (m, n)).astype(np.float32)
    xi = rng.integers(-3, 4, x.shape).astype(np.float32)
    ctx.h2d(dA, Ai); ctx.h2d(dx, xi)
    ctx.run(D.cmd_gemv(dA, dx, dy, m, n, trans=trans))
    gi = ctx.d2h(dy, got.shape)
    assert np.array_equal(gi, ((Ai.T if trans else Ai).astype(np.int64) @ xi.astype(np.int64)).astype(np.float32))
    ctx.h2d(dA, A); ctx.h2d(dx, x)
    ctx.run(D.cmd_gemv(dA, dx, dy, m, n, trans=trans))
    assert_bits_equal(ctx.d2h(dy, got.shape), got, "second launch")
    for p in (dA, dx, dy):
        ctx.free(p)


def test_outer_bit_exact(ctx):
    x = synth.normal(9, (37,))
    y = synth.normal(10, (53,))
    dx, dy = ctx.upload(x), ctx.upload(y)
    dA = ctx.malloc(37 * 53 * 4)
    ctx.run(D.cmd_outer(dx, dy, dA, 37, 53))
    assert_bits_equal(ctx.d2h(dA, (37, 53)), O.outer(x, y), "outer")
    for p in (dx, dy, dA):
        ctx.free(p)


@pytest.mark.parametrize("m,n,trans", [(64, 64, False), (300, 784, False), (100, 300, True), (5, 3, True), (1, 1, False)])
def test_matvec_and_outer_float64(ctx, m, n, trans):
    """Dgemv / Dger paths of Engine.MatVecMul / Outer (cuda/linalg.go:94-159)."""
    from gorgonia_amd import _ffi
    A = synth.normal(7, (m, n)).astype(np.float64) + 1e-9 * synth.normal(17, (m, n)).astype(np.float64)
    x = synth.normal(8, (m if trans else n,)).astype(np.float64)
    dA, dx = ctx.upload(A), ctx.upload(x)
    dy = ctx.malloc((n if trans else m) * 8)
    ctx.run(D.cmd_gemv(dA, dx, dy, m, n, trans=trans, dtype=_ffi.F64))
    got = ctx.d2h(dy, (n if trans else m,), np.float64)
    ref = (A.T if trans else A) @ x
    assert rel_frobenius(got, ref) <= 1e-13
    Ai = np.round(A * 4)
    xi = np.round(x * 4)
    ctx.h2d(dA, Ai); ctx.h2d(dx, xi)
    ctx.run(D.cmd_gemv(dA, dx, dy, m, n, trans=trans, dtype=_ffi.F64))
    assert np.array_equal(ctx.d2h(dy, (n if trans else m,), np.float64), (Ai.T if trans else Ai) @ xi)
    # outer: one product per element, exact
    y = synth.normal(9, (n,)).astype(np.float64) * 1.000000001
    dyv, dO = ctx.upload(y), ctx.malloc(x.size * n * 8)
    ctx.run(D.cmd_outer(dx, dyv, dO, x.size, n, dtype=_ffi.F64))
    assert_bits_equal(ctx.d2h(dO, (x.size, n), np.float64), np.multiply.outer(xi, y), "float64 outer")
    for p in (dA, dx, dy, dyv, dO):
        ctx.free(p)


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
def test_matmul_float64(ctx, ta, tb):
    """Dgemm path of Engine.MatMul (cuda/linalg.go:204-227): float64 on the matrix cores,
    against numpy's float64 product (1e-13 relative) and exactly on integer data."""
    from gorgonia_amd import _ffi
    rng = np.random.default_rng(17)
    for (m, k, n) in [(1, 1, 1), (3, 5, 7), (16, 4, 16), (65, 129, 33), (128, 128, 128), (256, 300, 100), (100, 37, 259),
                      (66, 130, 34), (32, 2, 32), (2050, 70, 2046), (1024, 24, 4100)]:
        for integer in (False, True):
            A = rng.integers(-8, 9, (k, m) if ta else (m, k)).astype(np.float64) if integer else \
                rng.standard_normal((k, m) if ta else (m, k))
            B = rng.integers(-8, 9, (n, k) if tb else (k, n)).astype(np.float64) if integer else \
                rng.standard_normal((n, k) if tb else (k, n))
            dA, dB = ctx.upload(A), ctx.upload(B)
            dC = ctx.malloc(m * n * 8)
            ctx.run(D.cmd_gemm(dA, dB, dC, m, n, k, trans_a=ta, trans_b=tb, dtype=_ffi.F64))
            got = ctx.d2h(dC, (m, n), dtype=np.float64)
            for p in (dA, dB, dC):
                ctx.free(p)
            want = (A.T if ta else A) @ (B.T if tb else B)
            if integer:
                assert np.array_equal(got, want), f"integer dgemm {m}x{k}x{n} ta={ta} tb={tb}"
            else:
                assert rel_frobenius(got, want) <= 1e-13, f"dgemm {m}x{k}x{n} ta={ta} tb={tb}"


def test_batched_matmul_float64(ctx):
    from gorgonia_amd import _ffi
    rng = np.random.default_rng(18)
    A, B = rng.standard_normal((5, 40, 24)), rng.standard_normal((5, 24, 36))
    dA, dB, dC = ctx.upload(A), ctx.upload(B), ctx.malloc(5 * 40 * 36 * 8)
    ctx.run(D.cmd_gemm(dA, dB, dC, 40, 36, 24, batch=5, stride_a=40 * 24, stride_b=24 * 36, stride_c=40 * 36,
                       dtype=_ffi.F64))
    got = ctx.d2h(dC, (5, 40, 36), dtype=np.float64)
    for p in (dA, dB, dC):
        ctx.free(p)
    assert rel_frobenius(got, A @ B) <= 1e-13


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False)])
def test_batched_matmul_float64_large_tiles(ctx, ta, tb):
    """Enough even-sized batches that the float64 product takes its 128x128 tiles, with
    ragged edges in every extent; integer data, so the result is exact."""
    from gorgonia_amd import _ffi
    rng = np.random.default_rng(19)
    bt, m, k, n = 70, 130, 36, 258
    A = rng.integers(-8, 9, (bt, k, m) if ta else (bt, m, k)).astype(np.float64)
    B = rng.integers(-8, 9, (bt, n, k) if tb else (bt, k, n)).astype(np.float64)
    dA, dB, dC = ctx.upload(A), ctx.upload(B), ctx.malloc(bt * m * n * 8)
    ctx.run(D.cmd_gemm(dA, dB, dC, m, n, k, trans_a=ta, trans_b=tb, batch=bt, stride_a=m * k, stride_b=k * n,
                       stride_c=m * n, dtype=_ffi.F64))
    got = ctx.d2h(dC, (bt, m, n), dtype=np.float64)
    for p in (dA, dB, dC):
        ctx.free(p)
    want = (A.transpose(0, 2, 1) if ta else A) @ (B.transpose(0, 2, 1) if tb else B)
    assert np.array_equal(got, want)


def test_matmul_float64_views_sweep(ctx):
    """Seeded sweep of the float64 product over all three kernels (small-output, 64x64 and
    128x128 tiles): every transpose, odd and even extents, operands that are windows of
    larger buffers (leading dimension beyond the row, base 8 bytes off a 16-byte boundary)
    and a strided output.  Integer data: every result must be exact, and the output's
    padding columns must stay untouched."""
    from gorgonia_amd import _ffi
    rng = np.random.default_rng(23)
    shapes = [(70, 96, 33), (130, 200, 64), (17, 300, 9), (200, 66, 140), (512, 40, 512), (1100, 16, 1300),
              (257, 129, 1027), (64, 1024, 48)]
    for idx, (m, k, n) in enumerate(shapes):
        for ta in (False, True):
            for tb in (False, True):
                pa, pb, pc = int(rng.integers(0, 4)), int(rng.integers(0, 4)), int(rng.integers(0, 3))
                oa, ob = int(rng.integers(0, 2)), int(rng.integers(0, 2))
                ra, ca = (k, m) if ta else (m, k)
                rb, cb = (n, k) if tb else (k, n)
                bufA = rng.integers(-6, 7, ra * (ca + pa) + oa).astype(np.float64)
                bufB = rng.integers(-6, 7, rb * (cb + pb) + ob).astype(np.float64)
                A = bufA[oa:].reshape(ra, ca + pa)[:, :ca]
                B = bufB[ob:].reshape(rb, cb + pb)[:, :cb]
                want = (A.T if ta else A) @ (B.T if tb else B)
                Cbuf = np.full((m, n + pc), -77.0)
                dA, dB, dC = ctx.upload(bufA), ctx.upload(bufB), ctx.upload(Cbuf)
                ctx.run(D.cmd_gemm(dA + 8 * oa, dB + 8 * ob, dC, m, n, k, lda=ca + pa, ldb=cb + pb, ldc=n + pc,
                                   trans_a=ta, trans_b=tb, dtype=_ffi.F64))
                got = ctx.d2h(dC, (m, n + pc), dtype=np.float64)
                for p in (dA, dB, dC):
                    ctx.free(p)
                tag = f"case {idx} {m}x{k}x{n} ta={ta} tb={tb} pads {pa},{pb},{pc} offs {oa},{ob}"
                assert np.array_equal(got[:, :n], want), tag
                assert np.all(got[:, n:] == -77.0), tag + ": padding written"
