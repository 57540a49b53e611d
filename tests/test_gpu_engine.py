"""GPU parity through the host mirror of cuda.Engine: the reference's own GPU
test tables (op_math_cuda_test.go, cuda_test.go) replayed against the HIP
engine, plus reuse / unsafe semantics and the linalg case table."""
import json
import os

import numpy as np
import pytest

from gorgonia_amd import synth
from gorgonia_amd.engine import Engine, EngineError
from oracle import binding as O
from tests.util import assert_bits_equal, rel_frobenius

pytestmark = pytest.mark.gpu
G = os.path.join(os.path.dirname(__file__), "golden")


@pytest.fixture(scope="module")
def eng():
    e = Engine()
    e.Init(0, 64 << 20)
    yield e
    e.Close()
    e.destroy()


GO_OP = {"Add": "Add", "Sub": "Sub", "Mul": "Mul", "HadamardProd": "Mul", "Div": "Div", "HadamardDiv": "Div"}


def test_cuda_basic_arithmetic_table(eng):
    """TestCUDABasicArithmetic (op_math_cuda_test.go:44-99) over binOpTests
    (op_math_test.go:23-360): values must be equal, exactly."""
    cases = json.load(open(os.path.join(G, "binop.json")))["cases"]
    ran = 0
    for c in cases:
        dt = np.float32 if c["a"]["bits"] == 32 else np.float64
        a = np.array(c["a"]["v"], dtype=dt)
        b = np.array(c["b"]["v"], dtype=dt)
        want = np.array(c["correct"]["v"], dtype=dt)
        sa, sb = c["a"]["scalar"], c["b"]["scalar"]
        if (c["op"] == "Mul" and not (sa or sb)) or (a.size != b.size and not (sa or sb)):
            continue
        ta = eng.to_device(a, () if sa else None)
        tb = eng.to_device(b, () if sb else None)
        name = GO_OP[c["op"]]
        if sa and sb:
            out = getattr(eng, name)(ta, tb, unsafe=True)
        elif sb:
            out = getattr(eng, name + "Scalar")(ta, tb, True, unsafe=True)
        elif sa:
            out = getattr(eng, name + "Scalar")(tb, ta, False, unsafe=True)
        else:
            out = getattr(eng, name)(ta, tb, unsafe=True)
        eng.DoWork()
        got = eng.to_host(out).reshape(-1)
        assert np.array_equal(got, want), (c["op"], got, want)
        eng.Put(ta.mem, ta.nbytes); eng.Put(tb.mem, tb.nbytes)
        ran += 1
    assert ran >= 20


def test_cuda_cube(eng):
    """TestCUDACube (op_math_cuda_test.go:16-42)."""
    x = np.arange(32, dtype=np.float32)
    t = eng.to_device(x)
    eng.Unary("cube", t)
    eng.DoWork()
    assert np.array_equal(eng.to_host(t), x * x * x)


def test_transfer_round_trip(eng):
    """TestExternMetadata_Transfer (cuda_test.go:60-103): CPU -> GPU -> CPU."""
    x = synth.normal(1, (37, 5))
    t = eng.to_device(x)
    assert t.managed and t.mem != 0
    assert_bits_equal(eng.to_host(t), x, "round trip")
    u = eng.new_tensor((37, 5))
    eng.Memcpy(u, t)  # Engine.Memcpy is eager
    assert_bits_equal(eng.to_host(u), x, "Memcpy")


def test_reuse_and_unsafe_semantics(eng):
    """cuda/arith.go:34-49: with reuse the result lands in reuse and a is left
    alone; unsafe overwrites a; the returned tensor is the one written."""
    a = synth.uniform(2, (1000,), -4, 4)
    b = synth.uniform(3, (1000,), -4, 4)
    ta, tb, tr = eng.to_device(a), eng.to_device(b), eng.new_tensor((1000,))
    ret = eng.Sub(ta, tb, reuse=tr)
    eng.DoWork()
    assert ret is tr
    assert_bits_equal(eng.to_host(tr), a - b, "reuse result")
    assert_bits_equal(eng.to_host(ta), a, "a untouched")
    ret = eng.Sub(ta, tb, unsafe=True)
    eng.DoWork()
    assert ret is ta
    assert_bits_equal(eng.to_host(ta), a - b, "unsafe result in a")
    # scalar on the left writes into the tensor operand / reuse (sv kernels)
    s = eng.to_device(np.array(10.0, np.float32), ())
    ret = eng.DivScalar(tb, s, False, reuse=tr)
    eng.DoWork()
    assert_bits_equal(eng.to_host(tr), np.float32(10.0) / b, "10 / b")
    assert_bits_equal(eng.to_host(tb), b, "b untouched")
    with pytest.raises(EngineError, match="Impossible state"):
        eng.Add(ta, tb)


def test_enqueue_then_flush(eng):
    """Work is only submitted at DoWork/Signal: several ops cost one C-ABI
    submit call (the per-segment batching of the cgo crossing)."""
    x = synth.uniform(4, (4096,), -1, 1)
    t = eng.to_device(x)
    before = eng.submit_calls()
    for name in ("tanh", "square", "neg", "exp"):
        eng.Unary(name, t)
    assert eng.pending() == 4 and eng.submit_calls() == before
    eng.Signal()
    assert eng.pending() == 0 and eng.submit_calls() == before + 1
    want = O.unary("exp", O.unary("neg", O.unary("square", O.unary("tanh", x))))
    from tests.util import ulp_diff
    assert ulp_diff(eng.to_host(t), want).max() <= 4


@pytest.mark.parametrize("za,zb", [(False, False), (True, False), (False, True), (True, True)])
def test_matmul_case_table(eng, za, zb):
    """cuda/linalg.go:161-202: row-major operands, each optionally a transposed view."""
    m, k, n = 70, 45, 52
    A = synth.normal(5, (m, k))
    B = synth.normal(6, (k, n))
    ta = eng.to_device(A.T.copy()).T() if za else eng.to_device(A)
    tb = eng.to_device(B.T.copy()).T() if zb else eng.to_device(B)
    assert ta.shape == (m, k) and tb.shape == (k, n)
    tc = eng.new_tensor((m, n))
    eng.MatMul(ta, tb, tc)
    eng.DoWork()
    ref = A.astype(np.float64) @ B.astype(np.float64)
    assert rel_frobenius(eng.to_host(tc), ref) <= 1e-5


def _col_major(eng, logical, transposed):
    """A column-major tensor of logical shape `logical.shape` on the device.  Without the
    transposed flag its memory is that of logical.T laid out row by row (column-major:
    element (i, j) at j * rows + i); with it, the tensor is the transposed view of the
    column-major matrix logical.T, whose memory is logical row by row."""
    from gorgonia_amd.engine import Tensor
    stored = logical.copy() if transposed else logical.T.copy()
    t = eng.to_device(stored.reshape(-1))
    return Tensor(t.mem, logical.shape, logical.dtype, transposed=transposed, col_major=True)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("za,zb", [(False, False), (True, False), (False, True), (True, True)])
def test_matmul_column_major_case_table(eng, za, zb, dtype):
    """cuda/linalg.go:142-160: column-major operands, each optionally flagged transposed; the
    result is column-major with its row count as leading dimension."""
    from gorgonia_amd.engine import Tensor
    m, k, n = 70, 45, 52
    A = synth.normal(5, (m, k)).astype(dtype)
    B = synth.normal(6, (k, n)).astype(dtype)
    ta, tb = _col_major(eng, A, za), _col_major(eng, B, zb)
    tc = eng.new_tensor((m, n), dtype)
    tc = Tensor(tc.mem, (m, n), dtype, col_major=True)
    eng.MatMul(ta, tb, tc)
    eng.DoWork()
    got = eng.to_host(Tensor(tc.mem, (n, m), dtype)).T   # column-major (m, n) = row-major (n, m), transposed
    ref = A.astype(np.float64) @ B.astype(np.float64)
    assert rel_frobenius(got, ref) <= (1e-5 if dtype == np.float32 else 1e-13)
    # on integer data every summing order is exact: the same bits as the row-major product of the same values
    Ai = np.round(A * 4).astype(dtype)
    Bi = np.round(B * 4).astype(dtype)
    ta, tb = _col_major(eng, Ai, za), _col_major(eng, Bi, zb)
    eng.MatMul(ta, tb, tc)
    eng.DoWork()
    got = eng.to_host(Tensor(tc.mem, (n, m), dtype)).T
    assert np.array_equal(got, (Ai.astype(np.float64) @ Bi.astype(np.float64)).astype(dtype))


def test_matmul_rejects_mixed_data_orders(eng):
    """cuda/linalg.go:118-122."""
    from gorgonia_amd.engine import Tensor, EngineError
    a = eng.to_device(synth.normal(1, (8, 6)))
    b = eng.to_device(synth.normal(2, (6, 5)))
    bc = Tensor(b.mem, (6, 5), np.float32, col_major=True)
    c = eng.new_tensor((8, 5))
    with pytest.raises(EngineError, match="does not have the same data order"):
        eng.MatMul(a, bc, c)


@pytest.mark.parametrize("z", [False, True])
def test_matvec_column_major(eng, z):
    """cuda/linalg.go:57-75: the column-major cases of MatVecMul."""
    A = synth.normal(7, (33, 47))
    x = synth.normal(8, (47,))
    ta, tx, ty = _col_major(eng, A, z), eng.to_device(x), eng.new_tensor((33,))
    eng.MatVecMul(ta, tx, ty)
    eng.DoWork()
    assert rel_frobenius(eng.to_host(ty), A.astype(np.float64) @ x) <= 1e-5


def test_matvec_and_outer(eng):
    A = synth.normal(7, (33, 47))
    x = synth.normal(8, (47,))
    ta, tx, ty = eng.to_device(A), eng.to_device(x), eng.new_tensor((33,))
    eng.MatVecMul(ta, tx, ty)
    eng.DoWork()
    assert rel_frobenius(eng.to_host(ty), A.astype(np.float64) @ x) <= 1e-5
    # transposed view: logical (47, 33) times a 33-vector
    x2 = synth.normal(9, (33,))
    tx2, ty2 = eng.to_device(x2), eng.new_tensor((47,))
    eng.MatVecMul(ta.T(), tx2, ty2)
    eng.DoWork()
    assert rel_frobenius(eng.to_host(ty2), A.T.astype(np.float64) @ x2) <= 1e-5
    to = eng.new_tensor((47, 33))
    eng.Outer(tx, tx2, to)
    eng.DoWork()
    assert_bits_equal(eng.to_host(to), O.outer(x, x2), "outer")


def test_nan_inf_watch(eng):
    x = synth.normal(10, (5000,))
    t = eng.to_device(x)
    assert not eng.HasNaN(t) and not eng.HasInf(t)
    x[4321] = np.nan
    t2 = eng.to_device(x)
    assert eng.HasNaN(t2) and not eng.HasInf(t2)
    x[4321] = -np.inf
    t3 = eng.to_device(x)
    assert eng.HasInf(t3) and not eng.HasNaN(t3)


def test_arena_oom_is_typed_error():
    e = Engine()
    e.Init(0, 1024)  # reserves 2*1024 + 512 + 256 bytes
    with pytest.raises(EngineError, match=r"allocated/reserved: \d+/\d+") as ei:
        e.Get(1 << 20)
    assert ei.value.code == 3
    p = e.Get(512)
    assert p % 32 == 0
    e.Put(p, 512)
    e.Close()
    e.destroy()
