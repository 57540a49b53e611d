"""Host mirror checks that need no GPU: exported symbols, the engine's argument
checks and error texts (cuda/utils.go:22-112, cuda/arith.go:17-49,
cuda/linalg.go:17-45), shape inference of the operators and the compiled tape
program (register reuse, flush placement)."""
import os
import re

import numpy as np
import pytest

from gorgonia_amd import configs, graph as G
from gorgonia_amd.engine import HOST_SYMBOLS, Engine, EngineError, Tensor, load_host

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_header_symbols_all_exported():
    hdr = open(os.path.join(ROOT, "include", "gorgonia_host.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = set(re.findall(r"\b(ghh_[a-z0-9_]+)\s*\(", hdr))
    lib = load_host()
    for name in sorted(declared):
        assert hasattr(lib, name), name
    assert declared == set(HOST_SYMBOLS), declared ^ set(HOST_SYMBOLS)


@pytest.fixture()
def eng():
    e = Engine()  # not initialised: every check below happens before any device call
    yield e
    e.destroy()


def T(shape, dtype=np.float32, mem=0x1000, **kw):
    return Tensor(mem, shape, dtype, **kw)


def test_binary_checks(eng):
    with pytest.raises(EngineError, match=r"Basic checks failed for Add: Shape mismatch. Expected \(4\). Got \(2\)"):
        eng.Add(T((2,)), T((4,)), unsafe=True)
    with pytest.raises(EngineError, match="TypeMismatch: a float64 and b float32"):
        eng.Gt(T((2,), np.float64), T((2,), np.float32), unsafe=True)
    with pytest.raises(EngineError, match="Unsupported Dtype for a"):
        eng.Mul(T((2,), np.int32), T((2,), np.int32), unsafe=True)
    with pytest.raises(EngineError, match="a requires an iterator"):
        eng.Sub(T((2,), needs_iterator=True), T((2,)), unsafe=True)
    # safe without reuse is an error; incr is unsupported (cuda/arith.go:47-49)
    with pytest.raises(EngineError, match="Impossible state: A reuse tensor must be passed in"):
        eng.Add(T((2,)), T((2,)))
    with pytest.raises(EngineError, match="Incr"):
        eng.Add(T((2,)), T((2,)), reuse=T((2,), mem=0x2000), incr=True)
    # reuse checks (cuda/utils.go:35-47)
    with pytest.raises(EngineError, match="Cannot use reuse: shape mismatch"):
        eng.Add(T((4,)), T((4,)), reuse=T((3,), mem=0x2000))
    with pytest.raises(EngineError, match="Cannot use reuse: TypeMismatch"):
        eng.Add(T((4,)), T((4,)), reuse=T((4,), np.float64, mem=0x2000))
    # the reference's Mod stops at "does not have the function" (no kernel in elembinop.cu:201-210);
    # here it goes through the same checks as every other binary method
    with pytest.raises(EngineError, match=r"Basic checks failed for Mod: Shape mismatch"):
        eng.Mod(T((2,)), T((4,)), unsafe=True)
    with pytest.raises(EngineError, match="b has to be a tensor.Memory"):
        eng.AddScalar(T((4,)), None, True, unsafe=True)
    # a valid call only records a command
    eng.Add(T((4,)), T((4,)), unsafe=True)
    eng.MulScalar(T((4,)), 0x3000, False, reuse=T((4,), mem=0x2000))
    assert eng.pending() == 2


def test_linalg_checks(eng):
    a, b, c = T((3, 4)), T((4, 5)), T((3, 5))
    with pytest.raises(EngineError, match="a isn't"):
        eng.MatMul(T((3, 4), managed=False), b, c)
    with pytest.raises(EngineError, match="same Dtype"):
        eng.MatMul(a, T((4, 5), np.float64), c)
    with pytest.raises(EngineError, match="Shape mismatch"):
        eng.MatMul(a, T((3, 5)), c)
    with pytest.raises(EngineError, match="Shape mismatch"):
        eng.MatMul(a, b, T((5, 3)))
    eng.MatMul(a, b, c)
    eng.MatMul(T((4, 3)).T(), b, c)          # transposed view of a (4,3) buffer
    eng.MatVecMul(a, T((4,)), T((3,)))
    eng.Outer(T((3,)), T((5,)), c)
    assert eng.pending() == 4
    # data orders (cuda/linalg.go:118-122): both operands row-major or both column-major
    with pytest.raises(EngineError, match="a does not have the same data order as b. a is RowMajor. b is ColMajor"):
        eng.MatMul(a, T((4, 5), col_major=True), c)
    eng.MatMul(T((3, 4), col_major=True), T((4, 5), col_major=True), T((3, 5), col_major=True))
    eng.MatVecMul(T((3, 4), col_major=True), T((4,)), T((3,)))
    assert eng.pending() == 6


def test_has_func_and_unknown_unary(eng):
    assert eng.HasFunc("elembinop.add_vv_f32") and eng.HasFunc("elemunaryop.tanh_f64")
    assert eng.HasFunc("elembinop.mod_vv_f32") and eng.HasFunc("elembinop.mod_sv_f64")
    with pytest.raises(EngineError, match="does not have the function"):
        eng.Unary("erf", T((4,)))
    assert eng.AllocAccessible() is False


def test_unimplemented_engine_methods_say_so(eng):
    """cuda/engine.go:93-99,130-132 panic with these words; here they are errors."""
    for call in (lambda: eng.Memset(0), lambda: eng.Memclr(0), lambda: eng.Accessible(0)):
        with pytest.raises(EngineError, match="not implemented"):
            call()
    assert eng.AllocFlags() == (True, True) and eng.WorksWith() is True
    eng.NonStdAlloc()


def test_elem_grid_size_matches_reference_rule(eng):
    """cuda/external.go:52-85 with the device limits defaulted (1024 threads)."""
    assert eng.ElemGridSize(100) == (1, 1, 1, 100, 1, 1)
    assert eng.ElemGridSize(1024) == (1, 1, 1, 1024, 1, 1)
    assert eng.ElemGridSize(1025) == (2, 1, 1, 1024, 1, 1)
    assert eng.ElemGridSize(1 << 24) == (16384, 1, 1, 1024, 1, 1)


def test_read_takes_the_node_dtype():
    """A float64 value lands in a float64 host array; a mismatched request is refused
    (the machine copies bytes, so a float32 array would be overrun)."""
    g = G.NewGraph()
    x = G.NewTensor(g, np.zeros((4, 6), np.float64))
    w = G.NewTensor(g, np.zeros((6, 3), np.float64))
    y = G.Mul(x, w)
    assert y.Dtype() == np.float64 and G.Read(y).dtype == np.float64
    with pytest.raises(EngineError, match="holds float64"):
        G.Read(y, dtype=np.float32)
    z = G.Rectify(G.NewTensor(g, np.zeros((2, 2), np.float32)))
    assert G.Read(z).dtype == np.float32 and G.Read(z, np.float32).shape == (2, 2)


def test_shape_inference_and_errors():
    g = G.NewGraph()
    x = G.NewTensor(g, np.zeros((2, 3, 8, 8), np.float32))
    w = G.NewTensor(g, np.zeros((5, 3, 3, 3), np.float32))
    assert G.Conv2d(x, w, (3, 3), (1, 1), (1, 1), (1, 1)).Shape() == (2, 5, 8, 8)
    assert G.Conv2d(x, w, (3, 3), (0, 0), (2, 2), (1, 1)).Shape() == (2, 5, 3, 3)
    assert G.MaxPool2D(x, (2, 2), (0, 0), (2, 2)).Shape() == (2, 3, 4, 4)
    assert G.MaxPool2D(x, (2, 2), (1, 0, 1, 0), (1, 1)).Shape() == (2, 3, 8, 8)
    with pytest.raises(EngineError, match="Cannot use strides of less than or equal 0"):
        G.Conv2d(x, w, (3, 3), (1, 1), (0, 1), (1, 1))
    with pytest.raises(EngineError, match="Cannot use padding of less than 0"):
        G.MaxPool2D(x, (2, 2), (-1, 0), (2, 2))
    with pytest.raises(EngineError, match="Impossible height/kernel/pad combination"):
        G.MaxPool2D(x, (9, 2), (0, 0), (1, 1))
    with pytest.raises(EngineError, match="im should have 4 dims, got 2 dims"):
        G.Conv2d(G.NewTensor(g, np.zeros((2, 3), np.float32)), w, (3, 3))
    a = G.NewTensor(g, np.zeros((4, 6), np.float32))
    b = G.NewTensor(g, np.zeros((1, 6), np.float32))
    assert G.BroadcastAdd(a, b).Shape() == (4, 6)
    assert G.Mul(a, G.NewTensor(g, np.zeros((6, 2), np.float32))).Shape() == (4, 2)
    assert G.Mul(a, G.NewTensor(g, np.zeros((5, 6), np.float32)), transB=True).Shape() == (4, 5)
    with pytest.raises(EngineError, match="Shape mismatch"):
        G.Add(a, b)
    assert G.Reshape(a, (2, 12)).Shape() == (2, 12)
    with pytest.raises(EngineError, match="invalid runningMean shape"):
        G.BatchNorm(x, None, None, G.NewTensor(g, np.zeros((2, 2), np.float32)),
                    G.NewTensor(g, np.zeros(3, np.float32)))


def test_tape_program_keeps_live_values():
    """Config 2: z feeds both Tanh and Pow, so Sigmoid may overwrite its dead
    input but Tanh must not overwrite z (regalloc.go:211-243)."""
    inp = configs.elementwise_inputs(8)
    g, outs = configs.build_elementwise(inp)
    m = G.NewTapeMachine(g, compile_only=True)
    prog = m.program()
    lines = [l for l in prog.splitlines() if "execOp" in l]
    assert len(lines) == 5
    assert "elembin.mul [unsafe]" in lines[0]          # x*y overwrites x (dead afterwards)
    assert "broadcast.add" in lines[1]
    assert "elemunary.sigmoid [unsafe]" in lines[2]    # its input is dead
    assert "elemunary.tanh [reuse]" in lines[3]        # z is still needed by Pow
    assert "elembin.pow [reuse]" in lines[4]           # z is read by the host afterwards
    # one flush, in front of the host reads
    assert prog.count("flush") == 1
    assert prog.index("flush") < prog.index("read")
    m.Close()


def test_tape_program_convnet_fusion():
    inp = configs.convnet_inputs(2)
    g, _ = configs.build_convnet(inp)
    m = G.NewTapeMachine(g, compile_only=True, fuse_activations=True)
    assert m.fused == 9  # 4 activations, the three pools, the softmax, and the first layer into the second
    prog = m.program()
    assert prog.count("conv2d+rectify+maxpool2d+conv2d+rectify+maxpool2d") == 1   # layers 0 and 1: one command
    assert prog.count("execOp") == 4 and prog.count(" rectify") == 0
    assert prog.count("maxpool2d") == 3 and prog.count("softmax") == 1
    m.Close()
    # a first layer whose result something else reads as well stays a command of its own
    g3 = G.NewGraph()
    x = G.NewTensor(g3, inp["x"], True)
    h = G.MaxPool2D(G.Rectify(G.Conv2d(x, G.NewTensor(g3, inp["w0"], True), (3, 3), (1, 1), (1, 1), (1, 1))), (2, 2), (0, 0), (2, 2))
    y = G.Conv2d(h, G.NewTensor(g3, inp["w1"], True), (3, 3), (1, 1), (1, 1), (1, 1))
    G.Read(y)
    G.Read(h)
    m3 = G.NewTapeMachine(g3, compile_only=True, fuse_activations=True)
    assert m3.program().count("conv2d+rectify+maxpool2d+conv2d") == 0 and m3.program().count("execOp") == 2
    m3.Close()
    g2, _ = configs.build_convnet(inp)
    m2 = G.NewTapeMachine(g2, compile_only=True)
    assert m2.program().count(" rectify") == 4
    m2.Close()


def test_apply_refuses_functions_the_engine_does_not_have():
    """Operator kind, binary function and solver numbers are range-checked when the
    node is made (no name table is ever indexed with them); Mod is a real entry."""
    from gorgonia_amd import _ffi
    g = G.NewGraph()
    a = G.NewTensor(g, np.zeros((4, 6), np.float32))
    b = G.NewTensor(g, np.zeros((4, 6), np.float32))
    for kind, fn in ((G.K_ELEMBIN, 12), (G.K_ELEMBIN, -1), (G.K_BCAST, 99), (G.K_SOLVER, 3), (26, 0), (-1, 0)):
        with pytest.raises(EngineError) as ei:
            g.apply(kind, [a, b], fn=fn)
        assert ei.value.code == _ffi.GH_ENOFUNC, (kind, fn, str(ei.value))
    y = g.apply(G.K_ELEMBIN, [a, b], fn=_ffi.BIN_FN["mod"])
    G.Read(y)
    m = G.NewTapeMachine(g, compile_only=True)
    assert "elembin.mod" in m.program()
    m.Close()


def test_conv1d_is_conv2d_with_unit_height():
    g = G.NewGraph()
    x = G.NewTensor(g, np.zeros((2, 3, 1, 40), np.float32))
    w = G.NewTensor(g, np.zeros((5, 3, 1, 3), np.float32))
    assert G.Conv1d(x, w, 3, 1, 1, 1).Shape() == (2, 5, 1, 40)
    assert G.Conv1d(x, w, 3, 0, 2, 1).Shape() == (2, 5, 1, 19)
    assert G.Conv1d(x, w, 3, 2, 1, 2).Shape() == (2, 5, 1, 40)
    m = G.NewTapeMachine(g, compile_only=True)
    assert "conv2d" in m.program()
    m.Close()


def test_borrowed_reads_in_the_program():
    """ReadBorrowed: a value only the host reads is written by its kernel into the machine's
    pinned buffer (allocHost), one with other readers is staged by a copy inside the segment
    (stageOut), both whatever their size; an ordinary Read past 8 MB is copied after the flush
    instead.  Nothing but a borrowed read has a buffer to lend."""
    def build(read):
        g = G.NewGraph()
        a = G.NewTensor(g, np.zeros((3, 1024, 1024), np.float32))
        b = G.NewTensor(g, np.zeros((3, 1024, 1024), np.float32))
        s = G.Add(a, b)
        t = G.HadamardProd(s, b)
        return g, a, read(s), read(t)
    g, a, rs, rt = build(G.ReadBorrowed)
    m = G.NewTapeMachine(g, compile_only=True)
    prog = m.program()
    assert "allocHost node 3" in prog and "stageOut node 2" in prog
    assert prog.index("stageOut") < prog.index("flush") < prog.index("read node 2")
    with pytest.raises(EngineError):
        m.value(G.BorrowedRead(a))
    m.Close()
    g2, _, _, _ = build(G.Read)
    m2 = G.NewTapeMachine(g2, compile_only=True)
    assert "allocHost" not in m2.program() and "stageOut" not in m2.program()
    m2.Close()
    with pytest.raises(EngineError):
        g.lib.ghh_graph_read_borrowed(g.h, 99) and g._check(g.lib.ghh_graph_read_borrowed(g.h, 99))


def test_pooled_rectify_is_folded_only_when_nothing_else_reads_it():
    """FuseActivations folds Rectify into the pool and both gradients (a = Rectify(z); MaxPool2D(a);
    RectifyDiff(z, MaxPool2DDiff(a, g))) only when a and the pooling gradient have no other reader, the
    two pooling operators agree on their geometry and both gradients hang off the same z."""
    def build(read_a=False, other_geometry=False, read_da=False, other_z=False):
        g = G.NewGraph()
        x = G.NewTensor(g, np.zeros((2, 3, 8, 8), np.float32))
        w = G.NewTensor(g, np.zeros((4, 3, 3, 3), np.float32), resident=True)
        z = G.Conv2d(x, w, (3, 3), (1, 1), (1, 1), (1, 1))
        a = G.Rectify(z)
        p = G.MaxPool2D(a, (2, 2), (0, 0), (2, 2))
        G.Read(p)
        grad = G.NewTensor(g, np.zeros((2, 4, 4, 4), np.float32))
        da = G.MaxPool2DDiff(a, grad, (2, 2), (0, 0), (1, 1) if other_geometry else (2, 2)) if not other_geometry else \
            G.MaxPool2DDiff(a, G.NewTensor(g, np.zeros((2, 4, 7, 7), np.float32)), (2, 2), (0, 0), (1, 1))
        z2 = G.Conv2d(x, w, (3, 3), (1, 1), (1, 1), (1, 1)) if other_z else z
        G.Read(G.RectifyDiff(z2, da))
        if read_a:
            G.Read(a)
        if read_da:
            G.Read(da)
        return g
    m = G.NewTapeMachine(build(), compile_only=True, fuse_activations=True)
    assert m.fused == 2 and m.program().count("rectify+maxpool2d") == 2 and "rectifyDiff" not in m.program()
    m.Close()
    for kw in (dict(read_a=True), dict(other_geometry=True), dict(read_da=True), dict(other_z=True)):
        m = G.NewTapeMachine(build(**kw), compile_only=True, fuse_activations=True)
        # (with a z of its own the activation folds into its convolution instead, the ordinary way)
        assert m.fused == (1 if "other_z" in kw else 0) and ("conv2d+rectify" in m.program()) == ("other_z" in kw), kw
        assert "rectify+maxpool2d" not in m.program() and "rectifyDiff" in m.program(), kw
        m.Close()


def test_pool_is_folded_into_a_convolution_whose_result_is_kept():
    """Graph::fuse_kept_conv: where a convolution's result has other readers than its 2x2 pool (a backward pass,
    a host read) and the kernel for the shape stores both, the pool's node runs the convolution and the
    convolution's node keeps its register without an instruction; not when something reads the result in
    between, and not for shapes whose kernel cannot keep it."""
    def build(C=32, between=False):
        g = G.NewGraph()
        x = G.NewTensor(g, np.zeros((2, C, 8, 8), np.float32))
        w = G.NewTensor(g, np.zeros((16, C, 3, 3), np.float32), resident=True)
        z = G.Conv2d(x, w, (3, 3), (1, 1), (1, 1), (1, 1))
        if between:
            G.Read(G.Rectify(z))
        p = G.MaxPool2D(z, (2, 2), (0, 0), (2, 2))
        G.Read(p)
        G.Read(z)
        return g
    m = G.NewTapeMachine(build(), compile_only=True, fuse_activations=True)
    prog = m.program()
    assert m.fused == 1 and prog.count("conv2d(kept)+maxpool2d") == 1 and prog.count("execOp") == 1, prog
    assert "alloc node 2" in prog and "execOp node 2" not in prog and "execOp node 3" in prog   # z: a register, no instruction
    m.Close()
    for kw in (dict(between=True), dict(C=3)):
        m = G.NewTapeMachine(build(**kw), compile_only=True, fuse_activations=True)
        assert "conv2d(kept)" not in m.program() and " maxpool2d" in m.program(), kw
        m.Close()


def test_pooling_query_over_random_geometries():
    """gh_conv2d_can_pool runs every 3x3 kernel's planner on the host.  Over a few thousand random
    geometries (channel counts around every kernel's limits, images from 3x3 to 500x500) it must
    answer 0 or 1 without a device, say no to everything the pool cannot follow (other kernel sizes,
    strides, dilation, float64, results smaller than a window) and give one answer per geometry."""
    from gorgonia_amd import _ffi, device as D
    lib = _ffi.load()
    rng = np.random.default_rng(123)
    yes = kept = folded = 0
    for it in range(4000):
        B = int(rng.choice([1, 2, 3, 8, 16, 128, 130]))
        C = int(rng.choice([1, 2, 3, 4, 5, 8, 12, 16, 24, 32, 48, 64, 96, 128, 256, 512, 1000]))
        F = int(rng.choice([1, 5, 16, 17, 32, 40, 64, 128, 425, 1024]))
        H = int(rng.choice([3, 4, 7, 13, 14, 16, 17, 26, 28, 52, 104, 208, 416, 500]))
        W = int(rng.choice([3, 4, 7, 13, 14, 16, 17, 26, 28, 52, 104, 208, 416, 500]))
        k = int(rng.choice([3, 3, 3, 1, 5]))
        pad = int(rng.choice([0, 1, 1, 2]))
        stride = int(rng.choice([1, 1, 1, 2]))
        dil = int(rng.choice([1, 1, 1, 2]))
        if H + 2 * pad < dil * (k - 1) + 1 or W + 2 * pad < dil * (k - 1) + 1:
            continue
        if B * C * H * W >= 2 ** 31 or B * F * H * W >= 2 ** 31:
            continue
        cmd = D.cmd_conv2d(0x1000, 0x2000, 0x3000, B, C, H, W, F, k, k, (pad, pad), (stride, stride), (dil, dil))
        a = lib.gh_conv2d_can_pool(cmd)
        assert a in (0, 1) and a == lib.gh_conv2d_can_pool(cmd)
        oh = (H + 2 * pad - (dil * (k - 1) + 1)) // stride + 1
        ow = (W + 2 * pad - (dil * (k - 1) + 1)) // stride + 1
        if a:
            yes += 1
            assert k == 3 and stride == 1 and dil == 1 and oh >= 2 and ow >= 2, (B, C, H, W, F, k, pad, stride, dil)
        f64 = D.cmd_conv2d(0x1000, 0x2000, 0x3000, B, C, H, W, F, k, k, (pad, pad), (stride, stride), (dil, dil),
                           dtype=_ffi.F64)
        assert lib.gh_conv2d_can_pool(f64) == 0
        # the folds that only the small-image kernels offer: a kept result goes with a pool, a folded first layer
        # with 32 channels on small images; both queries answer without a device and never for float64
        keep, pre = lib.gh_conv2d_can_keep(cmd), lib.gh_conv2d_can_pre(cmd)
        assert keep in (0, 1) and pre in (0, 1)
        if keep:
            kept += 1
            assert a == 1 and C in (1, 32, 64) and H <= 64 and W <= 64, (B, C, H, W, F, k, pad, stride, dil)
        if pre:
            folded += 1
            assert C == 32 and k == 3 and stride == 1 and dil == 1 and pad <= 1 and 4 <= W <= 16 and H <= 16, (B, C, H, W, F, pad)
        assert lib.gh_conv2d_can_keep(f64) == 0 and lib.gh_conv2d_can_pre(f64) == 0
    assert yes > 300 and kept > 20 and folded > 5, (yes, kept, folded)


def test_broadcast_patterns_shapes_and_errors():
    """Broadcast (broadcast.go:69-129) with explicit patterns, graph construction only: the result shapes of the
    reference's table and its two error cases (operations_broadcast_test.go:147-164: an axis the other operand
    does not have; repeats that do not reach the other operand's shape)."""
    from gorgonia_amd import graph as G
    from gorgonia_amd.engine import EngineError

    def shapes(ashp, bshp, left, right):
        g = G.NewGraph()
        a, b = G.NewTensor(g, np.zeros(ashp)), G.NewTensor(g, np.zeros(bshp))
        return G.BroadcastAdd(a, b, left, right).Shape()

    assert shapes((2,), (2, 2), [1], None) == (2, 2)
    assert shapes((2, 2), (2,), None, [1]) == (2, 2)
    assert shapes((1, 2), (2, 2), [0], None) == (2, 2)
    assert shapes((2, 1), (1, 3), [1], [0]) == (2, 3)
    assert shapes((), (3, 4), [0, 1], None) == (3, 4)          # a scalar is all ones (shape.go:50-53)
    assert shapes((4,), (3, 4, 5), [0, 2], None) == (3, 4, 5)  # the operand's extent takes the free slot
    with pytest.raises(EngineError, match="axis 2 of b"):
        shapes((2, 1), (2, 2), [2], None)                      # "rowvec-mat: wrong axis"
    with pytest.raises(EngineError, match="Shape mismatch"):
        shapes((2, 4), (1, 2), None, [0, 1])                   # "impossible mat-mat"
    with pytest.raises(EngineError):
        shapes((3,), (2, 2), [1], None)                        # three values do not fill (?, 1) of a (2, 2)


def test_operands_of_different_dtypes_are_refused_when_the_graph_is_built():
    """The reference's type inference fails such an expression at construction ("cannot be unified"); here Apply does."""
    from gorgonia_amd import graph as G
    from gorgonia_amd.engine import EngineError
    g = G.NewGraph()
    a32, a64 = G.NewTensor(g, np.ones((2, 3), np.float32)), G.NewTensor(g, np.ones((2, 3), np.float64))
    for build in (lambda: G.Add(a32, a64), lambda: G.Mul(a32, G.NewTensor(g, np.ones((3, 2), np.float64))),
                  lambda: G.BroadcastAdd(a64, G.NewTensor(g, np.ones((1, 3), np.float32))),
                  lambda: G.Conv2d(G.NewTensor(g, np.ones((1, 1, 4, 4), np.float64)),
                                   G.NewTensor(g, np.ones((2, 1, 3, 3), np.float32)), (3, 3))):
        with pytest.raises(EngineError, match="cannot be unified"):
            build()
    assert G.Add(a64, a64).Dtype() == np.float64


def test_new_tensor_refuses_shapes_the_machine_cannot_hold():
    from gorgonia_amd import graph as G
    from gorgonia_amd.engine import EngineError
    g = G.NewGraph()
    with pytest.raises(EngineError, match="positive"):
        G.NewTensor(g, np.ones((0, 3), np.float32))
    with pytest.raises(EngineError, match="8 dimensions"):
        G.NewTensor(g, np.ones((1,) * 9, np.float32))
    assert G.NewTensor(g, np.ones((1,) * 8, np.float32)).Shape() == (1,) * 8
    assert G.NewScalar(g, 2.0).Shape() == ()


def test_mul_follows_the_reference_dispatch():
    """operations.go:52-74: a scalar operand makes a HadamardProd, two vectors the inner product (a scalar),
    vector x matrix the product with the transposed matrix; anything else is refused."""
    g = G.NewGraph()
    v6, m23, v2, v3 = (G.NewTensor(g, np.zeros(s, np.float32)) for s in ((6,), (2, 3), (2,), (3,)))
    s = G.NewScalar(g, 2.0)
    assert G.Mul(s, m23).Shape() == (2, 3) and G.Mul(m23, s).Shape() == (2, 3) and G.Mul(s, s).Shape() == ()
    assert G.Mul(v6, v6).Shape() == ()
    assert G.Mul(v2, m23).Shape() == (3,)
    assert G.Mul(m23, v3).Shape() == (2,)
    with pytest.raises(G.EngineError):
        G.Mul(v2, v3)
    with pytest.raises(G.EngineError):
        G.Mul(v3, m23)          # 3 against the 2 rows of the matrix
    with pytest.raises(G.EngineError):
        G.Mul(G.NewTensor(g, np.zeros((2, 2, 2), np.float32)), m23)


def test_comparisons_take_ret_same_and_div_is_hadamard_div():
    """api_gen.go:80-127 (retSame), operations.go:114-122 (Div)."""
    g = G.NewGraph()
    a, b = G.NewTensor(g, np.zeros((2, 3), np.float32)), G.NewTensor(g, np.ones((2, 3), np.float32))
    for cmp in (G.Lt, G.Lte, G.Gt, G.Gte, G.Eq, G.Ne):
        assert cmp(a, b, True).Shape() == (2, 3)
        with pytest.raises(G.EngineError):
            cmp(a, b, False)
    assert G.Div(a, b).Shape() == (2, 3) and G.Div(a, G.NewScalar(g, 2.0)).Shape() == (2, 3)
    with pytest.raises(G.EngineError):
        G.Div(a, G.NewTensor(g, np.ones((3, 2), np.float32)))


def test_softmax_takes_the_last_axis_only():
    g = G.NewGraph()
    a = G.NewTensor(g, np.zeros((4, 6), np.float32))
    assert G.SoftMax(a).Shape() == G.SoftMax(a, -1).Shape() == G.SoftMax(a, 1).Shape() == (4, 6)
    with pytest.raises(G.EngineError):
        G.SoftMax(a, 0)


def test_watch_options_reach_the_machine():
    """WithNaNWatch / WithInfWatch (vm.go:138-166) are options of both machines; the C entry refuses a null handle."""
    from gorgonia_amd import engine as E
    assert G.WithNaNWatch() == {"watch_nan": True} and G.WithInfWatch() == {"watch_inf": True}
    assert E.load_host().ghh_tape_watch(None, 1, 1) != 0
    g = G.NewGraph()
    G.Read(G.Neg(G.NewTensor(g, np.zeros((2, 2), np.float32))))
    m = G.NewTapeMachine(g, G.WithNaNWatch(), G.WithInfWatch(), compile_only=True)
    assert "neg" in m.program()
