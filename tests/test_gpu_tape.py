"""GPU parity of whole forward passes on the tape machine against the CPU
oracle's forward pass of the same seeded configuration, plus the segment
batching, hipGraph replay and Reset semantics."""
import numpy as np
import pytest

from gorgonia_amd import configs, graph as G, synth
from oracle import forward as F
from tests.util import assert_bits_equal, rel_frobenius, ulp_diff

pytestmark = pytest.mark.gpu


def run_once(build, inp, **kw):
    g, outs = build(inp)
    m = G.NewTapeMachine(g, **kw)
    m.RunAll()
    res = {k: v.copy() for k, v in outs.items()}
    return m, outs, res


def test_mlp_forward(ctx):
    inp = configs.mlp_inputs(256)
    m, _, res = run_once(configs.build_mlp, inp)
    want = F.mlp(inp)
    assert rel_frobenius(res["out"], want) <= 1e-5
    assert np.allclose(res["out"].sum(axis=1), 1.0, atol=1e-5)
    assert m.segments() == 1
    m.Close()


def test_mlp_dense_layers_fold_bias_activation_and_softmax(ctx):
    """Mul -> BroadcastAdd(bias) -> Rectify / SoftMax of every dense layer becomes one product
    command; the stored bits are those of the separate operators (non-zero biases here)."""
    inp = configs.mlp_inputs(64)
    for i, nb in enumerate((300, 100, 10)):
        inp[f"b{i}"] = synth.normal(900 + i, (1, nb), 0.0, 0.5)
    m1, _, r1 = run_once(configs.build_mlp, inp)
    m2, _, r2 = run_once(configs.build_mlp, inp, fuse_activations=True)
    assert rel_frobenius(r1["out"], F.mlp(inp)) <= 1e-5
    assert_bits_equal(r1["out"], r2["out"], "fused dense layers change nothing")
    assert m2.fused == 6  # three biases, two activations, the softmax
    prog = m2.program()
    assert prog.count("matmul+bias+rectify") == 2 and prog.count("matmul+bias+softmax") == 1
    m1.Close(); m2.Close()


def test_elementwise_chain_small_and_full(ctx):
    for n in (64, 1024):
        inp = configs.elementwise_inputs(n)
        m, _, res = run_once(configs.build_elementwise, inp)
        want = F.elementwise(inp)
        assert ulp_diff(res["z"], want["z"]).max() <= 2
        assert ulp_diff(res["tanh"], want["tanh"]).max() <= 4  # tanh of a z that may differ by 2 ulp
        assert_bits_equal(res["pow"], (res["z"] * res["z"]), "pow(z,2) == z*z")
        m.Close()


def test_convnet_forward_fused_and_unfused(ctx):
    inp = configs.convnet_inputs(32)
    want = F.convnet(inp)
    m1, _, r1 = run_once(configs.build_convnet, inp)
    m2, _, r2 = run_once(configs.build_convnet, inp, fuse_activations=True)
    assert rel_frobenius(r1["out"], want) <= 1e-5
    assert_bits_equal(r1["out"], r2["out"], "fused activations change nothing")
    assert m2.fused == 9  # 4 activations, the three pools, the softmax, the first layer into the second
    m1.Close(); m2.Close()


def test_yolo_shaped_forward_reduced(ctx):
    """Configuration 5 at batch 1, 96x96 (every layer type, the stride-1 pool included)."""
    inp = configs.yolo_inputs(1, 96)
    want = F.yolo(inp)
    m, _, res = run_once(configs.build_yolo, inp, fuse_activations=True)
    assert res["out"].shape == want.shape == (1, 425, 3, 3)
    assert rel_frobenius(res["out"], want) <= 1e-5
    # conv -> batchnorm -> leakyrelu (-> maxpool where it is 2x2 stride 2) run as
    # single commands; the folded program stores the bits of the plain one
    prog = m.program()
    assert prog.count("conv2d+batchnorm(eval)+leakyrelu") == 7
    assert prog.count("conv2d+batchnorm(eval)+leakyrelu+maxpool2d") == 5
    assert " batchnorm" not in prog and " leakyrelu" not in prog
    m.Close()
    m0, _, plain = run_once(configs.build_yolo, inp)
    assert "conv2d+" not in m0.program()
    assert_bits_equal(res["out"], plain["out"], "folded yolo-shaped forward == plain")
    m0.Close()


def test_graph_replay_matches_eager_every_time(ctx):
    """Segments captured into a hipGraph: replays after the first, with host
    work and synchronisation in between, must equal the eager result."""
    inp = configs.convnet_inputs(16)
    m0, _, eager = run_once(configs.build_convnet, inp)
    m0.Close()
    g, outs = configs.build_convnet(inp)
    m = G.NewTapeMachine(g, graph_replay=True)
    for it in range(6):
        outs["out"][...] = -1.0
        m.RunAll()
        assert_bits_equal(outs["out"], eager["out"], f"replay iteration {it}")
        _ = np.linalg.norm(outs["out"])  # unrelated host work between replays
    assert m.graph_launches() >= 4
    # new input values flow through the replayed graph (same addresses, new data)
    x2 = inp["x"][::-1].copy()
    inp2 = dict(inp, x=x2)
    m1, _, eager2 = run_once(configs.build_convnet, inp2)
    m1.Close()
    G.Let(G.Node(g, 0), x2)
    m.RunAll()
    assert_bits_equal(outs["out"], eager2["out"], "replay with rebound input")
    m.Close()


def test_reset_gives_same_addresses_and_results(ctx):
    inp = configs.mlp_inputs(64)
    g, outs = configs.build_mlp(inp)
    m = G.NewTapeMachine(g)
    m.RunAll()
    first = outs["out"].copy()
    addr = [m.register_address(G.Node(g, i)) for i in range(8)]
    m.Reset()
    m.RunAll()
    assert [m.register_address(G.Node(g, i)) for i in range(8)] == addr
    assert_bits_equal(outs["out"], first, "after Reset")
    m.RunAll()  # without Reset: registers are re-acquired in the same order
    assert_bits_equal(outs["out"], first, "second run without Reset")
    m.Close()


def test_one_submit_per_segment(ctx):
    """The whole forward pass is one tape segment: one gh_submit for all
    operators (the H2D copies and the final flush are separate calls)."""
    inp = configs.convnet_inputs(8)
    g, outs = configs.build_convnet(inp)
    m = G.NewTapeMachine(g)
    m.RunAll()
    s0 = m.submit_calls()
    m.RunAll()
    assert m.submit_calls() - s0 == 1
    assert m.segments() == 1
    m.Close()


def test_reupload_mode_matches_resident(ctx):
    """Inputs uploaded on every run (what the reference does with every input,
    vm_tape_cuda.go:220-243) travel inside the segment: all uploads sit at the head of the
    program, go through pinned buffers, and a run stays one gh_submit (eager) or one graph
    launch (replayed) - whatever the number of inputs."""
    inp = configs.convnet_inputs(8)
    m1, _, r1 = run_once(configs.build_convnet, inp)
    for kw in (dict(), dict(reupload_resident=True), dict(graph_replay=True, fuse_activations=True),
               dict(graph_replay=True, fuse_activations=True, reupload_resident=True)):
        g, outs = configs.build_convnet(inp, resident=False)
        m2 = G.NewTapeMachine(g, **kw)
        prog = [l.split()[1] for l in m2.program().splitlines()[1:] if "\t" in l]
        first_op = prog.index("execOp")
        assert "devTrans" not in prog[first_op:], "an upload after the first operator splits the segment"
        assert prog.count("devTrans") == 6
        for it in range(4):
            outs["out"][...] = -1.0
            s0, l0 = m2.submit_calls(), m2.graph_launches()
            m2.RunAll()
            crossings = (m2.submit_calls() - s0) + (m2.graph_launches() - l0)
            assert crossings <= 2, f"{kw} run {it}: {crossings} submits/launches"
            assert m2.segments() == 1
            assert_bits_equal(outs["out"], r1["out"], f"re-uploaded inputs {kw} run {it}")
        if kw.get("graph_replay"):
            assert m2.graph_launches() >= 2 and m2.submit_calls() - s0 == 0
        # a new value bound to an input reaches the device on the next run
        x2 = inp["x"][::-1].copy()
        G.Let(G.Node(g, 0), x2)
        m2.RunAll()
        m3, _, r3 = run_once(configs.build_convnet, dict(inp, x=x2))
        assert_bits_equal(outs["out"], r3["out"], f"rebound input {kw}")
        m3.Close()
        m2.Close()
    m1.Close()


def test_with_engine_machines_share_one_arena(ctx):
    """NewTapeMachine(g, WithEngine(e)) (vm.go:318-329): two machines run one after the
    other on the caller's engine, give the results of machines with engines of their
    own, hand their registers back on Close and leave the engine open."""
    from gorgonia_amd.engine import Engine, EngineError
    inp_a = configs.convnet_inputs(8)
    inp_b = configs.mlp_inputs(64)
    ma, _, want_a = run_once(configs.build_convnet, inp_a)
    ma.Close()
    mb, _, want_b = run_once(configs.build_mlp, inp_b)
    mb.Close()

    e = Engine()
    ga, outs_a = configs.build_convnet(inp_a)
    with pytest.raises(EngineError, match="not initialised"):
        G.NewTapeMachine(ga, G.WithEngine(e))
    e.Init(0, 256 << 20)
    m1 = G.NewTapeMachine(ga, G.WithEngine(e), graph_replay=True)
    gb, outs_b = configs.build_mlp(inp_b)
    m2 = G.NewTapeMachine(gb, G.WithEngine(e))
    for it in range(3):
        outs_a["out"][...] = -1.0
        m1.RunAll()
        assert_bits_equal(outs_a["out"], want_a["out"], f"shared engine, convnet run {it}")
        outs_b["out"][...] = -1.0
        m2.RunAll()
        assert_bits_equal(outs_b["out"], want_b["out"], f"shared engine, mlp run {it}")
    # the two machines hold different arena memory for their resident inputs (the weights)
    held_a = {m1.register_address(G.Node(ga, i)) for i in (1, 5, 9, 14, 17)}
    held_b = {m2.register_address(G.Node(gb, i)) for i in (1, 2)}
    assert 0 not in held_a | held_b and not (held_a & held_b)
    m1.Reset()
    m1.RunAll()
    assert_bits_equal(outs_a["out"], want_a["out"], "shared engine, after Reset")
    m1.Close()
    m2.RunAll()   # the other machine is untouched by the first one's Close
    assert_bits_equal(outs_b["out"], want_b["out"], "shared engine, after the other machine closed")
    m2.Close()
    # the engine is still open and its arena is whole again: a machine that needs most of it fits
    gc, outs_c = configs.build_convnet(inp_a)
    m3 = G.NewTapeMachine(gc, G.WithEngine(e))
    m3.RunAll()
    assert_bits_equal(outs_c["out"], want_a["out"], "shared engine, third machine")
    m3.Close()
    # an arena too small for the program is refused at init with the allocator's error code
    small = Engine()
    small.Init(0, 4096)
    gd, _ = configs.build_convnet(inp_a)
    with pytest.raises(EngineError, match="arena has"):
        G.NewTapeMachine(gd, G.WithEngine(small))
    small.Close(); small.destroy()
    e.Close(); e.destroy()


def test_conv1d_on_the_tape(ctx):
    """nnops.Conv1d (ops/nn/api_cuda.go:18-20) is Conv2d over a height-1 image."""
    from oracle import binding as O
    x = synth.uniform(11, (4, 8, 1, 96), -1, 1)
    w = synth.he_normal(12, (12, 8, 1, 5))
    for pad, stride, dil in ((2, 1, 1), (0, 2, 1), (4, 1, 2), (3, 3, 2)):
        g = G.NewGraph()
        y = G.Conv1d(G.NewTensor(g, x), G.NewTensor(g, w, resident=True), 5, pad, stride, dil)
        out = G.Read(y)
        m = G.NewTapeMachine(g)
        m.RunAll()
        want = O.conv2d_direct_f64(x, w, (0, pad), (1, stride), (1, dil))
        assert out.shape == want.shape == (4, 12, 1, (96 + 2 * pad - (dil * 4 + 1)) // stride + 1)
        assert rel_frobenius(out, want) <= 1e-5, (pad, stride, dil)
        m.Close()


def test_maxpool1d_on_the_tape(ctx):
    """MaxPool1D (nn.go:378-380) is MaxPool2D over a height-1 image: the oracle's bits, and behind a Conv1d
    whose result it may take over."""
    from oracle import binding as O
    x = synth.uniform(13, (3, 8, 1, 97), -1, 1)
    for kernel, pad, stride in ((2, 0, 2), (3, 1, 2), (4, 2, 3), (2, 1, 1)):
        g = G.NewGraph()
        out = G.Read(G.MaxPool1D(G.NewTensor(g, x), kernel, pad, stride))
        m = G.NewTapeMachine(g, fuse_activations=True)
        m.RunAll()
        want = O.maxpool2d(x, (1, kernel), (0, pad), (1, stride))
        assert out.shape == want.shape and want.shape[2] == 1
        assert_bits_equal(out, want, f"{kernel} {pad} {stride}")
        m.Close()
    w = synth.he_normal(14, (12, 8, 1, 3))
    res = []
    for kw in (dict(), dict(fuse_activations=True)):
        g = G.NewGraph()
        y = G.Rectify(G.Conv1d(G.NewTensor(g, x), G.NewTensor(g, w, resident=True), 3, 1, 1, 1))
        out = G.Read(G.MaxPool1D(y, 2, 0, 2))
        m = G.NewTapeMachine(g, **kw)
        m.RunAll()
        res.append(out.copy())
        m.Close()
    assert res[0].shape == (3, 12, 1, 48)
    assert_bits_equal(res[1], res[0], "folded against plain")


def test_borrowed_reads_hold_what_read_copies(ctx):
    """ReadBorrowed leaves a value in the machine's pinned buffer; Read copies it out.  Same bits,
    for a value only the host reads (written there by its kernel), one that other nodes also
    read (staged by a copy in the segment), a reshaped view and one past the staging limit of
    ordinary reads; on plain runs, replayed runs and after the input changes."""
    a0 = synth.uniform(31, (3, 1024, 1024), -1, 1)      # 12 MB: beyond the 8 MB of a staged Read
    b0 = synth.uniform(32, (3, 1024, 1024), -1, 1)

    def build(borrow):
        g = G.NewGraph()
        a, b = G.NewTensor(g, a0.copy()), G.NewTensor(g, b0, resident=True)
        s = G.Add(a, b)            # read by the host and by the next two nodes
        t = G.HadamardProd(s, b)   # only the host reads it: 12 MB
        u = G.Reshape(G.Tanh(s), (3 * 1024, 1024))
        small = G.Neg(G.NewTensor(g, synth.uniform(33, (7, 5), -1, 1)))   # 140 bytes
        rd = G.ReadBorrowed if borrow else G.Read
        return g, a, {"s": rd(s), "t": rd(t), "u": rd(u), "small": rd(small)}

    for mode in (False, True):
        g0, in0, want = build(False)
        m0 = G.NewTapeMachine(g0, graph_replay=mode)
        g1, in1, got = build(True)
        m1 = G.NewTapeMachine(g1, graph_replay=mode)
        addr = None
        for it in range(4):
            if it == 2:   # a new input value: both graphs see it
                fresh = synth.uniform(40, a0.shape, -2, 2)
                G.Let(in0, fresh); G.Let(in1, fresh)
            m0.RunAll(); m1.RunAll()
            views = {k: m1.value(v) for k, v in got.items()}
            for k in want:
                assert views[k].shape == want[k].shape
                assert_bits_equal(views[k], want[k], f"borrowed read {k}, replay={mode}, run {it}")
            here = {k: v.ctypes.data for k, v in views.items()}
            assert addr is None or addr == here   # one buffer per value for the machine's life
            addr = here
        with pytest.raises(Exception):
            m0.value(G.BorrowedRead(in0))          # not a borrowed read of that machine
        m0.Close(); m1.Close()


def test_borrowed_inputs_upload_what_the_caller_wrote(ctx):
    """LetBorrowed: the caller writes an input's value into the machine's pinned buffer and the run
    uploads it from there; same results as Let with a host array, on plain and replayed runs, with the
    value changed between runs, for a per-run input and for one that is resident (uploaded once)."""
    inp = configs.convnet_inputs(16)
    for mode in (False, True):
        m0, outs0, want = run_once(configs.build_convnet, inp, fuse_activations=True)
        m0.Close()
        g = G.NewGraph()
        x = G.LetBorrowed(G.NewTensor(g, inp["x"]))
        ws = [G.NewTensor(g, inp[f"w{i}"], resident=True) for i in range(5)]
        G.LetBorrowed(ws[4])                      # resident: taken from its buffer on the first run only
        h = x
        for i in range(3):
            h = G.MaxPool2D(G.Rectify(G.Conv2d(h, ws[i], (3, 3), (1, 1), (1, 1), (1, 1))), (2, 2), (0, 0), (2, 2))
        h = G.Rectify(G.Mul(G.Reshape(h, (16, 128 * 3 * 3)), ws[3]))
        out = G.Read(G.SoftMax(G.Mul(h, ws[4])))
        m = G.NewTapeMachine(g, graph_replay=mode, fuse_activations=True)
        m.input(x)[...] = inp["x"]
        m.input(ws[4])[...] = inp["w4"]
        addr = m.input(x).ctypes.data
        for it in range(3):
            m.RunAll()
            assert_bits_equal(out, want["out"], f"borrowed input, replay={mode}, run {it}")
            m.input(ws[4])[...] = 0.0             # resident and uploaded: ignored from now on
        assert m.input(x).ctypes.data == addr
        # a new batch: both ways of binding see it
        fresh = dict(inp, x=synth.uniform(99, inp["x"].shape, 0, 1))
        m1, _, want1 = run_once(configs.build_convnet, fresh, fuse_activations=True)
        m1.Close()
        m.input(x)[...] = fresh["x"]
        m.RunAll()
        assert_bits_equal(out, want1["out"], f"borrowed input, new batch, replay={mode}")
        with pytest.raises(Exception):
            m.input(ws[0])                        # bound with a host array, nothing to lend
        m.Close()


def test_large_input_uploaded_in_pieces_each_run(ctx):
    """An input of several megabytes that is uploaded on every run travels in pieces (host copy into pinned
    memory overlapping the bus): every byte arrives, on plain, replayed and measured runs, with the value changed
    between runs, for a size that is no multiple of the piece."""
    n = (5 << 20) // 4 + 1234 * 4
    yv = synth.uniform(8, (n,), -2, 2)
    for mode in (False, True, "measured"):
        g = G.NewGraph()
        x = G.NewTensor(g, synth.uniform(7, (n,), -2, 2))
        y = G.NewTensor(g, yv, resident=True)
        out = G.Read(G.Rectify(G.Add(G.HadamardProd(x, y), x)))
        m = G.NewTapeMachine(g, graph_replay=mode)
        for it in range(7):
            a = synth.uniform(100 + it, (n,), -2, 2)
            G.Let(x, a)
            m.RunAll()
            v = a * yv + a                      # two float32 roundings, as the two operators make them
            want = v * (v >= 0).astype(np.float32)
            assert_bits_equal(out, want.reshape(out.shape), f"large input, replay={mode}, run {it}")
        m.Close()


def test_measured_replay_keeps_results_and_settles(ctx, monkeypatch):
    """graph_replay="measured": the machine times plain submits against replays of a segment on
    its first runs and keeps the quicker; every run along the way, and after the verdict, stores
    the bits of the plain run.  (The convnet with its first layer left a command of its own: five
    commands, the shortest segment the machine measures at all.)"""
    monkeypatch.setenv("GORGONIA_HIP_CONV_NO_PRE", "1")
    for build, inp in ((configs.build_convnet, configs.convnet_inputs(16)),
                       (configs.build_mlp, configs.mlp_inputs(64))):
        m0, _, want = run_once(build, inp, fuse_activations=True)
        m0.Close()
        g, outs = build(inp)
        m = G.NewTapeMachine(g, graph_replay="measured", fuse_activations=True)
        assert m.segment_verdict() == "measuring"
        for it in range(12):
            outs["out"][...] = -1.0
            m.RunAll()
            assert_bits_equal(outs["out"], want["out"], f"measured replay, run {it}")
            if it < 3 and build is configs.build_convnet:
                assert m.segment_verdict() == "measuring"
        assert m.segment_verdict() in ("plain", "replay")
        if build is configs.build_mlp:
            assert m.segment_verdict() == "plain"   # three commands: too short to be worth a graph
        # launches: the capture and two timed replays, more only if replay won
        assert m.graph_launches() in (0, 3) or m.segment_verdict() == "replay"
        total, launch, wait = m.phase_ns()
        assert total >= launch + wait > 0
        m.Close()


# operations_broadcast_test.go:24-71 (broadcastAddTests) and :183-230 (broadcastMulTests): name, a, b,
# leftPattern, rightPattern, expected a op b
BROADCAST_TABLE = [
    ("vec-mat", ([100, 200], (2,)), ([1, 2, 3, 4], (2, 2)), [1], None, [101, 102, 203, 204], [10, 20, 60, 80]),
    ("mat-vec", ([1, 2, 3, 4], (2, 2)), ([100, 200], (2,)), None, [1], [101, 102, 203, 204], [10, 20, 60, 80]),
    ("rowvec-mat", ([100, 200], (2, 1)), ([1, 2, 3, 4], (2, 2)), [1], None, [101, 102, 203, 204], [10, 20, 60, 80]),
    ("mat-rowvec", ([1, 2, 3, 4], (2, 2)), ([100, 200], (2, 1)), None, [1], [101, 102, 203, 204], [10, 20, 60, 80]),
    ("colvec-mat", ([100, 200], (1, 2)), ([1, 2, 3, 4], (2, 2)), [0], None, [101, 202, 103, 204], [10, 40, 30, 80]),
    ("mat-colvec", ([1, 2, 3, 4], (2, 2)), ([100, 200], (1, 2)), None, [0], [101, 202, 103, 204], [10, 40, 30, 80]),
]


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_broadcast_pattern_table(ctx, dtype):
    """TestBroadcastAdd / TestBroadcastHadamardProd (operations_broadcast_test.go:167-183, 262-280): the reference's
    tables (float64 there) through BroadcastAdd / BroadcastHadamardProd with explicit patterns on the tape
    machine; the multiplication table holds the addition table's operands scaled by ten."""
    for name, (av, ashp), (bv, bshp), left, right, want_add, want_mul in BROADCAST_TABLE:
        for fn, scale, want in ((G.BroadcastAdd, 1, want_add), (G.BroadcastHadamardProd, 10, want_mul)):
            def operand(v, shp):   # the multiplication table's vector is 10, 20 where the addition table's is 100, 200
                v = np.array(v, dtype=dtype)
                return (v / scale if v.max() >= 100 else v).astype(dtype).reshape(shp)
            g = G.NewGraph()
            a, b = G.NewTensor(g, operand(av, ashp)), G.NewTensor(g, operand(bv, bshp))
            out = G.Read(fn(a, b, left, right))
            m = G.NewTapeMachine(g)
            m.RunAll()
            assert out.shape == (2, 2) and out.reshape(-1).tolist() == [float(v) for v in want], f"{name} {fn}"
            m.Close()
    # ExampleBroadcastGte_creatingTriangleMatrices (example_broadcast_op_test.go:62-105): both operands repeated,
    # a = 0..2 as (3, 1) along axis 1, b = 0..3 as (1, 4) along axis 0
    g = G.NewGraph()
    a = G.NewTensor(g, np.arange(3, dtype=dtype).reshape(3, 1))
    b = G.NewTensor(g, np.arange(4, dtype=dtype).reshape(1, 4))
    tl, tu = G.Read(G.BroadcastGte(a, b, True, [1], [0])), G.Read(G.BroadcastLt(a, b, True, [1], [0]))
    m = G.NewTapeMachine(g)
    m.RunAll()
    assert tl.tolist() == [[1, 0, 0, 0], [1, 1, 0, 0], [1, 1, 1, 0]]
    assert tu.tolist() == [[0, 1, 1, 1], [0, 0, 1, 1], [0, 0, 0, 1]]
    m.Close()
    # a (2, 1) along axis 1, b (1, 3) along axis 0; subtraction keeps the operand order
    g = G.NewGraph()
    a = G.NewTensor(g, np.array([[10], [20]], dtype=dtype))
    b = G.NewTensor(g, np.array([[1, 2, 3]], dtype=dtype))
    out = G.Read(G.BroadcastSub(a, b, [1], [0]))
    m = G.NewTapeMachine(g)
    m.RunAll()
    assert out.tolist() == [[9, 8, 7], [19, 18, 17]]
    m.Close()


def test_run_all_n_is_n_run_alls(ctx):
    """RunAllN(n): n whole RunAll calls - as many submits and waits, the last step's values on the host - and it
    stops at the first error."""
    inp = configs.convnet_inputs(8)
    m0, _, want = run_once(configs.build_convnet, inp, fuse_activations=True)
    m0.Close()
    g, outs = configs.build_convnet(inp)
    m = G.NewTapeMachine(g, fuse_activations=True)
    m.RunAll()                      # the first run also uploads the resident weights
    before = m.submit_calls()
    m.RunAll()
    per_run = m.submit_calls() - before
    outs["out"][...] = -1.0
    m.RunAllN(5)
    assert per_run >= 1 and m.submit_calls() == before + 6 * per_run
    assert_bits_equal(outs["out"], want["out"], "after RunAllN(5)")
    m.RunAllN(0)
    assert m.submit_calls() == before + 6 * per_run
    m.Close()
    with pytest.raises(Exception):
        m.RunAllN(2)   # a closed machine


def test_dev_cuda_graph(ctx):
    """TestDevCUDA (cuda_test.go:14-58): x = 2 and y = 8 as 1024 x 100 float64 matrices, x + y, x - y and their
    squares read back (the test's Slice has no device operator in the reference either)."""
    g = G.NewGraph()
    x = G.NewTensor(g, np.full((1024, 100), 2.0))
    y = G.NewTensor(g, np.full((1024, 100), 8.0))
    xpy, xmy = G.Add(x, y), G.Sub(x, y)
    outs = [G.Read(n) for n in (xpy, xmy, G.Square(xpy), G.Square(xmy))]
    for kw in (dict(), dict(graph_replay=True)):
        m = G.NewTapeMachine(g, **kw)
        for _ in range(3):
            for o in outs:
                o[...] = 0
            m.RunAll()
            for o, want in zip(outs, (10.0, -6.0, 100.0, 36.0)):
                assert o.dtype == np.float64 and (o == want).all()
        m.Close()


def test_a_node_read_twice_fills_both_values(ctx):
    """gorgonia.Read makes a readOp node per call (gorgonia.go:311-318): two Reads of one node fill two values,
    whether the value reaches the host through the staging copy of the segment or a copy after the flush."""
    for n in (64, (9 << 20) // 4):
        xv = synth.uniform(3, (n,), -2, 2)
        for lisp in (False, True):
            g = G.NewGraph()
            y = G.Neg(G.NewTensor(g, xv))
            a, b = G.Read(y), G.Read(y)
            z = G.Read(G.Square(y))
            m = G.NewLispMachine(g) if lisp else G.NewTapeMachine(g)
            for _ in range(2):
                a[...] = 0; b[...] = 0
                m.RunAll()
                assert_bits_equal(a, -xv, "first Read")
                assert_bits_equal(b, -xv, "second Read")
                assert_bits_equal(z, xv * xv, "a reader of the read value")
            m.Close()


def test_lisp_machine_differential(ctx):
    """The reference's main test pattern (nn_test.go:25-79, operatorPointwise_unary_test.go:14-95):
    one graph on the TapeMachine and on the LispMachine, equal values required.  Here the second
    machine runs node by node - a submit and a wait per operator, fresh memory for every value -
    and the first batches, overwrites dead inputs, folds followers into epilogues and replays."""
    cases = [
        (configs.build_elementwise, configs.elementwise_inputs(64)),
        (configs.build_mlp, configs.mlp_inputs(32)),
        (configs.build_convnet, configs.convnet_inputs(8)),
        (configs.build_yolo, configs.yolo_inputs(1, 64)),
    ]
    for build, inp in cases:
        g, outs = build(inp)
        lisp = G.NewLispMachine(g)
        lisp.RunAll()
        want = {k: v.copy() for k, v in outs.items()}
        n_ops = lisp.program().count("execOp")
        assert lisp.segments() == n_ops + 1, "one DoWork per node, and the one in front of the reads"
        assert "[unsafe]" not in lisp.program()
        lisp.RunAll()
        for k in outs:
            assert_bits_equal(outs[k], want[k], f"{build.__name__}.{k}: lisp machine, second run")
        lisp.Close()
        for kw in (dict(), dict(fuse_activations=True), dict(fuse_activations=True, graph_replay=True)):
            g2, outs2 = build(inp)
            m = G.NewTapeMachine(g2, **kw)
            for _ in range(3):
                m.RunAll()
            for k in outs2:
                assert_bits_equal(outs2[k], want[k], f"{build.__name__}.{k}: tape {kw} == lisp")
            m.Close()


def test_cuda_basic_arithmetic_table_with_gradients(ctx):
    """TestCUDABasicArithmetic (op_math_cuda_test.go:44-99) at graph level: every entry of binOpTests
    (op_math_test.go:23-360) as a graph on the tape machine, its value and the two derivatives of
    Sum(result) equal to the table's, exactly.  The derivative nodes are the ones the reference's
    symbolic differentiation inserts, built here from the same device operators: addDiffExpr,
    subDiffExpr, hadamardProdDiffExpr, hadamardDivDiffExpr (operatorPointwise_binary.go:430-840) on
    a gradient of ones; a scalar operand's derivative is the sum of the elementwise one
    (elemBinOp.SymDiff, op_math.go:232-240), taken on the host as the reference takes it (Sum has no
    device function there).  The vector-vector Mul entries are inner products, another operator."""
    import json
    import os
    cases = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "binop.json")))["cases"]
    ops = {"Add": G.Add, "Sub": G.Sub, "Mul": G.HadamardProd, "HadamardProd": G.HadamardProd,
           "Div": G.HadamardDiv, "HadamardDiv": G.HadamardDiv}
    ran = 0
    for n, c in enumerate(cases):
        sa, sb = c["a"]["scalar"], c["b"]["scalar"]
        if c["op"] == "Mul" and not (sa or sb):
            continue
        dt = np.float32 if c["a"]["bits"] == 32 else np.float64

        def node(g, side):
            v = np.array(side["v"], dtype=dt)
            return G.NewScalar(g, v[0], dtype=dt) if side["scalar"] else G.NewTensor(g, v)

        g = G.NewGraph()
        x, y = node(g, c["a"]), node(g, c["b"])
        z = ops[c["op"]](x, y)
        ones = np.ones(z.Shape(), dtype=dt)
        grad = G.NewScalar(g, 1.0, dtype=dt) if z.Shape() == () else G.NewTensor(g, ones)
        kind = ops[c["op"]]
        if kind is G.Add:
            dx, dy = grad, grad
        elif kind is G.Sub:
            dx, dy = grad, G.Neg(grad)
        elif kind is G.HadamardProd:
            dx, dy = G.HadamardProd(y, grad), G.HadamardProd(x, grad)
        else:
            dx, dy = G.HadamardDiv(grad, y), G.HadamardProd(G.Neg(G.HadamardDiv(z, y)), grad)
        got = {"z": G.Read(z)}
        if dx is not grad:
            got["dx"] = G.Read(dx)
        if dy is not grad:
            got["dy"] = G.Read(dy)
        m = G.NewTapeMachine(g)
        m.RunAll()
        m.Close()
        assert got["z"].dtype == dt
        assert np.array_equal(got["z"].reshape(-1), np.array(c["correct"]["v"], dtype=dt)), (n, c["op"], got["z"])
        for name, operand_is_scalar, key in (("dx", sa, "deriv_a"), ("dy", sb, "deriv_b")):
            d = got.get(name, ones).reshape(-1)
            if operand_is_scalar and d.size > 1:
                d = np.array([d.sum(dtype=dt)], dtype=dt)
            want = np.array(c[key]["v"], dtype=dt)
            assert d.dtype == dt and np.array_equal(d, want), (n, c["op"], name, d, want)
        ran += 1
    assert ran >= 26


@pytest.mark.parametrize("dt", [np.float64, np.float32])
def test_mul_table_with_gradients(ctx, dt):
    """TestMul (operations_test.go:43-110) over mulTests: Mul of a vector and a matrix, two matrices, two vectors
    on RangedFrom(0) operands, and the gradients of Sum(result) - of the inner product itself for two vectors -
    equal to the table.  The gradient nodes are those of matVecMulDiffExpr, matMulDiffExpr and vecDotDiffExpr
    (operatorLinAlg.go:51-101, 181-202, 232-244) on a gradient of ones."""
    def ranged(g, shape):
        return G.NewTensor(g, np.arange(int(np.prod(shape)), dtype=dt).reshape(shape))

    # x vector: Mul(x, w) is the matrix-vector product of w transposed (operations.go:62-64)
    g = G.NewGraph()
    x, w = ranged(g, (2,)), ranged(g, (2, 3))
    z = G.Mul(x, w)
    assert z.Shape() == (3,)
    grad = G.NewTensor(g, np.ones(3, dtype=dt))
    got = {"z": G.Read(z), "dw": G.Read(G.OuterProd(x, grad)), "dx": G.Read(G.Mul(w, grad))}
    m = G.NewTapeMachine(g); m.RunAll(); m.Close()
    assert np.array_equal(got["z"], [3, 4, 5])
    assert np.array_equal(got["dx"], [3, 12]) and got["dx"].shape == (2,)
    assert np.array_equal(got["dw"].reshape(-1), [0, 0, 0, 1, 1, 1]) and got["dw"].shape == (2, 3)

    # x mat
    g = G.NewGraph()
    x, w = ranged(g, (3, 2)), ranged(g, (2, 3))
    z = G.Mul(x, w)
    grad = G.NewTensor(g, np.ones((3, 3), dtype=dt))
    got = {"z": G.Read(z), "dx": G.Read(G.Mul(grad, w, transB=True)), "dw": G.Read(G.Mul(x, grad, transA=True))}
    m = G.NewTapeMachine(g); m.RunAll(); m.Close()
    assert np.array_equal(got["z"], np.arange(6).reshape(3, 2) @ np.arange(6).reshape(2, 3))
    assert np.array_equal(got["dx"].reshape(-1), [3, 12, 3, 12, 3, 12]) and got["dx"].shape == (3, 2)
    assert np.array_equal(got["dw"].reshape(-1), [6, 6, 6, 9, 9, 9]) and got["dw"].shape == (2, 3)

    # x_vec_w_vec: the inner product, a scalar, differentiated itself
    g = G.NewGraph()
    x, w = ranged(g, (6,)), ranged(g, (6,))
    z = G.Mul(x, w)
    assert z.Shape() == ()
    grad = G.NewScalar(g, 1.0, dtype=dt)
    got = {"z": G.Read(z), "dx": G.Read(G.HadamardProd(w, grad)), "dw": G.Read(G.HadamardProd(x, grad))}
    m = G.NewTapeMachine(g); m.RunAll(); m.Close()
    assert got["z"].dtype == dt and got["z"].reshape(-1)[0] == 55
    assert np.array_equal(got["dx"], np.arange(6)) and np.array_equal(got["dw"], np.arange(6))


@pytest.mark.parametrize("machine", [G.NewTapeMachine, G.NewLispMachine])
def test_nan_and_inf_watch(ctx, machine):
    """WithNaNWatch / WithInfWatch (vm.go:138-166, vm_tape.go:271-315): the run stops at the first operator
    whose value holds a NaN / an Inf, naming it; what comes after it is not run.  Without the watch the same
    graph runs through, and on a clean graph the watch changes no bit."""
    x = synth.uniform(71, (37, 129), 0.5, 2.0)

    def build(poison):
        g = G.NewGraph()
        v = x.copy()
        if poison == "nan":
            v[17, 5] = -1.0          # ln of a negative number
        if poison == "inf":
            v[3, 100] = 0.0          # ln 0
        a = G.NewTensor(g, v)
        b = G.Log(a)
        c = G.Square(G.Add(b, b))
        return g, {"log": G.Read(b), "after": G.Read(c)}

    g, want = build(None)
    m = machine(g); m.RunAll(); m.Close()
    g, got = build(None)
    m = machine(g, G.WithNaNWatch(), G.WithInfWatch())
    m.RunAll(); m.RunAll()
    m.Close()
    assert_bits_equal(got["log"], want["log"], "log")
    assert_bits_equal(got["after"], want["after"], "after")

    for poison, opt, other, word in (("nan", G.WithNaNWatch, G.WithInfWatch, "NaN"), ("inf", G.WithInfWatch, G.WithNaNWatch, "Inf")):
        g, got = build(poison)
        for v in got.values():
            v[...] = -7.0
        m = machine(g, opt())
        with pytest.raises(G.EngineError) as e:
            m.RunAll()
        assert f"{word} found in value. Node: elemunary.ln(1)" in str(e.value), str(e.value)
        assert np.all(got["after"] == -7.0) and np.all(got["log"] == -7.0)   # nothing behind the hit ran
        m.Close()
        # the other watch lets this value pass at the logarithm; unwatched, the graph runs through
        g, got = build(poison)
        m = machine(g)
        m.RunAll()
        assert (np.isnan(got["log"]).sum() == 1) if poison == "nan" else (np.isinf(got["log"]).sum() == 1)
        m.Close()
    # -Inf squared is +Inf, a NaN stays a NaN: the Inf watch alone sees the NaN graph through
    g, got = build("nan")
    m = machine(g, G.WithInfWatch())
    m.RunAll()
    assert np.isnan(got["after"]).sum() == 1
    m.Close()


def test_watch_sees_a_nan_a_pool_would_drop(ctx):
    """A max-pool never selects a NaN (strict >), so the pooled value of a convolution that produced one is clean:
    a watched machine folds nothing and stops at the convolution."""
    x = synth.uniform(91, (2, 8, 12, 12), 0, 1)
    x[1, 3, 5, 5] = np.nan
    w = synth.he_normal(92, (16, 8, 3, 3))

    def build():
        g = G.NewGraph()
        h = G.Conv2d(G.NewTensor(g, x), G.NewTensor(g, w, resident=True), (3, 3), (1, 1), (1, 1), (1, 1))
        return g, G.Read(G.MaxPool2D(G.Rectify(h), (2, 2), (0, 0), (2, 2)))

    g, out = build()
    m = G.NewTapeMachine(g, fuse_activations=True)
    assert m.fused > 0
    m.RunAll(); m.Close()
    assert not np.isnan(out).any()
    g, out = build()
    m = G.NewTapeMachine(g, G.WithNaNWatch(), fuse_activations=True)
    assert m.fused == 0
    with pytest.raises(G.EngineError) as e:
        m.RunAll()
    assert "NaN found in value. Node: conv2d(" in str(e.value), str(e.value)
    m.Close()


UNARY_API = {"Abs": "abs", "Sign": "sign", "Ceil": "ceil", "Floor": "floor", "Sin": "sin", "Cos": "cos", "Exp": "exp",
             "Log": "ln", "Log2": "log2", "Neg": "neg", "Square": "square", "Sqrt": "sqrt", "Inverse": "inverse",
             "InverseSqrt": "invsqrt", "Cube": "cube", "Tanh": "tanh", "Sigmoid": "sigmoid", "Log1p": "log1p",
             "Expm1": "expm1", "Softplus": "softplus"}
BINARY_API = {"Add": "add", "Sub": "sub", "HadamardProd": "mul", "HadamardDiv": "div", "Pow": "pow", "Mod": "mod",
              "Lt": "lt", "Lte": "lte", "Gt": "gt", "Gte": "gte", "Eq": "eq", "Ne": "ne"}


def _ulps(got, want):
    """Distance in units in the last place of the arrays' own type; equal NaNs and equal zeros count as 0."""
    it = np.int32 if got.dtype == np.float32 else np.int64
    top = np.iinfo(it).max
    gi, wi = got.reshape(-1).view(it).astype(np.int64), want.reshape(-1).view(it).astype(np.int64)
    gi = np.where(gi < 0, -(gi & top), gi)
    wi = np.where(wi < 0, -(wi & top), wi)
    d = np.abs(gi - wi)
    d[np.isnan(got.reshape(-1)) & np.isnan(want.reshape(-1))] = 0
    return d


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_every_pointwise_name_on_both_machines(ctx, dt):
    """Every unary and binary name of api_gen.go:6-127 as a graph on the tape machine and on the lisp machine
    (operatorPointwise_unary_test.go:14-95 runs each unary operator on both): the two machines agree bit for bit
    and stand within 2 ulp of the oracle's function of that name (0 for the single-operation ones), tensor with
    tensor, tensor with scalar and scalar with tensor."""
    from oracle import binding as O
    x = synth.uniform(111, (33, 65), 0.25, 3.0).astype(dt)
    y = synth.uniform(112, (33, 65), 0.5, 2.5).astype(dt)
    y[::7, ::5] = x[::7, ::5]                      # equal pairs for the comparisons
    s = np.array(1.75, dtype=dt)
    exact = {"abs", "sign", "ceil", "floor", "neg", "square", "sqrt", "inverse", "cube"} | (set(BINARY_API.values()) - {"pow"})

    def run(machine, build):
        g = G.NewGraph()
        out = G.Read(build(g))
        m = machine(g)
        m.RunAll()
        m.Close()
        return out

    def check(name, fn, build, want):
        a, b = run(G.NewTapeMachine, build), run(G.NewLispMachine, build)
        assert a.dtype == dt and a.shape == x.shape
        assert_bits_equal(a, b, f"{name}: tape against lisp")
        u = _ulps(a, np.asarray(want, dtype=dt).reshape(x.shape))
        assert u.max() <= (0 if fn in exact else 2), f"{name} ({np.dtype(dt).name}): {u.max()} ulp"

    with np.errstate(all="ignore"):
        for name, fn in UNARY_API.items():
            check(name, fn, lambda g: getattr(G, name)(G.NewTensor(g, x)), O.unary(fn, x))
        for name, fn in BINARY_API.items():
            op = getattr(G, name)
            check(name + " vv", fn, lambda g: op(G.NewTensor(g, x), G.NewTensor(g, y)), O.binop(fn, "vv", x, y))
            check(name + " vs", fn, lambda g: op(G.NewTensor(g, x), G.NewScalar(g, s, dtype=dt)),
                  O.binop(fn, "vs", x, s.reshape(1)))
            check(name + " sv", fn, lambda g: op(G.NewScalar(g, s, dtype=dt), G.NewTensor(g, y)),
                  O.binop(fn, "sv", s.reshape(1), y))


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_batched_matmul_graph(ctx, dt):
    """BatchedMatMul(a, b, transes...) (operations.go:76-98) as a graph operator on both machines, all four
    transpose combinations, leading dimensions of rank 1 and 2, against the float64 product."""
    tol = 1e-5 if dt == np.float32 else 1e-12
    for lead in ((5,), (2, 3)):
        for ta in (False, True):
            for tb in (False, True):
                a = synth.uniform(121, lead + ((9, 7) if ta else (7, 9)), -1, 1).astype(dt)
                b = synth.uniform(122, lead + ((11, 9) if tb else (9, 11)), -1, 1).astype(dt)
                want = np.matmul(np.swapaxes(a, -1, -2) if ta else a, np.swapaxes(b, -1, -2) if tb else b, dtype=np.float64)
                res = []
                for machine in (G.NewTapeMachine, G.NewLispMachine):
                    g = G.NewGraph()
                    out = G.Read(G.BatchedMatMul(G.NewTensor(g, a), G.NewTensor(g, b), ta, tb))
                    m = machine(g)
                    m.RunAll()
                    m.Close()
                    assert out.dtype == dt and out.shape == lead + (7, 11)
                    assert rel_frobenius(out, want) <= tol, (lead, ta, tb)
                    res.append(out)
                assert_bits_equal(res[0], res[1], f"{lead} {ta} {tb}: tape against lisp")
