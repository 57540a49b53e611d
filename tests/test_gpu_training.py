"""GPU parity of a whole training step: convnet forward, the diff ops of every
layer, and the in-place SGD update through Set, on the tape machine, against
the CPU oracle's step on the same seeded inputs (<= 1e-5 relative Frobenius per
gradient; every kernel on the way has its own tighter test)."""
import numpy as np
import pytest

from gorgonia_amd import configs, graph as G, synth
from oracle import forward as F
from tests.util import assert_bits_equal, rel_frobenius

pytestmark = pytest.mark.gpu
TOL = 1e-5


def _onehot(batch):
    y = np.zeros((batch, 10), np.float32)
    y[np.arange(batch), (np.arange(batch) * 7 + 3) % 10] = 1.0
    return y


def test_convnet_training_step_gradients(ctx):
    inp = configs.convnet_inputs(32)
    y = _onehot(32)
    g, outs = configs.build_convnet_train(inp, y, 0.05)
    m = G.NewTapeMachine(g)
    m.RunAll()
    out, cost, grads, new = F.convnet_train_step(inp, y, 0.05)
    assert rel_frobenius(outs["out"], out) <= TOL
    for i in range(5):
        err = rel_frobenius(outs[f"dw{i}"], grads[f"w{i}"])
        assert err <= TOL, f"dw{i}: {err:.3e}"
    # the weights moved on the device: the second step's forward pass sees them
    m.RunAll()
    inp2 = dict(inp, **new)
    out2, _, grads2, _ = F.convnet_train_step(inp2, y, 0.05)
    assert rel_frobenius(outs["out"], out2) <= TOL
    for i in range(5):
        assert rel_frobenius(outs[f"dw{i}"], grads2[f"w{i}"]) <= 5 * TOL
    assert not np.array_equal(out, out2)
    m.Close()


def test_training_step_with_folded_operators_keeps_every_bit(ctx):
    """FuseActivations on the training graph: the Rectify between each convolution's pool and the two
    gradients is read through by both (its result and the pooling gradient are never stored) and the last
    product carries its SoftMax.  Output and every weight gradient equal the unfolded machine's bit for bit,
    on the first step and on the second (weights updated on the device), plainly run and replayed."""
    inp = configs.convnet_inputs(24)
    y = _onehot(24)
    for replay in (False, True):
        g0, outs0 = configs.build_convnet_train(inp, y, 0.05)
        m0 = G.NewTapeMachine(g0)
        g1, outs1 = configs.build_convnet_train(inp, y, 0.05)
        m1 = G.NewTapeMachine(g1, fuse_activations=True, graph_replay=replay)
        assert m1.fused == 10          # 3 x (Rectify, MaxPool2DDiff) + the SoftMax + 3 x (pool into its convolution)
        prog = m1.program()
        assert prog.count("rectify+maxpool2d.diff") == 3
        # every convolution stores its own result (the backward pass reads it) and the pooled activation
        assert prog.count("conv2d(kept)+rectify+maxpool2d") == 3 and prog.count(" rectify+maxpool2d ") == 0
        assert prog.count("rectifyDiff") == 1       # the dense layer's activation is not pooled
        ops = lambda m: len([l for l in m.program().splitlines() if "execOp" in l])
        assert ops(m1) == ops(m0) - 10
        for step in range(3):
            m0.RunAll(); m1.RunAll()
            for k in outs0:
                assert_bits_equal(outs1[k], outs0[k], f"{k}, step {step}, replay={replay}")
        m0.Close(); m1.Close()


def test_training_steps_replayed_from_a_graph(ctx):
    """Steps 2.. run as hipGraph replays; the in-place weight updates persist
    between replays and the cost goes down."""
    inp = configs.convnet_inputs(16)
    y = _onehot(16)
    g, outs = configs.build_convnet_train(inp, y, 0.5, read_grads=False)
    m = G.NewTapeMachine(g, graph_replay=True)
    cur = dict(inp)
    costs = []
    for step in range(5):
        m.RunAll()
        want, cost, _, new = F.convnet_train_step(cur, y, 0.5)
        assert rel_frobenius(outs["out"], want) <= 2 * TOL * (step + 1), f"step {step}"
        costs.append(-float((outs["out"] * y).mean()))
        cur = dict(cur, **new)
    assert m.graph_launches() >= 3
    assert costs[-1] < costs[0]
    m.Close()


def test_training_with_device_solver_steps(ctx):
    """The same step with the update done by the fused solver kernels: vanilla equals the
    Set-spelled update bit for bit; RMSProp (the example's solver) follows the oracle."""
    inp = configs.convnet_inputs(16)
    y = _onehot(16)
    outs_by = {}
    for solver in ("set", "vanilla", "rmsprop"):
        g, outs = configs.build_convnet_train(inp, y, 0.05 if solver != "rmsprop" else 0.01, read_grads=False,
                                              solver=solver)
        m = G.NewTapeMachine(g, graph_replay=True)
        hist = []
        for _ in range(4):
            m.RunAll()
            hist.append(outs["out"].copy())
        assert m.graph_launches() >= 2
        outs_by[solver] = hist
        m.Close()
    for a, b in zip(outs_by["set"], outs_by["vanilla"]):
        assert_bits_equal(a, b, "vanilla solver step == w - lr*dw through Set")
    # RMSProp against the oracle: forward/backward by the oracle step, update by the oracle solver
    cur = dict(inp)
    caches = {k: np.zeros_like(inp[k]) for k in ("w0", "w1", "w2", "w3", "w4")}
    from oracle import binding as O
    for step in range(4):
        want, _, grads, _ = F.convnet_train_step(cur, y, 0.0)
        assert rel_frobenius(outs_by["rmsprop"][step], want) <= 2 * TOL * (step + 1), f"rmsprop step {step}"
        for k in caches:
            wn, _, cn, _ = O.solver_step("rmsprop", cur[k].reshape(-1), grads[k].reshape(-1), caches[k].reshape(-1),
                                         eta=0.01, l2reg=1e-6, clip=5.0)
            cur[k], caches[k] = wn.reshape(cur[k].shape), cn.reshape(cur[k].shape)


def test_set_updates_a_resident_input_in_place(ctx):
    g = G.NewGraph()
    a = G.NewTensor(g, np.arange(8, dtype=np.float32), resident=True)
    one = G.NewScalar(g, 1.0)
    out = G.Read(G.Set(a, G.Add(a, one)))
    m = G.NewTapeMachine(g)
    for k in range(1, 4):
        m.RunAll()
        assert_bits_equal(out, np.arange(8, dtype=np.float32) + k, f"after {k} runs")
    m.Close()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_adam_steps_replay_with_corrections_from_memory(ctx, dtype):
    """Adam's bias corrections change every iteration.  Bound as an input that the host rebinds
    before each run they are read from memory, so the step is the same command every time: the
    segment is captured once and replayed, and weights and both caches follow the oracle's
    iterations bit for bit (as command constants every step would be a new command)."""
    from oracle import binding as O
    n = 5000
    w0 = synth.normal(61, (n,)).astype(dtype)
    grads = [synth.normal(70 + t, (n,), 0.0, 2.0).astype(dtype) for t in range(6)]
    g = G.NewGraph()
    w = G.NewTensor(g, w0.copy(), resident=True)
    m1 = G.NewTensor(g, np.zeros(n, dtype), resident=True)
    m2 = G.NewTensor(g, np.zeros(n, dtype), resident=True)
    grad = G.NewTensor(g, grads[0])
    corr = G.NewTensor(g, G.AdamCorrections(1, dtype=dtype))
    # enough small operators in front of the step that the segment is worth a graph
    gg = grad
    for _ in range(4):
        gg = G.Neg(G.Neg(gg))
    out = G.Read(G.SolverStep("adam", w, gg, (m1, m2), eta=0.01, l2reg=1e-4, clip=3.0, corrections=corr))
    r1, r2 = G.Read(m1), G.Read(m2)
    m = G.NewTapeMachine(g, graph_replay=True)
    want_w, c1, c2 = w0.copy(), np.zeros(n, dtype), np.zeros(n, dtype)
    for t in range(6):
        G.Let(grad, grads[t])
        G.Let(corr, G.AdamCorrections(t + 1, dtype=dtype))
        m.RunAll()
        want_w, _, c1, c2 = O.solver_step("adam", want_w, grads[t], c1, c2, eta=0.01, l2reg=1e-4, clip=3.0, iteration=t + 1)
        assert_bits_equal(out, want_w, f"adam weights, iteration {t + 1}")
        assert_bits_equal(r1, c1, f"adam m, iteration {t + 1}")
        assert_bits_equal(r2, c2, f"adam v, iteration {t + 1}")
    assert m.graph_launches() >= 4, "the step did not stay the same command"
    m.Close()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("machine", [G.NewTapeMachine, G.NewLispMachine])
def test_batchnorm_training_graph(ctx, dt, machine):
    """BatchNorm in training mode and its gradient as graph operators on both machines: the oracle's values; the
    running statistics live in resident tensors and carry over from run to run; and what the reference's own
    (commented-out) device test asks of the result (ops/nn/api_cuda_test.go:24-75): on Gaussian input of shape
    (5, 2, 3, 4) every channel of the output has mean 0 within 1e-5 and mean square 1 within 1e-4."""
    from oracle import binding as O
    shape = (5, 2, 3, 4)
    x = synth.normal(61, shape).astype(dt)
    dy = synth.uniform(62, shape, -1, 1).astype(dt)
    Cn = shape[1]
    g = G.NewGraph()
    xn = G.NewTensor(g, x)
    rm = G.NewTensor(g, np.zeros(Cn, dt), resident=True)
    rv = G.NewTensor(g, np.ones(Cn, dt), resident=True)
    sm = G.NewTensor(g, np.zeros(Cn, dt), resident=True)
    sv = G.NewTensor(g, np.zeros(Cn, dt), resident=True)
    y = G.BatchNormTrain(xn, rm, rv, sm, sv, momentum=0.9, epsilon=1e-5)
    dx = G.BatchNormDiff(xn, G.NewTensor(g, dy), sm, sv, epsilon=1e-5)
    got = {"y": G.Read(y), "dx": G.Read(dx), "rm": G.Read(rm), "rv": G.Read(rv)}
    m = machine(g)
    tol = 1e-5 if dt == np.float32 else 1e-12
    want_rm, want_rv = np.zeros(Cn, dt), np.ones(Cn, dt)
    for run in range(3):
        m.RunAll()
        want_y, want_rm, want_rv, w_sm, w_sv = O.bn_train_stats(x, want_rm, want_rv, 0.9, 1e-5)
        want_dx = O.bn_bwd(x, dy, w_sm, w_sv, 1e-5, True)
        for k, want in (("y", want_y), ("dx", want_dx), ("rm", want_rm), ("rv", want_rv)):
            assert got[k].dtype == dt
            assert np.linalg.norm(got[k].astype(np.float64) - want) <= tol * np.linalg.norm(want), (run, k)
    m.Close()
    yv = got["y"].astype(np.float64)
    mean = yv.mean(axis=(0, 2, 3))
    mean_sq = (yv * yv).mean(axis=(0, 2, 3))
    assert np.all(np.abs(mean) < 1e-5), mean
    assert np.all(np.abs(mean_sq - 1.0) < 1e-4), mean_sq
