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
    assert m2.fused == 8  # 4 activations, the three pools and the softmax
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
    inp = configs.convnet_inputs(8)
    m1, _, r1 = run_once(configs.build_convnet, inp)
    g, outs = configs.build_convnet(inp, resident=False)
    m2 = G.NewTapeMachine(g)
    m2.RunAll(); m2.RunAll()
    assert_bits_equal(outs["out"], r1["out"], "re-uploaded weights")
    m1.Close(); m2.Close()
