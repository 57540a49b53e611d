#!/usr/bin/env python3
"""Benchmark of the MI355X tensor-engine hot path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--skip-cpu]

A step is one forward pass of the convnet configuration (batch 128x1x28x28,
3x[Conv2d 3x3 + ReLU + MaxPool 2x2] + 2 dense layers + SoftMax) on the tape
machine, with weights and the input batch already resident in HBM.  The same
run also measures the other two parts of the headline metric - the elementwise
chain on 4096x4096 tensors (HBM GB/s) and SGEMM 4096^3 (TFLOP/s) - with HIP
events on the engine's own stream, and times the CPU oracle on the host cores
as a reported baseline.  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E
MFMA_F32_PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix


def log(*a):
    print(*a, file=sys.stderr, flush=True)


EAGER_TIMING = False  # --eager-timing: no hipGraph anywhere (for hardware-counter runs)
# A tape machine in "measured" mode runs a segment plainly three times, captures it, replays it twice
# and then keeps the quicker way: the timed loops start after that.
WARM_RUNS = 8


def warm_up(m, warmup):
    """The untimed steps in front of a timed loop: the `warmup` asked for (at least WARM_RUNS), then more
    until SUSTAIN_MS of steps have run - the GPU raises its clocks only under load that lasts, and a timed
    loop of a few dozen 50 us steps would otherwise be measured on the ramp (time_cmds warms the same way)."""
    m.RunAllN(max(warmup, WARM_RUNS))
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < SUSTAIN_MS:
        m.RunAllN(16)
VERDICTS = {}  # workload -> how its segment ended up being run ("plain" / "replay")


def replay_mode():
    return False if EAGER_TIMING else "measured"


SUSTAIN_MS = 40.0   # a kernel is timed after this much back-to-back work of its own, over this much more
IN_FLIGHT = 32      # graph replays queued between two host waits of the sustained loop


def time_cmds(ctx, cmds, iters, warm=3):
    """Average milliseconds per pass over `cmds`: `iters` passes are captured into one hipGraph
    (so host enqueue time is out of the picture) and replays are bracketed by HIP events on the
    engine's stream.

    The GPU raises its clocks only under load that lasts: the same kernel measured over a 5 ms
    burst after idle time runs 15-20 % slower than in a loop that has been busy for tens of
    milliseconds (64 x 512^3 products: 178 us against 151 us).  A production loop is the second
    case, so the graph is first replayed for SUSTAIN_MS, then timed over at least SUSTAIN_MS.
    The first replay after the capture - the short-burst figure - is kept in
    time_cmds.last_burst_ms."""
    ctx.submit(list(cmds) * warm)
    ctx.sync()
    if EAGER_TIMING:
        ctx.event(0)
        ctx.submit(list(cmds) * iters)
        ctx.event(1)
        time_cmds.last_burst_ms = ctx.elapsed_ms(0, 1) / iters
        return time_cmds.last_burst_ms
    ctx.graph_begin()
    ctx.submit(list(cmds) * iters)
    gid = ctx.graph_end()
    ctx.graph_launch(gid)
    ctx.sync()
    ctx.event(0)
    ctx.graph_launch(gid)
    ctx.event(1)
    one = ctx.elapsed_ms(0, 1)
    time_cmds.last_burst_ms = one / iters
    if SUSTAIN_MS <= 0:
        ctx.graph_destroy(gid)
        return time_cmds.last_burst_ms
    reps = max(1, min(4000, int(SUSTAIN_MS / max(one, 1e-3)) + 1))

    def replay(n):
        # At most 2 * IN_FLIGHT replays are ever queued: every IN_FLIGHT launches an event goes into the
        # stream and the host waits for the event of the batch before (the device never runs dry: a whole
        # batch is still queued behind the one it waits for).  Thousands of graph launches queued at
        # once are what a run of this loop under a tracing profiler died of.
        slot = 2
        for i in range(n):
            ctx.graph_launch(gid)
            if (i + 1) % IN_FLIGHT == 0:
                ctx.event(slot)
                if i + 1 >= 2 * IN_FLIGHT:
                    ctx.elapsed_ms(5 - slot, 5 - slot)   # the other slot: the batch before this one
                slot = 5 - slot

    replay(reps)
    ctx.event(0)
    replay(reps)
    ctx.event(1)
    ms = ctx.elapsed_ms(0, 1) / (iters * reps)
    ctx.graph_destroy(gid)
    return ms


time_cmds.last_burst_ms = None


ELEMENTWISE_SETS = 8   # operand sets a timed kernel rotates over: 8 x (2..3) x 64 MiB >= 1 GiB, four times the last-level cache


def bench_elementwise(ctx, iters):
    """Config 2: z = Sigmoid(x*y + b); Tanh(z); Pow(z, 2) on 4096x4096 float32.

    Every kernel is timed twice.  `cold`: consecutive launches walk over ELEMENTWISE_SETS
    distinct operand sets (1-1.5 GiB in all), so no launch finds its operands in the 256 MB
    last-level cache and the bytes really cross the HBM interface - that is the figure
    reported as frac_hbm.  `warm`: the same launch on one operand set over and over (128-192
    MiB, cache-assisted), kept next to it as frac_llc_assisted."""
    from gorgonia_amd import configs, device as D
    inp = configs.elementwise_inputs(4096)
    N = 4096 * 4096
    S = ELEMENTWISE_SETS
    x0, y0, b = ctx.upload(inp["x"]), ctx.upload(inp["y"]), ctx.upload(inp["b"])
    two = ctx.upload(np.array([2.0], np.float32))
    xs, ys, ps = [x0], [y0], [ctx.malloc(4 * N)]
    for _ in range(S - 1):   # the other sets are device-side copies of the first
        xs.append(ctx.malloc(4 * N)); ys.append(ctx.malloc(4 * N)); ps.append(ctx.malloc(4 * N))
        ctx.run([D.cmd_copy(xs[-1], x0, 4 * N), D.cmd_copy(ys[-1], y0, 4 * N)])
    # z = Sigmoid(x*y + b) per set, written into ys (the chain's intermediate value)
    zs = ys

    def build(name, i):
        x, p, z = xs[i], ps[i], zs[i]
        if name == "HadamardProd":
            return D.cmd_bin("mul", "vv", x, zs[i], N, dst=p)
        if name == "BroadcastAdd":
            return D.cmd_bcast("add", p, x, b, 4096, 4096, 1)
        if name == "Sigmoid":   # in place, as the tape machine runs it in this chain: its operand x*y + b is dead
            return D.cmd_unary("sigmoid", z, N)
        if name == "Tanh":
            return D.cmd_unary("tanh", z, N, dst=p)
        return D.cmd_bin("pow", "vs", z, two, N, dst=p)

    sizes = {"HadamardProd": 3 * 4 * N, "BroadcastAdd": 2 * 4 * N + 4 * 4096, "Sigmoid": 2 * 4 * N,
             "Tanh": 2 * 4 * N, "Pow2": 2 * 4 * N}
    out, total_ms, total_ms_warm, total_bytes = {}, 0.0, 0.0, 0
    passes = max(2, iters // S)
    for name, nbytes in sizes.items():
        ms_cold = time_cmds(ctx, [build(name, i) for i in range(S)], passes) / S
        ms_warm = time_cmds(ctx, [build(name, 0)], iters)
        out[name] = {"us": round(ms_cold * 1e3, 2), "GBps": round(nbytes / ms_cold / 1e6, 1),
                     "frac_hbm": round(nbytes / ms_cold / 1e6 / HBM_PEAK_GBPS, 4), "bytes": nbytes,
                     "us_llc_assisted": round(ms_warm * 1e3, 2),
                     "frac_llc_assisted": round(nbytes / ms_warm / 1e6 / HBM_PEAK_GBPS, 4)}
        total_ms += ms_cold
        total_ms_warm += ms_warm
        total_bytes += nbytes
    # what a one-read-one-write kernel with no arithmetic at all reaches on the same rotating sets: the
    # ceiling Sigmoid, Tanh and Pow2 (same traffic) are measured against
    ms_neg = time_cmds(ctx, [D.cmd_unary("neg", xs[i], N, dst=ps[i]) for i in range(S)], passes) / S
    no_arith = {"us": round(ms_neg * 1e3, 2), "GBps": round(2 * 4 * N / ms_neg / 1e6, 1),
                "frac_hbm": round(2 * 4 * N / ms_neg / 1e6 / HBM_PEAK_GBPS, 4), "bytes": 2 * 4 * N,
                "kernel": "Neg, same tensors and rotation as Sigmoid"}
    # the chain as configuration 2 issues it - five launches in order on one set of tensors
    # (x, y, z, t, p: 320 MiB, intermediates re-read straight after they were written)
    z, t, p = ys[1], ps[0], ps[1]
    seq = [D.cmd_bin("mul", "vv", xs[0], ys[0], N, dst=z), D.cmd_bcast("add", z, z, b, 4096, 4096, 1),
           D.cmd_unary("sigmoid", z, N), D.cmd_unary("tanh", z, N, dst=t), D.cmd_bin("pow", "vs", z, two, N, dst=p)]
    ms_seq = time_cmds(ctx, seq, max(4, iters // 3))
    # tensors no cache can hold (8192 x 8192, 256 MiB each): the kernels' streaming form
    big = [ctx.malloc(16 * N) for _ in range(3)]
    ctx.run([D.cmd_fill(q, 4 * N, 1.5) for q in big[:2]])
    streaming = {}
    for name, cmd, nbytes in (("Neg_8192", D.cmd_unary("neg", big[0], 4 * N, dst=big[2]), 2 * 16 * N),
                              ("HadamardProd_8192", D.cmd_bin("mul", "vv", big[0], big[1], 4 * N, dst=big[2]), 3 * 16 * N)):
        ms = time_cmds(ctx, [cmd], max(4, iters // 4))
        streaming[name] = {"us": round(ms * 1e3, 2), "GBps": round(nbytes / ms / 1e6, 1),
                           "frac_hbm": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4), "bytes": nbytes}
    for q in big:
        ctx.free(q)
    # device copy of the same size as a measured ceiling next to the nominal one, cold and warm
    ms = time_cmds(ctx, [D.cmd_copy(ps[i], xs[i], 4 * N) for i in range(S)], passes) / S
    copy_gbps = 2 * 4 * N / ms / 1e6
    ms = time_cmds(ctx, [D.cmd_copy(ps[0], xs[0], 4 * N)], iters)
    copy_gbps_warm = 2 * 4 * N / ms / 1e6
    for q in xs + ys + ps + [b, two]:
        ctx.free(q)
    return {"chain_GBps": round(total_bytes / total_ms / 1e6, 1), "chain_bytes": total_bytes,
            "chain_us": round(total_ms * 1e3, 1), "frac_hbm": round(total_bytes / total_ms / 1e6 / HBM_PEAK_GBPS, 4),
            "frac_llc_assisted": round(total_bytes / total_ms_warm / 1e6 / HBM_PEAK_GBPS, 4),
            "chain_in_sequence_us": round(ms_seq * 1e3, 1), "chain_in_sequence_GBps": round(total_bytes / ms_seq / 1e6, 1),
            "streaming_8192": streaming, "operand_sets": S, "footprint_bytes": 3 * S * 4 * N,
            "device_copy_GBps": round(copy_gbps, 1), "device_copy_GBps_llc_assisted": round(copy_gbps_warm, 1),
            "kernels": out, "one_read_one_write_without_arithmetic": no_arith}


def bench_linalg(ctx, iters):
    """Config 3: SGEMM 4096^3, BatchedMatMul 64 x 512^3, MatVecMul 8192^2."""
    from gorgonia_amd import device as D, synth
    res = {}
    for name, (m, n, k, batch) in {"sgemm_4096": (4096, 4096, 4096, 1), "bmm_64x512": (512, 512, 512, 64)}.items():
        A = ctx.upload(synth.normal(1, (batch * m * k,)))
        B = ctx.upload(synth.normal(2, (batch * k * n,)))
        Cm = ctx.malloc(batch * m * n * 4)
        cmd = D.cmd_gemm(A, B, Cm, m, n, k, batch=batch, stride_a=m * k, stride_b=k * n, stride_c=m * n)
        ms = time_cmds(ctx, [cmd], max(5, iters // 2))
        fl = 2.0 * m * n * k * batch
        res[name] = {"us": round(ms * 1e3, 1), "TFLOPs": round(fl / ms / 1e9, 2),
                     "frac_mfma": round(fl / ms / 1e9 / MFMA_F32_PEAK_TFLOPS, 4), "flop": fl,
                     "us_short_burst": round(time_cmds.last_burst_ms * 1e3, 1)}
        for q in (A, B, Cm):
            ctx.free(q)
    # float64 product (Dgemm path), against the fp64 matrix peak of 78.6 TFLOP/s
    from gorgonia_amd import _ffi
    m = n = k = 2048
    A = ctx.upload(synth.normal(6, (m * k,)).astype(np.float64))
    B = ctx.upload(synth.normal(7, (k * n,)).astype(np.float64))
    Cm = ctx.malloc(m * n * 8)
    ms = time_cmds(ctx, [D.cmd_gemm(A, B, Cm, m, n, k, dtype=_ffi.F64)], max(5, iters // 2))
    res["dgemm_2048"] = {"us": round(ms * 1e3, 1), "TFLOPs": round(2.0 * m * n * k / ms / 1e9, 2),
                         "frac_mfma_f64": round(2.0 * m * n * k / ms / 1e9 / 78.6, 4)}
    for q in (A, B, Cm):
        ctx.free(q)
    m = n = 8192
    A = ctx.upload(synth.normal(3, (m * n,)))
    xv, yv = ctx.upload(synth.normal(4, (n,))), ctx.malloc(4 * m)
    ms = time_cmds(ctx, [D.cmd_gemv(A, xv, yv, m, n)], iters)
    nb = 4 * (m * n + m + n)
    res["gemv_8192"] = {"us": round(ms * 1e3, 1), "GBps": round(nb / ms / 1e6, 1),
                        "frac_hbm": round(nb / ms / 1e6 / HBM_PEAK_GBPS, 4), "bytes": nb}
    # the transposed product (x^T A): the same bytes, columns summed over rows
    xt, yt = ctx.upload(synth.normal(5, (m,))), ctx.malloc(4 * n)
    ms = time_cmds(ctx, [D.cmd_gemv(A, xt, yt, m, n, trans=True)], iters)
    res["gemv_t_8192"] = {"us": round(ms * 1e3, 1), "GBps": round(nb / ms / 1e6, 1),
                          "frac_hbm": round(nb / ms / 1e6 / HBM_PEAK_GBPS, 4), "bytes": nb}
    for q in (A, xv, yv, xt, yt):
        ctx.free(q)
    return res


# HBM bytes per launch of each conv layer's kernel as the step issues it (conv +
# ReLU + 2x2 max-pool in one launch): constants read off rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE runs of this script, not measured by this run (KiB per dispatch;
# FETCH_SIZE scaled by 2.0, WRITE_SIZE by 1.0, the factors a 64 MiB device copy
# in the same runs gives).  TRAFFIC_SOURCE names the summary that holds the runs.
MEASURED_TRAFFIC_BYTES = {
    "conv0": (2 * 1419.1 + 3584.0) * 1024,
    "conv1": (2 * 1969.1 + 1568.0) * 1024,
    "conv2": (2 * 2028.6 + 576.0) * 1024,
    "conv0+conv1": (2 * 627.7 + 1568.0) * 1024,
}
TRAFFIC_SOURCE = ("constant from profiles/convnet_yolo_elementwise_hbm_traffic_pmc.txt: rocprofv3 --pmc FETCH_SIZE "
                  "(x2.0) + WRITE_SIZE (x1.0), KiB per dispatch of this kernel in `bench.py --skip-cpu --skip-machines "
                  "--eager-timing --steps 5 --warmup 3 --only convnet,elementwise,yolo`")
# SQ_VALU_MFMA_BUSY_CYCLES / (128 * GRBM_GUI_ACTIVE) of the same kernels in a rocprofv3 --pmc run of this
# script (eager launches, one at a time: launch and drain are inside GUI_ACTIVE, clocks are not sustained)
MEASURED_MFMA_BUSY = {"conv0": 0.036, "conv1": 0.310, "conv2": 0.236, "conv0+conv1": 0.325}
MFMA_BUSY_SOURCE = ("constant from profiles/mfma_utilisation_pmc.txt: SQ_VALU_MFMA_BUSY_CYCLES / (128 x GRBM_GUI_ACTIVE) "
                    "per dispatch in `bench.py --skip-cpu --skip-machines --eager-timing --steps 5 --warmup 3 --only "
                    "convnet,linalg,yolo` (one eager launch at a time; launch and drain are inside GUI_ACTIVE)")
CONV_KERNEL_NAME = {"conv0": "k_conv3x3_rows1<true>", "conv1": "k_conv3x3_rows<8,3,2,true,16,1088,4,false>",
                    "conv2": "k_conv3x3_rows<16,1,1,true,9,336,8,false>",
                    "conv0+conv1": "k_conv3x3_rows<8,3,2,true,16,1088,4,true>"}
# gh_conv2d_route's answer -> the kernel family it names
CONV_ROUTE_KERNEL = {0: "k_conv3x3_direct", 1: "k_conv3x3_small", 2: "k_conv3x3_patch", 3: "k_conv3x3_wide",
                     4: "k_conv1x1", 5: "k_conv3x3_tiled", 6: "k_conv2d_gather", 7: "k_conv3x3_rows", 8: "k_conv3x3_rows1"}
# where the launch time of the dominant kernel can be checked: a kernel trace of the convnet legs alone
TRACE_SOURCE = ("profiles/convnet_step_kernel_trace.txt: rocprofv3 --kernel-trace --stats of `bench.py --skip-cpu "
                "--skip-machines --only convnet --sustain-ms 15 --in-flight 2`, average duration of this kernel")

CONVNET_LAYERS = [  # (name, B-relative shape) of configuration 4
    ("conv0", 1, 28, 32), ("conv1", 32, 14, 64), ("conv2", 64, 7, 128),
]


def bench_convnet_kernels(ctx, batch, iters):
    """Per-kernel time of the conv layers of the convnet step (for the roofline object):
    the commands the step itself issues - conv + ReLU + 2x2 max-pool in one launch where
    the library offers it, and layers 0 and 1 as one launch where it folds them
    ("conv0+conv1"; "in_step" marks the entries a fused step runs).  FLOPs are the
    convolutions' own (2*B*oh*ow*F*C*9)."""
    from gorgonia_amd import device as D, synth
    out = {}
    for name, cin, hw, f in CONVNET_LAYERS:
        x = ctx.upload(synth.uniform01(1, (batch * cin * hw * hw,)))
        w = ctx.upload(synth.normal(2, (f * cin * 9,)))
        y = ctx.malloc(batch * f * hw * hw * 4)
        plain = D.cmd_conv2d(x, w, y, batch, cin, hw, hw, f, 3, 3, (1, 1))
        pool = bool(ctx.lib.gh_conv2d_can_pool(plain))
        route = int(ctx.lib.gh_conv2d_route(plain))
        ms = time_cmds(ctx, [D.cmd_conv2d(x, w, y, batch, cin, hw, hw, f, 3, 3, (1, 1), act="relu", pool2=pool)], iters)
        fl = 2.0 * batch * hw * hw * f * cin * 9
        out_hw = (hw // 2) if pool else hw
        nb = 4 * (batch * cin * hw * hw + f * cin * 9 + batch * f * out_hw * out_hw)
        out[name] = {"us": round(ms * 1e3, 2), "TFLOPs": round(fl / ms / 1e9, 2), "flop": fl,
                     "GBps": round(nb / ms / 1e6, 1), "bytes": nb, "pool_fused": pool, "route": CONV_ROUTE_KERNEL.get(route, str(route)),
                     "us_short_burst": round(time_cmds.last_burst_ms * 1e3, 2), "in_step": True}
        for q in (x, w, y):
            ctx.free(q)
    # layers 0 and 1 in one launch: the first layer's result is made in LDS and never stored
    (_, c0, hw0, f0), (_, c1, hw1, f1) = CONVNET_LAYERS[0], CONVNET_LAYERS[1]
    probe = D.cmd_conv2d(1, 1, 1, batch, c1, hw1, hw1, f1, 3, 3, (1, 1))
    if c0 == 1 and f0 == c1 and hw0 == 2 * hw1 and ctx.lib.gh_conv2d_can_pre(probe) and out["conv0"]["pool_fused"]:
        x = ctx.upload(synth.uniform01(1, (batch * hw0 * hw0,)))
        w0 = ctx.upload(synth.normal(2, (f0 * 9,)))
        w1 = ctx.upload(synth.normal(3, (f1 * c1 * 9,)))
        y = ctx.malloc(batch * f1 * hw1 * hw1 * 4)
        pool = out["conv1"]["pool_fused"]
        ms = time_cmds(ctx, [D.cmd_conv2d(x, w1, y, batch, c1, hw1, hw1, f1, 3, 3, (1, 1), act="relu", pool2=pool, pre=w0)], iters)
        fl = out["conv0"]["flop"] + out["conv1"]["flop"]
        out_hw = (hw1 // 2) if pool else hw1
        nb = 4 * (batch * hw0 * hw0 + f0 * 9 + f1 * c1 * 9 + batch * f1 * out_hw * out_hw)
        out["conv0+conv1"] = {"us": round(ms * 1e3, 2), "TFLOPs": round(fl / ms / 1e9, 2), "flop": fl,
                              "GBps": round(nb / ms / 1e6, 1), "bytes": nb, "pool_fused": pool, "route": out["conv1"]["route"],
                              "us_short_burst": round(time_cmds.last_burst_ms * 1e3, 2), "in_step": True}
        out["conv0"]["in_step"] = out["conv1"]["in_step"] = False
        for q in (x, w0, w1, y):
            ctx.free(q)
    return out


def bench_convnet(steps, warmup, batch=128, resident_input=True, graph_replay=True, dtype=np.float32,
                  reupload_all=False, borrow_input=False):
    from gorgonia_amd import configs, graph as G
    inp = {k: v.astype(dtype) for k, v in configs.convnet_inputs(batch).items()}
    g = G.NewGraph()
    # same graph as configs.build_convnet, with the input batch optionally resident
    h = xin = G.NewTensor(g, inp["x"], resident=resident_input)
    if borrow_input:   # the batch is written into the machine's pinned buffer (a loader's job), not copied there
        G.LetBorrowed(xin)
    for i in range(3):
        w = G.NewTensor(g, inp[f"w{i}"], True)
        h = G.MaxPool2D(G.Rectify(G.Conv2d(h, w, (3, 3), (1, 1), (1, 1), (1, 1))), (2, 2), (0, 0), (2, 2))
    h = G.Reshape(h, (batch, 128 * 3 * 3))
    h = G.Rectify(G.Mul(h, G.NewTensor(g, inp["w3"], True)))
    out = G.Read(G.SoftMax(G.Mul(h, G.NewTensor(g, inp["w4"], True))))
    # reupload_all: every input, weights too, crosses the bus on every run as the
    # reference's tape machine does it (vm_tape_cuda.go:220-243)
    m = G.NewTapeMachine(g, graph_replay=graph_replay, fuse_activations=True, reupload_resident=reupload_all)
    if borrow_input:
        m.input(xin)[...] = inp["x"]
    warm_up(m, warmup)
    eng = m.engine()
    eng.DoWork()
    t0 = time.perf_counter()
    m.RunAllN(steps)   # the steps back to back as a compiled caller would issue them
    eng.DoWork()
    dt = time.perf_counter() - t0
    result = out.copy()
    launches = m.graph_launches()
    if graph_replay == "measured":
        VERDICTS[f"convnet{'_f64' if dtype == np.float64 else ''}{'' if resident_input else '_input_h2d'}"
                 f"{'_all_h2d' if reupload_all else ''}{'_borrowed' if borrow_input else ''}"] = m.segment_verdict()
    m.Close()
    return dt / steps * 1e3, result, inp, launches


def bench_convnet_machines(steps, warmup, count=2, batch=128):
    """Throughput of `count` tape machines (each its own engine, stream and weights, each
    running the same synchronous RunAll loop on its own batch) in as many host threads -
    what goroutines with one VM each would do.  A step's launch and wait latency then
    overlaps the other machines' kernels.  Returns (images/s, every machine's output)."""
    import threading
    from gorgonia_amd import configs, graph as G
    inp = configs.convnet_inputs(batch)
    machines = []
    for _ in range(count):
        g, outs = configs.build_convnet(inp, resident_input=True)
        m = G.NewTapeMachine(g, graph_replay=replay_mode(), fuse_activations=True)
        warm_up(m, warmup)
        machines.append((g, m, outs))
    gate = threading.Barrier(count + 1)

    def loop(m):
        gate.wait()
        m.RunAllN(steps)
        gate.wait()

    threads = [threading.Thread(target=loop, args=(m,)) for _, m, _ in machines]
    for t in threads:
        t.start()
    gate.wait()
    t0 = time.perf_counter()
    gate.wait()
    dt = time.perf_counter() - t0
    for t in threads:
        t.join()
    results = [outs["out"].copy() for _, _, outs in machines]
    for _, m, _ in machines:
        m.Close()
    return count * steps * batch / dt, results


def bench_yolo(steps, warmup, resident_input=True, borrow_output=True, borrow_input=False, graph_replay=None):
    """Config 5: Tiny-YOLO-v2-shaped forward, batch 8 x 3 x 416 x 416, on the tape
    machine with conv+BatchNorm+LeakyReLU(+MaxPool) folded, graph replay,
    weights and input resident.  borrow_output: the 8 x 425 x 13 x 13 result (2.3 MB) is read
    where the last kernel wrote it, in the machine's pinned host buffer (ReadBorrowed);
    otherwise Read copies it from there into the caller's array on every step."""
    from gorgonia_amd import configs, graph as G
    inp = configs.yolo_inputs(8, 416)
    g, outs = configs.build_yolo(inp, resident_input=resident_input, borrow_output=borrow_output,
                                 borrow_input=borrow_input)
    m = G.NewTapeMachine(g, graph_replay=replay_mode() if graph_replay is None else graph_replay, fuse_activations=True)
    if borrow_input:
        m.input(g.x_node)[...] = inp["x"]
    warm_up(m, warmup)
    eng = m.engine()
    eng.DoWork()
    t0 = time.perf_counter()
    m.RunAllN(steps)   # the steps back to back as a compiled caller would issue them
    eng.DoWork()
    dt = time.perf_counter() - t0
    result = (m.value(outs["out"]) if borrow_output else outs["out"]).copy()
    if graph_replay is None:
        VERDICTS["yolo" if resident_input else "yolo_input_h2d"] = m.segment_verdict()
    m.Close()
    return dt / steps * 1e3, result, inp


def bench_mlp(steps, warmup, resident_input=True):
    """Config 1: MLP 256 x 784 -> 300 -> 100 -> 10 forward on the tape machine (three
    dense layers, ReLU and SoftMax folded into the products' epilogues), graph replay,
    weights and input resident."""
    from gorgonia_amd import configs, graph as G
    inp = configs.mlp_inputs(256)
    g, outs = configs.build_mlp(inp, resident_input=resident_input)
    m = G.NewTapeMachine(g, graph_replay=replay_mode(), fuse_activations=True)
    warm_up(m, warmup)
    eng = m.engine()
    eng.DoWork()
    t0 = time.perf_counter()
    m.RunAllN(steps)   # the steps back to back as a compiled caller would issue them
    eng.DoWork()
    dt = time.perf_counter() - t0
    result = outs["out"].copy()
    VERDICTS["mlp" if resident_input else "mlp_input_h2d"] = m.segment_verdict()
    m.Close()
    return dt / steps * 1e3, result, inp


def bench_convnet_train(steps, warmup, batch=128, dtype=np.float32):
    """Config 4 as a training step: forward, every layer's gradient, RMSProp
    update (examples/convnet/main.go:195) of the resident weights; only the
    128x10 output leaves the device."""
    from gorgonia_amd import configs, graph as G
    inp = {k: v.astype(dtype) for k, v in configs.convnet_inputs(batch).items()}
    onehot = np.zeros((batch, 10), dtype)
    onehot[np.arange(batch), np.arange(batch) % 10] = 1.0
    g, outs = configs.build_convnet_train(inp, onehot, 0.01, read_grads=False, solver="rmsprop")
    m = G.NewTapeMachine(g, graph_replay=replay_mode(), fuse_activations=True)
    warm_up(m, warmup)
    eng = m.engine()
    eng.DoWork()
    t0 = time.perf_counter()
    m.RunAllN(steps)   # the steps back to back as a compiled caller would issue them
    eng.DoWork()
    dt = time.perf_counter() - t0
    VERDICTS["convnet_train" + ("_f64" if dtype == np.float64 else "")] = m.segment_verdict()
    m.Close()
    return dt / steps * 1e3, inp, onehot


def bench_backward_kernels(ctx, iters):
    """Per-kernel time of the backward passes at the convnet's and the
    yolo-shaped stack's layer shapes."""
    from gorgonia_amd import device as D, synth
    out = {}
    for name, (B, C, HW, F) in {"convnet_conv1": (128, 32, 14, 64), "convnet_conv2": (128, 64, 7, 128),
                                "yolo_conv3": (8, 64, 52, 128), "yolo_conv6": (8, 512, 13, 1024)}.items():
        x = ctx.upload(synth.uniform01(1, (B * C * HW * HW,)))
        w = ctx.upload(synth.normal(2, (F * C * 9,)))
        dy = ctx.upload(synth.normal(3, (B * F * HW * HW,)))
        dx, dw = ctx.malloc(B * C * HW * HW * 4), ctx.malloc(F * C * 9 * 4)
        fl = 2.0 * B * HW * HW * F * C * 9
        ms = time_cmds(ctx, [D.cmd_conv2d_bwd_filter(x, dy, dw, B, C, HW, HW, F, 3, 3, (1, 1))], iters)
        out[name + "_filter_grad"] = {"us": round(ms * 1e3, 2), "TFLOPs": round(fl / ms / 1e9, 2)}
        ms = time_cmds(ctx, [D.cmd_conv2d_bwd_data(dy, w, dx, B, C, HW, HW, F, 3, 3, (1, 1))], iters)
        out[name + "_image_grad"] = {"us": round(ms * 1e3, 2), "TFLOPs": round(fl / ms / 1e9, 2)}
        for q in (x, w, dy, dx, dw):
            ctx.free(q)
    B, C, HW = 8, 32, 208
    n = B * C * HW * HW
    x, dy = ctx.upload(synth.normal(4, (n,))), ctx.upload(synth.normal(5, (n // 4,)))
    dx = ctx.malloc(n * 4)
    ms = time_cmds(ctx, [D.cmd_maxpool2d_bwd(x, dy, dx, B, C, HW, HW, 2, 2, (0, 0), (2, 2))], iters)
    out["maxpool_bwd_8x32x208x208"] = {"us": round(ms * 1e3, 2), "GBps": round(4 * (2 * n + n // 4) / ms / 1e6, 1)}
    g = ctx.upload(synth.normal(6, (n,)))
    st = [ctx.upload(np.zeros(C, np.float32)) for _ in range(4)]
    ms = time_cmds(ctx, [D.cmd_bn_train(x, dx, st[0], st[1], st[2], st[3], B, C, HW * HW, 1e-5, 0.9)], iters)
    out["bn_train_8x32x208x208"] = {"us": round(ms * 1e3, 2), "GBps": round(4 * 4 * n / ms / 1e6, 1),
                                    "bytes": "3 reads + 1 write of x"}
    ms = time_cmds(ctx, [D.cmd_bn_bwd(x, g, dx, st[2], st[3], B, C, HW * HW, 1e-5)], iters)
    out["bn_bwd_8x32x208x208"] = {"us": round(ms * 1e3, 2), "GBps": round(4 * 5 * n / ms / 1e6, 1),
                                  "bytes": "2 reads of x and dy + 1 write"}
    for q in [x, dy, dx, g] + st:
        ctx.free(q)
    return out


def cpu_baseline_convnet(inp, budget_s=12.0):
    """The CPU oracle's forward pass of the same configuration on the host cores."""
    from oracle import binding as O, forward as F
    threads = min(os.cpu_count() or 1, 16)
    O.set_threads(threads)
    t0 = time.perf_counter()
    ref = F.convnet(inp)
    one = time.perf_counter() - t0
    reps = 1
    while (reps + 1) * one < budget_s and reps < 1000:   # about 12 s of host work
        F.convnet(inp)
        reps += 1
    total = time.perf_counter() - t0
    O.set_threads(1)
    return ref, inp["x"].shape[0] * reps / total, threads, reps


def cpu_baseline_micro():
    """Oracle timings of the other two metric parts on a bounded sample."""
    from oracle import binding as O
    from gorgonia_amd import synth
    res = {}
    n = 1 << 22  # 4 Mi elements of the 16 Mi-element chain, single thread like the reference's loops
    x, y = synth.uniform(1, (n,), -4, 4), synth.uniform(2, (n,), -4, 4)
    b = synth.uniform(3, (4096,), -4, 4)
    t0 = time.perf_counter()
    z = O.unary("sigmoid", O.bcast_binop("add", O.binop("mul", "vv", x, y), b, n // 4096, 4096, 1))
    O.unary("tanh", z)
    O.binop("pow", "vs", z, np.array([2.0], np.float32))
    dt = time.perf_counter() - t0
    res["elementwise_chain_GBps"] = round(738_213_888 * (n / (4096 * 4096)) / dt / 1e9, 3)
    res["elementwise_sample"] = "4 Mi of 16 Mi elements, 1 thread"
    threads = min(os.cpu_count() or 1, 16)
    O.set_threads(threads)
    m, k, nn = 256, 4096, 4096  # a 256-row slab of the 4096^3 product
    A, B = synth.normal(4, (m, k)), synth.normal(5, (k, nn))
    t0 = time.perf_counter()
    O.gemm(A, B)
    dt = time.perf_counter() - t0
    O.set_threads(1)
    res["sgemm_TFLOPs"] = round(2.0 * m * k * nn / dt / 1e12, 4)
    res["sgemm_sample"] = f"256x4096x4096 slab, {threads} threads"
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--skip-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--skip-machines", action="store_true",
                    help="leave out the runs of several tape machines in parallel host threads (kernel traces: "
                         "overlapping kernels stretch each other's durations)")
    ap.add_argument("--eager-timing", action="store_true",
                    help="launch every kernel eagerly, no hipGraph (use under rocprofv3 --pmc)")
    ap.add_argument("--short-timing", action="store_true",
                    help="time each kernel over one graph replay only (no sustained-clock loop): for runs under a "
                         "tracing profiler, which records every launch")
    ap.add_argument("--sustain-ms", type=float, default=None,
                    help="length of the warm-up and of the timed loop of each kernel measurement (default 40)")
    ap.add_argument("--in-flight", type=int, default=None,
                    help="graph replays queued between two host waits of a kernel measurement (default 32)")
    ap.add_argument("--only", default="", help="comma list of: convnet,elementwise,linalg,mlp,yolo,train")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this engine runs on one GPU; --gpus must be 1 (no multi-GPU path is built)")
    only = set(filter(None, a.only.split(",")))
    global EAGER_TIMING, SUSTAIN_MS
    EAGER_TIMING = a.eager_timing
    if a.short_timing:
        SUSTAIN_MS = 0.0
    elif a.sustain_ms is not None:
        SUSTAIN_MS = a.sustain_ms
    global IN_FLIGHT
    if a.in_flight:
        IN_FLIGHT = max(1, a.in_flight)

    from gorgonia_amd.device import Context
    ctx = Context(0, 0)
    info = ctx.info()
    log(f"device {info.arch.decode()} CUs={info.compute_units}")

    ms_step, gpu_out, inp, launches = bench_convnet(a.steps, a.warmup, graph_replay=replay_mode())
    images_s = 128 / ms_step * 1e3
    log(f"convnet: {ms_step:.4f} ms/step  {images_s:.0f} images/s  (graph launches {launches})")
    two_images_s = four_images_s = None
    two_out = four_out = []
    if not a.skip_machines:
        two_images_s, two_out = bench_convnet_machines(a.steps, a.warmup, 2)
        four_images_s, four_out = bench_convnet_machines(a.steps, a.warmup, 4)
        log(f"convnet, machines in parallel host threads: two {two_images_s:.0f}, four {four_images_s:.0f} images/s")
    ms_h2d, _, _, _ = bench_convnet(max(20, a.steps // 4), a.warmup, resident_input=False, graph_replay=replay_mode())
    ms_h2d_b, out_h2d_b, _, _ = bench_convnet(max(20, a.steps // 4), a.warmup, resident_input=False,
                                              graph_replay=replay_mode(), borrow_input=True)
    ms_h2d_all, out_h2d_all, _, _ = bench_convnet(max(20, a.steps // 4), a.warmup, resident_input=False,
                                                  reupload_all=True, graph_replay=replay_mode())
    ms_eager, _, _, _ = bench_convnet(max(20, a.steps // 4), a.warmup, graph_replay=False)
    ms_replay, _, _, _ = bench_convnet(max(20, a.steps // 4), a.warmup, graph_replay=not EAGER_TIMING)

    yolo = None
    if not only or "yolo" in only:
        ms_yolo, yolo_out, yolo_inp = bench_yolo(max(20, a.steps // 4), a.warmup)
        ms_yolo_h2d, _, _ = bench_yolo(max(10, a.steps // 8), a.warmup, resident_input=False)
        ms_yolo_copy, yolo_out_copy, _ = bench_yolo(max(10, a.steps // 8), a.warmup, borrow_output=False)
        ms_yolo_h2d_b, yolo_out_b, _ = bench_yolo(max(10, a.steps // 8), a.warmup, resident_input=False, borrow_input=True)
        # every command submitted one by one (no hipGraph): the host cost of the library's kernel plans shows here
        ms_yolo_eager, yolo_out_eager, _ = bench_yolo(max(10, a.steps // 8), a.warmup, graph_replay=False)
        yolo = {"ms_per_step": round(ms_yolo, 4), "images_s": round(8 / ms_yolo * 1e3, 1),
                "TFLOPs": round(31_080_857_600 / ms_yolo / 1e9, 2), "flop_per_step": 31_080_857_600,
                "ms_per_step_with_input_h2d": round(ms_yolo_h2d, 4),
                "ms_per_step_with_input_h2d_from_borrowed_pinned_buffer": round(ms_yolo_h2d_b, 4),
                "borrowed_input_output_equals_resident": bool(np.array_equal(yolo_out, yolo_out_b)),
                "output": "read in the machine's pinned buffer (ReadBorrowed), 2298400 bytes",
                "ms_per_step_eager_no_graph": round(ms_yolo_eager, 4),
                "eager_output_equals_replayed": bool(np.array_equal(yolo_out, yolo_out_eager)),
                "ms_per_step_output_copied_to_caller": round(ms_yolo_copy, 4),
                "copied_output_equals_borrowed": bool(np.array_equal(yolo_out, yolo_out_copy))}
        log(f"yolo-shaped: {ms_yolo:.4f} ms/step  {8 / ms_yolo * 1e3:.0f} images/s")

    mlp = None
    if not only or "mlp" in only:
        ms_mlp, mlp_out, mlp_inp = bench_mlp(a.steps, a.warmup)
        ms_mlp_h2d, _, _ = bench_mlp(max(20, a.steps // 4), a.warmup, resident_input=False)
        mlp = {"ms_per_step": round(ms_mlp, 5), "images_s": round(256 / ms_mlp * 1e3, 1), "flop_per_step": 136_294_400,
               "ms_per_step_with_input_h2d": round(ms_mlp_h2d, 5)}
        log(f"mlp: {ms_mlp:.4f} ms/step  {256 / ms_mlp * 1e3:.0f} rows/s")

    train = None
    if not only or "train" in only:
        ms_train, train_inp, train_y = bench_convnet_train(max(20, a.steps // 4), a.warmup)
        train = {"ms_per_step": round(ms_train, 4), "images_s": round(128 / ms_train * 1e3, 1)}
        log(f"convnet training step: {ms_train:.4f} ms/step  {128 / ms_train * 1e3:.0f} images/s")

    # the same network in float64, the default dtype of the reference's example
    # (examples/convnet/main.go:28): forward and training step on the fp64 matrix cores
    f64 = None
    if not only or "float64" in only:
        n64 = max(20, a.steps // 4)
        ms64, out64, inp64, _ = bench_convnet(n64, a.warmup, graph_replay=replay_mode(), dtype=np.float64)
        ms64t, _, _ = bench_convnet_train(n64, a.warmup, dtype=np.float64)
        f64 = {"forward_ms_per_step": round(ms64, 4), "forward_images_s": round(128 / ms64 * 1e3, 1),
               "training_ms_per_step": round(ms64t, 4), "training_images_s": round(128 / ms64t * 1e3, 1)}
        if not a.skip_cpu:
            from oracle import binding as O
            O.set_threads(min(16, os.cpu_count() or 1))
            h = inp64["x"]
            for i in range(3):
                h = O.conv2d(h, inp64[f"w{i}"], (1, 1), (1, 1), (1, 1))
                h = O.maxpool2d(O.relu(h).reshape(h.shape), (2, 2), (0, 0), (2, 2))
            h = O.relu(h.reshape(128, -1) @ inp64["w3"]).reshape(128, -1)
            ref64 = O.softmax(h @ inp64["w4"])
            O.set_threads(1)
            f64["forward_rel_frobenius_vs_oracle"] = float(np.linalg.norm(out64 - ref64) / np.linalg.norm(ref64))
        log(f"float64 convnet: forward {ms64:.4f} ms/step, training {ms64t:.4f} ms/step")

    iters = 30
    conv_k = bench_convnet_kernels(ctx, 128, iters) if not only or "convnet" in only else {}
    elem = bench_elementwise(ctx, iters) if not only or "elementwise" in only else {}
    lin = bench_linalg(ctx, iters) if not only or "linalg" in only else {}
    bwd = bench_backward_kernels(ctx, iters) if not only or "train" in only else {}
    ctx.close()

    # the dominant kernel of the step: the conv layer with the largest time
    roofline = None
    if conv_k:
        name = max((k for k in conv_k if conv_k[k]["in_step"]), key=lambda k: conv_k[k]["us"])
        r = conv_k[name]
        kname = CONV_KERNEL_NAME[name]
        if not kname.startswith(r["route"]):   # the library chose another kernel than the one the constants are for
            kname = r["route"] + " (traffic and mfma_busy constants are not this kernel's)"
        tail = "ReLU and the 2x2 max-pool in the epilogue" if r["pool_fused"] else "ReLU in the epilogue"
        if name == "conv0+conv1":
            tail += "; conv0 + ReLU + pool computed in LDS in front of it, its result never stored"
        roofline = {"kernel": f"{kname}: {name} of the convnet step with {tail}", "bound": "mfma",
                    "achieved": r["TFLOPs"], "peak": MFMA_F32_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(r["TFLOPs"] / MFMA_F32_PEAK_TFLOPS, 4),
                    "traffic": int(MEASURED_TRAFFIC_BYTES[name]) if name in MEASURED_TRAFFIC_BYTES else None,
                    "traffic_source": TRAFFIC_SOURCE,
                    "mfma_busy": MEASURED_MFMA_BUSY.get(name), "mfma_busy_source": MFMA_BUSY_SOURCE,
                    "launch_us_source": "HIP events around back-to-back launches of this kernel on the library's "
                                        "stream in this run; cross-check: " + TRACE_SOURCE,
                    "launch_us": r["us"], "launch_us_short_burst": r.get("us_short_burst"),
                    "algorithmic_flop": r["flop"]}

    cpu = None
    parity = None
    if not a.skip_cpu:
        ref, cpu_images_s, threads, reps = cpu_baseline_convnet(inp)
        err = float(np.linalg.norm(gpu_out.astype(np.float64) - ref) / np.linalg.norm(ref))
        parity = {"convnet_rel_frobenius_vs_oracle": err, "tolerance": 1e-5, "ok": err <= 1e-5}
        cpu = {"value": round(cpu_images_s, 1), "unit": "images/s", "cores": threads, "kind": "port",
               "sample": f"{reps} forward passes of the same 128-image batch (CPU oracle, OpenMP)"}
        cpu.update(cpu_baseline_micro())
        if train is not None:
            from oracle import binding as O, forward as F
            O.set_threads(threads)
            t0 = time.perf_counter()
            reps_t = 0
            while reps_t < 20 and time.perf_counter() - t0 < 6.0:
                F.convnet_train_step(train_inp, train_y, 0.01)
                reps_t += 1
            tdt = time.perf_counter() - t0
            O.set_threads(1)
            cpu["convnet_train_images_s"] = round(128 * reps_t / tdt, 1)
            cpu["convnet_train_sample"] = f"{reps_t} training steps of the same 128-image batch, {threads} threads"
        if mlp is not None:
            from oracle import binding as O, forward as F
            O.set_threads(threads)
            t0 = time.perf_counter()
            reps_m = 0
            while reps_m < 200 and time.perf_counter() - t0 < 3.0:
                mref = F.mlp(mlp_inp)
                reps_m += 1
            mdt = time.perf_counter() - t0
            O.set_threads(1)
            cpu["mlp_images_s"] = round(256 * reps_m / mdt, 1)
            cpu["mlp_sample"] = f"{reps_m} forward passes of the same 256-row batch, {threads} threads"
            merr = float(np.linalg.norm(mlp_out.astype(np.float64) - mref) / np.linalg.norm(mref))
            parity["mlp_rel_frobenius_vs_oracle"] = merr
            parity["ok"] = parity["ok"] and merr <= 1e-5
        if yolo is not None:
            from oracle import binding as O, forward as F
            O.set_threads(threads)
            t0 = time.perf_counter()
            yref = F.yolo(yolo_inp)
            ydt = time.perf_counter() - t0
            O.set_threads(1)
            cpu["yolo_images_s"] = round(8 / ydt, 2)
            cpu["yolo_sample"] = f"1 forward pass of the same 8-image batch, {threads} threads"
            yerr = float(np.linalg.norm(yolo_out.astype(np.float64) - yref) / np.linalg.norm(yref))
            parity["yolo_rel_frobenius_vs_oracle"] = yerr
            parity["ok"] = parity["ok"] and yerr <= 1e-5

    line = {
        "metric": "convnet fwd images/s (1 GPU); elementwise HBM GB/s; SGEMM TFLOP/s",
        "value": round(images_s, 1), "unit": "images/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "convnet forward, float32 NCHW batch 128x1x28x28 (config 4): "
                               "3x[Conv2d 3x3 pad1 + ReLU + MaxPool 2x2] -> Dense 625 ReLU -> Dense 10 SoftMax; "
                               "tape machine, one segment of four commands (layers 0 and 1 folded into one), submitted "
                               "plainly - segments of five commands and more run the quicker of plain submits and "
                               "hipGraph replay, timed by the machine on its first runs; weights and input resident, "
                               "every step ends with the output on the host",
                   "batch": 128, "flop_per_step": 2_093_410_816,
                   "untimed_warmup": f"max({a.warmup}, {WARM_RUNS}) steps, then steps until {SUSTAIN_MS:g} ms have passed "
                                     "(the clocks' ramp), then the timed steps"},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "extra": {
            "elementwise_hbm_GBps": elem.get("chain_GBps"), "elementwise_frac_hbm": elem.get("frac_hbm"),
            "sgemm_TFLOPs": lin.get("sgemm_4096", {}).get("TFLOPs"),
            "sgemm_frac_mfma": lin.get("sgemm_4096", {}).get("frac_mfma"),
            "convnet_ms_per_step_with_input_h2d": round(ms_h2d, 5),
            "convnet_images_s_with_input_h2d": round(128 / ms_h2d * 1e3, 1),
            "convnet_ms_per_step_with_input_h2d_from_borrowed_pinned_buffer": round(ms_h2d_b, 5),
            "convnet_borrowed_input_output_equals_resident": bool(np.array_equal(out_h2d_b, gpu_out)),
            "convnet_ms_per_step_all_inputs_reuploaded": round(ms_h2d_all, 5),
            "convnet_images_s_all_inputs_reuploaded": round(128 / ms_h2d_all * 1e3, 1),
            "convnet_all_inputs_reuploaded_bytes_per_step": int(sum(v.nbytes for v in inp.values())),
            "convnet_reuploaded_output_equals_resident": bool(np.array_equal(out_h2d_all, gpu_out)),
            "convnet_ms_per_step_eager_no_graph": round(ms_eager, 5),
            "convnet_ms_per_step_graph_replay_always": round(ms_replay, 5),
            "segment_run_as": dict(VERDICTS),
            "convnet_images_s_two_machines_two_host_threads": two_images_s and round(two_images_s, 1),
            "convnet_images_s_four_machines_four_host_threads": four_images_s and round(four_images_s, 1),
            "convnet_parallel_machines_outputs_equal_single": (bool(all(np.array_equal(o, gpu_out) for o in two_out + four_out))
                                                               if two_out else None),
            "mlp_forward": mlp, "yolo_shaped_forward": yolo, "convnet_training_step": train, "convnet_float64": f64, "backward_kernels": bwd, "convnet_kernels": conv_k, "elementwise": elem, "linalg": lin, "parity": parity,
        },
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
