"""GPU parity of gh_submit_noalloc, the submit entry point that allocates nothing: the
same commands through gh_submit (scratch = the context's workspace) and through
gh_submit_noalloc (scratch = the fixed array inside the library's device image) must
store the same bits, on two calls in a row, the second with smaller operands, so stale
scratch contents from the first call cannot leak into the second.  Every operator in
the segment is one that uses scratch: a split-K product, a split-K convolution, the
filter gradient (slab sums), the image gradient (mirrored filters at the top of the
scratch) and the training-mode BatchNorm (reduction partials).  A command whose plan
needs more than the fixed array holds must be refused with GH_EINVAL, leave its output
untouched, and leave the context usable after gh_clear_error."""
import ctypes as C

import numpy as np
import pytest

from gorgonia_amd import _ffi
from gorgonia_amd import device as D
from gorgonia_amd import synth
from gorgonia_amd._ffi import GhCmd
from tests.util import assert_bits_equal

pytestmark = pytest.mark.gpu


def _submit_noalloc(ctx, cmds):
    arr = (GhCmd * len(cmds))(*cmds)
    ctx.check(ctx.lib.gh_submit_noalloc(ctx.h, arr, len(cmds)))
    ctx.sync()


def _segment(ctx, seed, m, k, n, B, Cin, F, hw):
    """Device buffers and the command list; returns (cmds, [(name, ptr, shape)], all pointers)."""
    A = synth.normal(seed + 1, (m, k))
    Bm = synth.normal(seed + 2, (k, n))
    x = synth.normal(seed + 3, (B, Cin, hw, hw))
    w = synth.normal(seed + 4, (F, Cin, 3, 3)) * np.float32(0.1)
    dy = synth.normal(seed + 5, (B, F, hw, hw))
    bx = synth.normal(seed + 6, (B, F, hw * hw))
    dA, dB, dx_, dw_, ddy, dbx = (ctx.upload(a) for a in (A, Bm, x, w, dy, bx))
    run_mean = ctx.upload(np.zeros(F, np.float32))
    run_var = ctx.upload(np.ones(F, np.float32))
    outs = [("gemm", ctx.malloc(m * n * 4), (m, n)),
            ("conv", ctx.malloc(B * F * hw * hw * 4), (B, F, hw, hw)),
            ("wgrad", ctx.malloc(F * Cin * 9 * 4), (F, Cin, 3, 3)),
            ("dgrad", ctx.malloc(B * Cin * hw * hw * 4), (B, Cin, hw, hw)),
            ("bn_y", ctx.malloc(B * F * hw * hw * 4), (B, F, hw * hw)),
            ("bn_mean", ctx.malloc(F * 4), (F,)),
            ("bn_var", ctx.malloc(F * 4), (F,))]
    o = {name: p for name, p, _ in outs}
    cmds = [D.cmd_gemm(dA, dB, o["gemm"], m, n, k),
            D.cmd_conv2d(dx_, dw_, o["conv"], B, Cin, hw, hw, F, 3, 3, pad=(1, 1)),
            D.cmd_conv2d_bwd_filter(dx_, ddy, o["wgrad"], B, Cin, hw, hw, F, 3, 3, pad=(1, 1)),
            D.cmd_conv2d_bwd_data(ddy, dw_, o["dgrad"], B, Cin, hw, hw, F, 3, 3, pad=(1, 1)),
            D.cmd_bn_train(dbx, o["bn_y"], run_mean, run_var, o["bn_mean"], o["bn_var"], B, F, hw * hw, 1e-5, 0.9)]
    reset = [D.cmd_fill(p, int(np.prod(s)), np.nan) for _, p, s in outs]
    reset += [D.cmd_fill(run_mean, F, 0.0), D.cmd_fill(run_var, F, 1.0)]
    ptrs = [dA, dB, dx_, dw_, ddy, dbx, run_mean, run_var] + [p for _, p, _ in outs]
    return cmds, reset, outs, ptrs


def _both_ways(ctx, seed, **shape):
    cmds, reset, outs, ptrs = _segment(ctx, seed, **shape)
    ctx.run(reset)
    ctx.run(cmds)                                   # gh_submit
    want = {name: ctx.d2h(p, s) for name, p, s in outs}
    ctx.run(reset)
    _submit_noalloc(ctx, cmds)                      # the entry point under test
    got = {name: ctx.d2h(p, s) for name, p, s in outs}
    for p in ptrs:
        ctx.free(p)
    for name in want:
        assert np.isfinite(want[name]).all(), f"{name}: gh_submit left unwritten or non-finite values"
        assert_bits_equal(got[name], want[name], f"gh_submit_noalloc vs gh_submit, {name} {shape}")


def test_no_alloc_submit_matches_submit_twice(ctx):
    # first call: 7 slabs of 1.3 MB for the product, 8 slabs for the convolution
    _both_ways(ctx, 100, m=576, k=1024, n=576, B=2, Cin=256, F=512, hw=13)
    # second call, smaller operands, same scratch array still holding the first call's slabs
    _both_ways(ctx, 200, m=544, k=512, n=544, B=2, Cin=128, F=256, hw=13)


def test_no_alloc_submit_refuses_what_does_not_fit(ctx):
    B, Cin, F, hw = 2, 512, 1024, 13          # the mirrored filters are 18.9 MB, the array 16 MiB
    dy = ctx.upload(synth.normal(2, (B, F, hw, hw)))
    w = ctx.upload(synth.normal(3, (F, Cin, 3, 3)))
    dx = ctx.malloc(B * Cin * hw * hw * 4)
    ctx.run(D.cmd_fill(dx, 64, 7.0))
    cmd = D.cmd_conv2d_bwd_data(dy, w, dx, B, Cin, hw, hw, F, 3, 3, pad=(1, 1))
    arr = (GhCmd * 1)(cmd)
    rc = ctx.lib.gh_submit_noalloc(ctx.h, arr, 1)
    buf = C.create_string_buffer(512)
    ctx.lib.gh_last_error(ctx.h, buf, 512)
    assert rc == _ffi.GH_EINVAL, (rc, buf.value)
    assert b"scratch" in buf.value and b"gh_submit_noalloc" in buf.value, buf.value
    ctx.clear_error()
    assert np.array_equal(ctx.d2h(dx, (64,)), np.full(64, 7.0, np.float32)), "a refused command wrote its output"
    ctx.run(cmd)                               # gh_submit takes it (64 MiB workspace)
    assert np.isfinite(ctx.d2h(dx, (B, Cin, hw, hw))).all()
    for p in (dy, w, dx):
        ctx.free(p)
