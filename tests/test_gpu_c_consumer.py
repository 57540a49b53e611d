"""A consumer of the C ABI that is not Python and not C++: tests/c_consumer/consumer.c is C99,
fills a gh_cmd[] for a small forward pass, makes one gh_submit and writes what the device stored.
The same commands submitted through the ctypes binding must give the same bytes, and both must
agree with the CPU oracle."""
import os
import subprocess

import numpy as np
import pytest

from gorgonia_amd import _ffi, synth
from gorgonia_amd import device as D
from oracle import binding as O
from tests.util import assert_bits_equal, rel_frobenius, ulp_diff

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "c_consumer", "consumer.bin")

B, C, H, W, F, PH, PW, NO, NE = 4, 3, 12, 12, 8, 6, 6, 10, 1000


def test_plain_c_consumer_matches_ctypes_path_and_oracle(ctx, tmp_path):
    assert os.path.exists(BIN), "tests/c_consumer/consumer.bin is built by `python -m gorgonia_amd.build`"
    x = synth.uniform(21, (B, C, H, W), -1, 1)
    w = synth.he_normal(22, (F, C, 3, 3))
    wd = synth.he_normal(23, (F * PH * PW, NO))
    bias = synth.normal(24, (NO,), 0.0, 0.5)
    a = synth.uniform(25, (NE,), -3, 3)
    b = synth.uniform(26, (NE,), -3, 3)
    fin, fout = tmp_path / "in.bin", tmp_path / "out.bin"
    np.concatenate([v.reshape(-1) for v in (x, w, wd, bias, a, b)]).astype(np.float32).tofile(fin)
    print("running", BIN, flush=True)
    p = subprocess.run([BIN, str(fin), str(fout)], capture_output=True, text=True, timeout=100)
    assert p.returncode == 0, p.stdout + p.stderr
    assert "6 commands in one gh_submit" in p.stdout
    got = np.fromfile(fout, dtype=np.float32)
    sizes = [B * F * H * W, B * F * PH * PW, B * NO, NE]
    assert got.size == sum(sizes)
    c_conv, c_pool, c_prob, c_e = np.split(got, np.cumsum(sizes)[:-1])

    # the same six commands through the ctypes binding, one submit
    dx, dw, dwd, dbias, da, db = (ctx.upload(v) for v in (x, w, wd, bias, a, b))
    dconv, dpool, dlogit, dprob, de = (ctx.malloc(4 * n) for n in (sizes[0], sizes[1], sizes[2], sizes[2], NE))
    ctx.run([
        D.cmd_conv2d(dx, dw, dconv, B, C, H, W, F, 3, 3, (1, 1), (1, 1), (1, 1), act="relu"),
        D.cmd_maxpool2d(dconv, dpool, B, F, H, W, 2, 2, (0, 0), (2, 2)),
        D.cmd_gemm(dpool, dwd, dlogit, B, NO, F * PH * PW, bias=dbias),
        D.cmd_softmax(dlogit, dprob, B, NO),
        D.cmd_bin("mul", "vv", da, db, NE, dst=de),
        D.cmd_unary("sigmoid", de, NE),
    ])
    p_conv, p_pool = ctx.d2h(dconv, (sizes[0],)), ctx.d2h(dpool, (sizes[1],))
    p_prob, p_e = ctx.d2h(dprob, (sizes[2],)), ctx.d2h(de, (NE,))
    for ptr in (dx, dw, dwd, dbias, da, db, dconv, dpool, dlogit, dprob, de):
        ctx.free(ptr)
    assert_bits_equal(c_conv, p_conv, "C consumer conv+rectify == ctypes path")
    assert_bits_equal(c_pool, p_pool, "C consumer maxpool == ctypes path")
    assert_bits_equal(c_prob, p_prob, "C consumer softmax == ctypes path")
    assert_bits_equal(c_e, p_e, "C consumer sigmoid(a*b) == ctypes path")

    # and against the CPU oracle
    conv = O.relu(O.conv2d(x, w, (1, 1), (1, 1), (1, 1))).reshape(B, F, H, W)
    assert rel_frobenius(c_conv.reshape(conv.shape), conv) <= 1e-5
    dev_conv = c_conv.reshape(B, F, H, W)
    assert_bits_equal(c_pool.reshape(B, F, PH, PW), O.maxpool2d(dev_conv, (2, 2), (0, 0), (2, 2)),
                      "pool of the device's conv output")
    logits = O.gemm(c_pool.reshape(B, -1), wd) + bias[None, :]
    assert rel_frobenius(c_prob.reshape(B, NO), O.softmax(logits.astype(np.float32))) <= 1e-5
    prod = O.binop("mul", "vv", a, b)
    assert ulp_diff(c_e, O.unary("sigmoid", prod)).max() <= 2
