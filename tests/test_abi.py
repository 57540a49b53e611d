"""C-ABI checks that need no GPU: the library loads, exports every symbol
include/gorgonia_hip.h declares, validates commands on the host and resolves the
reference's kernel names."""
import ctypes as C
import os
import re

import pytest

from gorgonia_amd import _ffi
from gorgonia_amd import device as D

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_header_symbols_all_exported():
    hdr = open(os.path.join(ROOT, "include", "gorgonia_hip.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = set(re.findall(r"\b(gh_[a-z0-9_]+)\s*\(", hdr))
    assert declared, "no declarations parsed"
    lib = _ffi.load()
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} declared in gorgonia_hip.h but not exported"
    assert declared == set(_ffi.SYMBOLS), declared ^ set(_ffi.SYMBOLS)


def test_struct_layout_matches_header():
    assert C.sizeof(_ffi.GhCmd) == 4 + 4 + 8 * 8 + 16 * 8 + 12 * 4
    assert _ffi.GhCmd.ptr.offset == 8 and _ffi.GhCmd.dim.offset == 72 and _ffi.GhCmd.f.offset == 200


def test_kernel_name_registry():
    """Names built by constructName2/constructName1 (cuda/utils.go:114-139) and
    by elemUnaryOp.CUDADo (op_math_cuda.go:38)."""
    lib = _ffi.load()
    for fn in ["add", "sub", "mul", "div", "pow", "lt", "lte", "gt", "gte", "eq", "ne", "mod"]:
        for mode in ["vv", "vs", "sv", "ss"]:
            for bits in (32, 64):
                assert lib.gh_has_func(f"elembinop.{fn}_{mode}_f{bits}".encode()) == 1
    for fn in ["abs", "sign", "ceil", "floor", "sin", "cos", "exp", "ln", "log2", "neg", "square",
               "sqrt", "inv", "invSqrt", "inverse", "cube", "tanh", "sigmoid", "log1p", "expm1",
               "softplus"]:
        assert lib.gh_has_func(f"elemunaryop.{fn}_f32".encode()) == 1, fn
    assert lib.gh_has_func(b"misc.hasNaN_f32") == 1 and lib.gh_has_func(b"misc.hasInf_f64") == 1
    # (mod is declared by the reference engine without a kernel, elembinop.cu:201-210; it has one here)
    assert lib.gh_has_func(b"elembinop.add_vv_f16") == 0
    assert lib.gh_has_func(b"nosuch.add_vv_f32") == 0
    op, fl = C.c_uint32(), C.c_uint32()
    assert lib.gh_lookup_func(b"elembinop.sub_sv_f64", C.byref(op), C.byref(fl)) == 0
    assert op.value == _ffi.OP_ELEM_BIN
    assert fl.value == (1 | (2 << 8) | (1 << 12))


def _validate(cmd):
    lib = _ffi.load()
    arr = (_ffi.GhCmd * 1)(cmd)
    buf = C.create_string_buffer(256)
    rc = lib.gh_validate(arr, 1, buf, 256)
    return rc, buf.value.decode()


def test_validation_rejects_bad_commands():
    ok = D.cmd_gemm(0x1000, 0x2000, 0x3000, 4, 5, 6)
    assert _validate(ok)[0] == 0
    assert _validate(D.cmd_gemm(0x1000, 0x2000, 0x3000, 4, 5, 6, lda=3))[0] == _ffi.GH_EINVAL
    assert _validate(D.cmd_gemm(0, 0x2000, 0x3000, 4, 5, 6))[0] == _ffi.GH_EINVAL
    assert _validate(D.cmd_gemm(0x1000, 0x2000, 0x3000, 0, 5, 6))[0] == _ffi.GH_EINVAL
    rc, msg = _validate(D.cmd_conv2d(1, 2, 3, 1, 1, 5, 5, 1, 3, 3, stride=(0, 1)))
    assert rc == _ffi.GH_EINVAL and "strides" in msg  # nn.go:229-233 wording
    rc, msg = _validate(D.cmd_maxpool2d(1, 2, 1, 1, 2, 2, 5, 5, (0, 0), (1, 1)))
    assert rc == _ffi.GH_EINVAL and "Impossible" in msg  # nn.go:355-363
    bad = D.make_cmd(99)
    assert _validate(bad)[0] == _ffi.GH_ENOFUNC
    bad = D.make_cmd(_ffi.OP_ELEM_BIN, 200, (1, 2), (4,))
    assert _validate(bad)[0] == _ffi.GH_ENOFUNC
    bad = D.make_cmd(_ffi.OP_ELEM_BIN, _ffi.flag_dtype(3), (1, 2), (4,))
    assert _validate(bad)[0] == _ffi.GH_EINVAL


def test_version_string():
    assert b"gfx950" in _ffi.load().gh_version()


def test_headers_are_plain_c99(tmp_path):
    """cgo compiles the header as C: both headers, and the plain-C consumer that fills a gh_cmd[]
    and calls gh_submit, must pass gcc -std=c99 -pedantic -Werror (no C++-isms, no extensions)."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    assert gcc, "gcc is part of the image"
    tu = tmp_path / "both.c"
    tu.write_text('#include "gorgonia_hip.h"\n#include "gorgonia_host.h"\n'
                  "int main(void) { gh_cmd c; ghh_tensor t; (void)c; (void)t; return (int)sizeof(gh_cmd) - 248; }\n")
    flags = ["-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include")]
    p = subprocess.run([gcc] + flags + ["-fsyntax-only", str(tu)], capture_output=True, text=True)
    assert p.returncode == 0, p.stderr
    src = os.path.join(ROOT, "tests", "c_consumer", "consumer.c")
    p = subprocess.run([gcc] + flags + ["-c", src, "-o", str(tmp_path / "consumer.o")], capture_output=True, text=True)
    assert p.returncode == 0, p.stderr


ROUTE = {"direct": 0, "small": 1, "patch": 2, "wide": 3, "pointwise": 4, "tiled": 5, "gather": 6, "rows": 7, "rows1": 8}


def _route(B, C, H, W, F, k, pad, stride=(1, 1), dil=(1, 1), pool2=False):
    lib = _ffi.load()
    cmd = D.cmd_conv2d(0x10000, 0x20000, 0x30000, B, C, H, W, F, k[0], k[1], pad, stride, dil, pool2=pool2)
    return lib.gh_conv2d_route(C_byref(cmd))


def C_byref(cmd):
    return C.byref(cmd)


def test_conv_routes_of_the_benchmark_layers():
    """gh_conv2d_route: every layer of the two convolutional configurations runs on the kernel the
    design names for it."""
    # convnet (configuration 4), batch 128
    assert _route(128, 1, 28, 28, 32, (3, 3), (1, 1)) == ROUTE["rows1"]
    assert _route(128, 32, 14, 14, 64, (3, 3), (1, 1)) == ROUTE["rows"]
    assert _route(128, 64, 7, 7, 128, (3, 3), (1, 1)) == ROUTE["rows"]
    # tiny-yolo-shaped (configuration 5), batch 8
    for (Cn, F, S) in ((3, 16, 416), (16, 32, 208), (32, 64, 104)):
        assert _route(8, Cn, S, S, F, (3, 3), (1, 1)) == ROUTE["wide"], (Cn, F, S)
    for (Cn, F, S) in ((64, 128, 52), (128, 256, 26), (256, 512, 13), (512, 1024, 13)):
        assert _route(8, Cn, S, S, F, (3, 3), (1, 1)) == ROUTE["patch"], (Cn, F, S)
    assert _route(8, 1024, 13, 13, 425, (1, 1), (0, 0)) == ROUTE["pointwise"]
    # and what the specialised kernels leave: other filter sizes, strides, Conv1d
    assert _route(2, 5, 9, 9, 7, (5, 5), (2, 2)) == ROUTE["gather"]
    assert _route(2, 2, 10, 11, 3, (3, 2), (2, 1), (2, 3)) == ROUTE["gather"]
    assert _route(2, 8, 1, 64, 16, (1, 5), (0, 2), (1, 2)) == ROUTE["gather"]
    assert _route(1, 4, 7, 7, 6, (1, 1), (0, 0)) == ROUTE["gather"]          # 1x1 with few channels
    assert _route(2, 16, 66, 68, 40, (3, 3), (0, 0)) in (ROUTE["tiled"], ROUTE["wide"])
    lib = _ffi.load()
    assert lib.gh_conv2d_route(C.byref(D.cmd_relu(0x1000, 0x2000, 16))) == -1


def test_conv_route_of_every_parity_case_list():
    """The case lists of the GPU parity tests reach the kernels they are written for."""
    from tests import test_gpu_nn as T
    for (B, Cn, H, W, F, pad) in T.SMALL_IMAGE_CASES:
        assert _route(B, Cn, H, W, F, (3, 3), (pad, pad)) == ROUTE["small"], (B, Cn, H, W, F, pad)
    for (B, Cn, H, W, F, pad) in T.ROWS_CASES:
        assert _route(B, Cn, H, W, F, (3, 3), (pad, pad)) == ROUTE["rows"], (B, Cn, H, W, F, pad)
    for (B, Cn, H, W, F, pad) in T.ROWS1_CASES:
        assert _route(B, Cn, H, W, F, (3, 3), (pad, pad)) == ROUTE["rows1"], (B, Cn, H, W, F, pad)
    for (B, Cn, H, W, F, pad) in T.PATCH_CASES:
        assert _route(B, Cn, H, W, F, (3, 3), (pad, pad)) == ROUTE["patch"], (B, Cn, H, W, F, pad)
    for (B, Cn, H, W, F, pad) in T.WIDE_CASES:
        assert _route(B, Cn, H, W, F, (3, 3), (pad, pad)) == ROUTE["wide"], (B, Cn, H, W, F, pad)
    taken = [c for c in T.POINTWISE_CASES if c[1] % 256 == 0 and c[2] * c[3] >= 4]
    assert len(taken) >= 9 and len(taken) < len(T.POINTWISE_CASES)
    for (B, Cn, H, W, F) in T.POINTWISE_CASES:
        want = ROUTE["pointwise"] if (B, Cn, H, W, F) in taken else ROUTE["gather"]
        assert _route(B, Cn, H, W, F, (1, 1), (0, 0)) == want, (B, Cn, H, W, F)
    # the general lists between them reach all nine kernels
    seen = set()
    for (B, Cn, H, W, F, kh, kw, pad, stride, dil) in T.CONV_CASES:
        seen.add(_route(B, Cn, H, W, F, (kh, kw), pad, stride, dil))
    for (B, Cn, H, W, F, k, pad) in T.TAIL_CASES:
        seen.add(_route(B, Cn, H, W, F, (k, k), (pad, pad)))
    for (B, Cn, H, W, F, pad) in T.WIDE_CASES[:1]:
        seen.add(_route(B, Cn, H, W, F, (3, 3), (pad, pad)))
    assert seen == set(ROUTE.values()), seen


def test_filter_gradient_routes():
    """gh_conv2d_bwd_filter_route: the backward case table reaches all four float32 kernels, the cases written
    for the small-image kernel run on it, and the training configurations' layers run where the design says."""
    from tests import test_gpu_backward as T
    lib = _ffi.load()

    def route(B, Cn, H, W, F, kh, kw, pad, stride=(1, 1), dil=(1, 1), dtype=_ffi.F32):
        cmd = D.cmd_conv2d_bwd_filter(0x10000, 0x20000, 0x30000, B, Cn, H, W, F, kh, kw, pad, stride, dil, dtype=dtype)
        return lib.gh_conv2d_bwd_filter_route(C.byref(cmd))

    DIRECT, SMALL, GEMM, F64, SINGLE = 0, 1, 2, 3, 4
    seen = [route(*c) for c in T.CONV_BWD_CASES]
    assert set(seen) == {DIRECT, SMALL, GEMM, SINGLE}
    small = [c for c in T.CONV_BWD_CASES if c[1] % 16 == 0 and c[2] <= 16 and c[3] <= 16 and c[4] >= 16 and c[5] == 3]
    assert len(small) >= 8
    for c in small:
        assert route(*c) == SMALL, c
    assert route(128, 1, 28, 28, 32, 3, 3, (1, 1)) == SINGLE          # convnet conv0
    assert route(4, 1, 6, 6, 8, 3, 3, (0, 0)) == DIRECT               # sixteen output pixels: less than a wavefront
    assert route(2, 1, 130, 130, 8, 3, 3, (1, 1)) == DIRECT           # the padded image does not fit the LDS budget
    assert route(2, 3, 28, 28, 8, 3, 3, (1, 1)) == DIRECT
    assert route(128, 32, 14, 14, 64, 3, 3, (1, 1)) == SMALL          # conv1
    assert route(128, 64, 7, 7, 128, 3, 3, (1, 1)) == SMALL           # conv2
    assert route(8, 512, 13, 13, 1024, 3, 3, (1, 1)) == SMALL         # yolo-shaped layer 6
    assert route(8, 64, 52, 52, 128, 3, 3, (1, 1)) == GEMM            # layer 3: images too large for LDS
    assert route(128, 32, 14, 14, 64, 3, 3, (1, 1), dtype=_ffi.F64) == F64
    assert lib.gh_conv2d_bwd_filter_route(C.byref(D.cmd_relu(0x1000, 0x2000, 16))) == -1


def test_gemm_routes():
    """gh_gemm_route: the matrix-product case table reaches the small-output kernel and the tiled one with and
    without K slices; the benchmark's products run where the design says."""
    from tests import test_gpu_linalg as T
    lib = _ffi.load()

    def route(m, k, n, ta=False, tb=False, batch=1, dtype=_ffi.F32):
        sp = C.c_int(0)
        kind = lib.gh_gemm_route(C.byref(D.cmd_gemm(0x1000, 0x2000, 0x3000, m, n, k, trans_a=ta, trans_b=tb, batch=batch,
                                                    dtype=dtype)), C.byref(sp))
        return kind, sp.value

    SMALL, T128, T64, T128X64, F64 = range(5)
    seen = set()
    for (m, k, n) in T.SHAPES:
        for ta in (False, True):
            for tb in (False, True):
                kind, sp = route(m, k, n, ta, tb)
                seen.add((kind, sp > 1))
    assert {(SMALL, False), (T64, False), (T64, True)} <= seen, seen
    assert route(4096, 4096, 4096) == (T128, 1)                      # configuration 3
    assert route(512, 512, 512, batch=64) == (T128, 1)
    for (m, k, n) in ((256, 784, 300), (256, 300, 100), (256, 100, 10), (128, 1152, 625), (128, 625, 10)):
        assert route(m, k, n) == (SMALL, 1), (m, k, n)               # dense layers of configurations 1 and 4
    assert route(1152, 128, 625, ta=True) == (T64, 1)                # a dense layer's weight gradient: K = batch
    assert route(1152, 2048, 625)[0] == T64 and route(1152, 2048, 625)[1] > 1
    assert route(64, 64, 64, dtype=_ffi.F64)[0] == F64
    # a transposed view with fewer than 16 rows has no small-output kernel: the launcher takes the tiled one
    assert route(8, 128, 64, ta=True)[0] == T64 and route(8, 128, 64)[0] == SMALL and route(16, 128, 64, ta=True)[0] == SMALL
    assert lib.gh_gemm_route(C.byref(D.cmd_relu(0x1000, 0x2000, 16)), None) == -1
