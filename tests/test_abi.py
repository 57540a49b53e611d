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
