"""Build recipe for the native libraries (hipcc for gfx950, g++ for host code).

    python -m gorgonia_amd.build            # build everything in-tree
    python -m gorgonia_amd.build --force    # rebuild even if up to date

Outputs, next to this file:
    lib/libgorgonia_hip.so   device engine, C ABI of include/gorgonia_hip.h
    lib/libgorgonia_host.so  C++ host mirror of cuda.Engine / the tape segment
                             batcher, C ABI of include/gorgonia_host.h

hipcc cross-compiles for gfx950 without a GPU present.
"""
from __future__ import annotations

import argparse
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
HOST = os.path.join(HERE, "host")
INCLUDE = os.path.join(ROOT, "include")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(LIBDIR, "obj")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -ffp-contract=off, denormals kept, IEEE divide/sqrt: add/sub/mul/div results
# must be bit-identical to the CPU engine (the reference builds its kernels with
# -fmad=false -ftz=false -prec-div=true -prec-sqrt=true, cmd/cudagen/main.go:41-43).
# Packed-fp32 instructions are switched off for all device code.
HIP_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950",
    "-ffp-contract=off", "-fno-gpu-flush-denormals-to-zero",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fvisibility=hidden", "-Wall", "-Wno-unused-function", "-Wno-unused-value", "-Wno-unused-result", "-Wno-unknown-warning-option",
    "-I", INCLUDE, "-I", CSRC,
]

HIP_SOURCES = ["gh_api.hip", "gh_validate.cpp", "k_elem.hip", "k_gemm.hip", "k_conv_small.hip", "k_conv_rows.hip", "k_conv_rows1.hip", "k_conv_patch.hip", "k_conv_wide.hip", "k_conv_pointwise.hip", "k_conv_wgrad_small.hip", "k_nn.hip", "k_nn64.hip", "k_bwd.hip", "k_bwd64.hip"]

HOST_FLAGS = [
    "-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall", "-Wextra",
    "-I", INCLUDE, "-I", HOST,
]


def _newer(src_list, out):
    if not os.path.exists(out):
        return True
    t = os.path.getmtime(out)
    return any(os.path.getmtime(s) > t for s in src_list)


def _run(cmd):
    p = subprocess.run(cmd, capture_output=True, text=True)
    if p.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + p.stdout + p.stderr)
        raise RuntimeError("build step failed: " + " ".join(cmd[:3]))
    # the host pass of hipcc warns that it does not know packed-fp32-ops: harmless
    err = "\n".join(l for l in p.stderr.splitlines()
                    if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if err.strip():
        sys.stderr.write(err + "\n")


def _headers(d):
    return [os.path.join(d, f) for f in os.listdir(d) if f.endswith((".h", ".hpp"))]


def build_device(force=False):
    os.makedirs(OBJDIR, exist_ok=True)
    deps = _headers(CSRC) + _headers(INCLUDE)
    objs, jobs = [], []
    for s in HIP_SOURCES:
        src = os.path.join(CSRC, s)
        obj = os.path.join(OBJDIR, os.path.splitext(s)[0] + ".o")
        objs.append(obj)
        if force or _newer([src] + deps, obj):
            lang = ["-x", "hip"] if s.endswith(".hip") else []
            jobs.append([HIPCC] + HIP_FLAGS + ["-DGH_BUILDING"] + lang + ["-c", src, "-o", obj])
    with ThreadPoolExecutor(max_workers=min(6, max(1, len(jobs)))) as ex:
        list(ex.map(_run, jobs))
    out = os.path.join(LIBDIR, "libgorgonia_hip.so")
    if force or jobs or _newer(objs, out):
        _run([HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", out] + objs)
    return out


def build_host(force=False):
    if not os.path.isdir(HOST):
        return None
    os.makedirs(OBJDIR, exist_ok=True)
    srcs = sorted(os.path.join(HOST, f) for f in os.listdir(HOST) if f.endswith(".cpp"))
    if not srcs:
        return None
    out = os.path.join(LIBDIR, "libgorgonia_host.so")
    deps = srcs + _headers(HOST) + _headers(INCLUDE)
    if force or _newer(deps, out):
        cxx = shutil.which("g++") or "g++"
        # links against the device library through its C ABI only
        _run([cxx] + HOST_FLAGS + ["-shared", "-o", out] + srcs +
             ["-L", LIBDIR, "-lgorgonia_hip", "-Wl,-rpath,$ORIGIN"])
    return out


C_CONSUMER_DIR = os.path.join(ROOT, "tests", "c_consumer")
# The device header is meant for C callers (cgo compiles it as C): the consumer
# is built as strict C99 so anything that is not C in the header stops the build.
C_CONSUMER_FLAGS = ["-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-O1", "-I", INCLUDE]


def build_c_consumer(force=False):
    """The plain-C program of tests/c_consumer: links the device library only."""
    src = os.path.join(C_CONSUMER_DIR, "consumer.c")
    if not os.path.exists(src):
        return None
    out = os.path.join(C_CONSUMER_DIR, "consumer.bin")
    if force or _newer([src] + _headers(INCLUDE), out):
        cc = shutil.which("gcc") or "gcc"
        _run([cc] + C_CONSUMER_FLAGS + [src, "-o", out, "-L", LIBDIR, "-lgorgonia_hip",
                                        "-Wl,-rpath,$ORIGIN/../../gorgonia_amd/lib"])
    return out


def build_all(force=False):
    return [p for p in (build_device(force), build_host(force), build_c_consumer(force)) if p]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    a = ap.parse_args()
    for p in build_all(a.force):
        print("built", os.path.relpath(p, ROOT))


if __name__ == "__main__":
    main()
