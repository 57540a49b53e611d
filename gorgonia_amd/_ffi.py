"""ctypes binding of libgorgonia_hip.so (the C ABI of include/gorgonia_hip.h).

The library is the product; this module only loads it.  There is no CPU
fallback: if the shared object is missing the import fails with instructions,
and if it is present but no GPU is visible every compute call fails with the
library's own error.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libgorgonia_hip.so")

GH_OK, GH_EINVAL, GH_EDEVICE, GH_EOOM, GH_ENOFUNC, GH_ESTATE = range(6)
ERR_NAMES = {0: "GH_OK", 1: "GH_EINVAL", 2: "GH_EDEVICE", 3: "GH_EOOM", 4: "GH_ENOFUNC", 5: "GH_ESTATE"}

# opcodes
(OP_NOP, OP_ELEM_BIN, OP_ELEM_UNARY, OP_BCAST_BIN, OP_MEMCPY_D2D, OP_GEMM, OP_GEMV, OP_OUTER,
 OP_CONV2D, OP_MAXPOOL2D, OP_BN_INFER, OP_RELU, OP_LEAKY_RELU, OP_SOFTMAX, OP_HAS_NAN, OP_HAS_INF,
 OP_FILL, OP_MAXPOOL2D_BWD, OP_CONV2D_BWD_DATA, OP_CONV2D_BWD_FILTER, OP_BN_TRAIN, OP_BN_BWD,
 OP_SOFTMAX_BWD, OP_SOLVER_STEP, OP_RAND_UNIFORM, OP_DROPOUT, OP_DROPOUT_BWD, OP_RELU_BWD) = range(28)

BIN_FN = {"mod": 11, "add": 0, "sub": 1, "mul": 2, "div": 3, "pow": 4, "lt": 5, "lte": 6, "gt": 7, "gte": 8,
          "eq": 9, "ne": 10}
MODE = {"vv": 0, "vs": 1, "sv": 2, "ss": 3}
F32, F64 = 0, 1
UNARY_FN = {"abs": 0, "sign": 1, "ceil": 2, "floor": 3, "sin": 4, "cos": 5, "exp": 6, "ln": 7,
            "log2": 8, "neg": 9, "square": 10, "sqrt": 11, "inverse": 12, "invsqrt": 13, "cube": 14,
            "tanh": 15, "sigmoid": 16, "log1p": 17, "expm1": 18, "softplus": 19}

FLAG_TRANS_A = 1 << 16
FLAG_TRANS_B = 1 << 17
FLAG_SMALL_LEFT = 1 << 18
FLAG_EXPLICIT_PAD = 1 << 19
FLAG_HAS_GAMMA = 1 << 20
FLAG_HAS_BETA = 1 << 21
FLAG_ACT_RELU = 1 << 22
FLAG_ACT_LEAKY = 1 << 23
FLAG_CONV_BN = 1 << 24
FLAG_CONV_POOL2 = 1 << 25
FLAG_BN_EVAL = 1 << 26
FLAG_GEMM_SOFTMAX = 1 << 27
FLAG_GEMM_BIAS = 1 << 28
FLAG_CONV_PRE = 1 << 29
FLAG_CONV_KEEP = 1 << 30


def flag_fn(f):
    return f & 0xFF


def flag_mode(m):
    return (m & 0xF) << 8


def flag_dtype(d):
    return (d & 0xF) << 12


class GhCmd(C.Structure):
    _fields_ = [("opcode", C.c_uint32), ("flags", C.c_uint32), ("ptr", C.c_uint64 * 8),
                ("dim", C.c_int64 * 16), ("f", C.c_float * 12)]


class GhDevInfo(C.Structure):
    _fields_ = [("wavefront_size", C.c_int32), ("max_threads_per_block", C.c_int32),
                ("max_grid_x", C.c_int32), ("max_grid_y", C.c_int32), ("max_grid_z", C.c_int32),
                ("max_block_x", C.c_int32), ("max_block_y", C.c_int32), ("max_block_z", C.c_int32),
                ("compute_units", C.c_int32), ("lds_bytes_per_block", C.c_int32),
                ("free_mem", C.c_int64), ("total_mem", C.c_int64), ("arch", C.c_char * 32)]


# Every symbol include/gorgonia_hip.h declares: name -> (restype, argtypes)
_P = C.c_void_p
SYMBOLS = {
    "gh_init": (C.c_int, [C.c_int, C.c_int64, C.POINTER(_P)]),
    "gh_close": (C.c_int, [_P]),
    "gh_device_info": (C.c_int, [_P, C.POINTER(GhDevInfo)]),
    "gh_device_count": (C.c_int, [C.POINTER(C.c_int)]),
    "gh_arena_base": (C.c_uint64, [_P]),
    "gh_arena_size": (C.c_int64, [_P]),
    "gh_malloc": (C.c_int, [_P, C.c_int64, C.POINTER(C.c_uint64)]),
    "gh_free": (C.c_int, [_P, C.c_uint64]),
    "gh_host_alloc": (C.c_int, [_P, C.c_int64, C.POINTER(_P)]),
    "gh_host_free": (C.c_int, [_P, _P]),
    "gh_memcpy_h2d": (C.c_int, [_P, C.c_uint64, _P, C.c_int64]),
    "gh_memcpy_d2h": (C.c_int, [_P, _P, C.c_uint64, C.c_int64]),
    "gh_memcpy_d2d": (C.c_int, [_P, C.c_uint64, C.c_uint64, C.c_int64]),
    "gh_submit": (C.c_int, [_P, C.POINTER(GhCmd), C.c_int]),
    "gh_submit_noalloc": (C.c_int, [_P, C.POINTER(GhCmd), C.c_int]),
    "gh_validate": (C.c_int, [C.POINTER(GhCmd), C.c_int, C.c_char_p, C.c_int]),
    "gh_conv2d_can_pool": (C.c_int, [C.POINTER(GhCmd)]),
    "gh_conv2d_can_pre": (C.c_int, [C.POINTER(GhCmd)]),
    "gh_conv2d_can_keep": (C.c_int, [C.POINTER(GhCmd)]),
    "gh_conv2d_route": (C.c_int, [C.POINTER(GhCmd)]),
    "gh_conv2d_bwd_filter_route": (C.c_int, [C.POINTER(GhCmd)]),
    "gh_gemm_route": (C.c_int, [C.POINTER(GhCmd), C.POINTER(C.c_int)]),
    "gh_gemm_can_softmax": (C.c_int, [C.POINTER(GhCmd)]),
    "gh_sync": (C.c_int, [_P]),
    "gh_graph_begin": (C.c_int, [_P]),
    "gh_graph_end": (C.c_int, [_P, C.POINTER(C.c_int)]),
    "gh_graph_launch": (C.c_int, [_P, C.c_int]),
    "gh_graph_destroy": (C.c_int, [_P, C.c_int]),
    "gh_has_func": (C.c_int, [C.c_char_p]),
    "gh_lookup_func": (C.c_int, [C.c_char_p, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]),
    "gh_last_error": (C.c_int, [_P, C.c_char_p, C.c_int]),
    "gh_clear_error": (C.c_int, [_P]),
    "gh_event_record": (C.c_int, [_P, C.c_int]),
    "gh_event_elapsed_ms": (C.c_int, [_P, C.c_int, C.c_int, C.POINTER(C.c_float)]),
    "gh_version": (C.c_char_p, []),
}

_lib = None


def load():
    """Load libgorgonia_hip.so; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m gorgonia_amd.build` "
            "(the HIP engine has no CPU fallback)")
    lib = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)  # AttributeError if the ABI lost a symbol
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib
