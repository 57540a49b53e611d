"""Python binding of the C++ host mirror (libgorgonia_host.so): the engine
(cuda.Engine), its BFC arena, and the graph / tape machine.  Method names follow
the Go methods they stand in for.  All logic lives in the native library; this
module only marshals arguments."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

from . import _ffi

HERE = os.path.dirname(os.path.abspath(__file__))
HOST_LIB_PATH = os.path.join(HERE, "lib", "libgorgonia_host.so")


class GhhTensor(C.Structure):
    _fields_ = [("mem", C.c_uint64), ("dtype", C.c_int32), ("ndim", C.c_int32),
                ("shape", C.c_int64 * 8), ("flags", C.c_uint32)]


class GhhOp(C.Structure):
    _fields_ = [("kind", C.c_int32), ("fn", C.c_int32), ("name", C.c_char * 24),
                ("trans_a", C.c_int32), ("trans_b", C.c_int32), ("n_ints", C.c_int32),
                ("ints", C.c_int64 * 16), ("f0", C.c_double), ("f1", C.c_double), ("fs", C.c_double * 10)]


T_NOT_MANAGED, T_TRANSPOSED, T_NEEDS_ITER, T_COL_MAJOR = 1, 2, 4, 8
_P = C.c_void_p
_TP = C.POINTER(GhhTensor)

HOST_SYMBOLS = {
    "ghh_bfc_new": (_P, [C.c_int64]),
    "ghh_bfc_destroy": (None, [_P]),
    "ghh_bfc_reserve": (None, [_P, C.c_uint64, C.c_int64]),
    "ghh_bfc_release": (C.c_uint64, [_P]),
    "ghh_bfc_alloc": (C.c_int, [_P, C.c_int64, C.POINTER(C.c_uint64), C.POINTER(C.c_int64)]),
    "ghh_bfc_free": (None, [_P, C.c_uint64]),
    "ghh_bfc_coalesce": (None, [_P]),
    "ghh_bfc_reset_allocator": (None, [_P]),
    "ghh_bfc_freelist_len": (C.c_int, [_P]),
    "ghh_bfc_freelist": (C.c_int, [_P, C.POINTER(C.c_uint64), C.POINTER(C.c_int64), C.c_int]),
    "ghh_bfc_align": (C.c_int64, [_P, C.c_int64]),
    "ghh_bfc_allocated": (C.c_int64, [_P]),
    "ghh_bfc_used_count": (C.c_int, [_P]),
    "ghh_engine_new": (_P, []),
    "ghh_engine_destroy": (None, [_P]),
    "ghh_engine_init": (C.c_int, [_P, C.c_int, C.c_int64]),
    "ghh_engine_close": (C.c_int, [_P]),
    "ghh_engine_last_error": (C.c_char_p, [_P]),
    "ghh_engine_get": (C.c_int, [_P, C.c_int64, C.POINTER(C.c_uint64)]),
    "ghh_engine_put": (C.c_int, [_P, C.c_uint64, C.c_int64]),
    "ghh_engine_reset_allocator": (C.c_int, [_P]),
    "ghh_engine_alloc_accessible": (C.c_int, [_P]),
    "ghh_engine_memset": (C.c_int, [_P, C.c_uint64, _P]),
    "ghh_engine_memclr": (C.c_int, [_P, C.c_uint64]),
    "ghh_engine_accessible": (C.c_int, [_P, C.c_uint64, _P]),
    "ghh_engine_alloc_flags": (C.c_int, [_P, _P]),
    "ghh_engine_memcpy": (C.c_int, [_P, C.c_uint64, C.c_int64, C.c_uint64, C.c_int64]),
    "ghh_engine_h2d": (C.c_int, [_P, C.c_uint64, _P, C.c_int64]),
    "ghh_engine_d2h": (C.c_int, [_P, _P, C.c_uint64, C.c_int64]),
    "ghh_engine_has_func": (C.c_int, [_P, C.c_char_p]),
    "ghh_engine_elem_grid_size": (C.c_int, [_P, C.c_int, C.POINTER(C.c_int32 * 6)]),
    "ghh_engine_binop": (C.c_int, [_P, C.c_int, _TP, _TP, _TP, C.c_int, C.c_int, C.POINTER(C.c_uint64)]),
    "ghh_engine_binop_scalar": (C.c_int, [_P, C.c_int, _TP, C.c_uint64, C.c_int, _TP, C.c_int,
                                          C.POINTER(C.c_uint64)]),
    "ghh_engine_unary": (C.c_int, [_P, C.c_char_p, _TP, C.c_uint64]),
    "ghh_engine_matmul": (C.c_int, [_P, _TP, _TP, _TP]),
    "ghh_engine_matvecmul": (C.c_int, [_P, _TP, _TP, _TP]),
    "ghh_engine_outer": (C.c_int, [_P, _TP, _TP, _TP]),
    "ghh_engine_has_nan": (C.c_int, [_P, _TP, C.POINTER(C.c_int)]),
    "ghh_engine_has_inf": (C.c_int, [_P, _TP, C.POINTER(C.c_int)]),
    "ghh_engine_do_work": (C.c_int, [_P]),
    "ghh_engine_pending": (C.c_int, [_P]),
    "ghh_engine_submit_calls": (C.c_int64, [_P]),
    "ghh_graph_new": (_P, []),
    "ghh_graph_destroy": (None, [_P]),
    "ghh_graph_last_error": (C.c_char_p, [_P]),
    "ghh_graph_new_tensor": (C.c_int, [_P, C.POINTER(C.c_int64), C.c_int, C.c_int, _P, C.c_int]),
    "ghh_graph_apply": (C.c_int, [_P, C.POINTER(GhhOp), C.POINTER(C.c_int), C.c_int, C.POINTER(C.c_int)]),
    "ghh_graph_let": (C.c_int, [_P, C.c_int, _P]),
    "ghh_graph_read": (C.c_int, [_P, C.c_int, _P]),
    "ghh_graph_read_borrowed": (C.c_int, [_P, C.c_int]),
    "ghh_graph_let_borrowed": (C.c_int, [_P, C.c_int]),
    "ghh_graph_node_shape": (C.c_int, [_P, C.c_int, C.POINTER(C.c_int64), C.c_int]),
    "ghh_graph_node_dtype": (C.c_int, [_P, C.c_int]),
    "ghh_graph_fuse_activations": (C.c_int, [_P]),
    "ghh_tape_new": (_P, [_P, C.c_int, C.c_int]),
    "ghh_lisp_new": (_P, [_P, C.c_int]),
    "ghh_tape_new_with_engine": (_P, [_P, _P, C.c_int, C.c_int]),
    "ghh_tape_destroy": (None, [_P]),
    "ghh_tape_last_error": (C.c_char_p, [_P]),
    "ghh_tape_init": (C.c_int, [_P, C.c_int]),
    "ghh_tape_compile_only": (C.c_int, [_P]),
    "ghh_tape_run_all": (C.c_int, [_P]),
    "ghh_tape_run_all_n": (C.c_int, [_P, C.c_int]),
    "ghh_tape_watch": (C.c_int, [_P, C.c_int, C.c_int]),
    "ghh_tape_reset": (C.c_int, [_P]),
    "ghh_tape_close": (C.c_int, [_P]),
    "ghh_tape_gpumem": (C.c_int64, [_P]),
    "ghh_tape_segments": (C.c_int, [_P]),
    "ghh_tape_graph_launches": (C.c_int, [_P]),
    "ghh_tape_submit_calls": (C.c_int64, [_P]),
    "ghh_tape_register_address": (C.c_uint64, [_P, C.c_int]),
    "ghh_tape_read_buffer": (_P, [_P, C.c_int]),
    "ghh_tape_input_buffer": (_P, [_P, C.c_int]),
    "ghh_tape_program_string": (C.c_int, [_P, C.c_char_p, C.c_int]),
    "ghh_tape_engine": (_P, [_P]),
    "ghh_tape_segment_verdict": (C.c_int, [_P, C.c_int]),
    "ghh_tape_phase_ns": (None, [_P, C.POINTER(C.c_int64)]),
}

_hlib = None


def load_host():
    global _hlib
    if _hlib is not None:
        return _hlib
    _ffi.load()  # the host library links against the device library
    if not os.path.exists(HOST_LIB_PATH):
        raise ImportError(f"{HOST_LIB_PATH} is missing: build it with `python -m gorgonia_amd.build`")
    lib = C.CDLL(HOST_LIB_PATH)
    for name, (res, args) in HOST_SYMBOLS.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _hlib = lib
    return lib


class EngineError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(msg)
        self.code = code


DTYPES = {np.dtype(np.float32): 0, np.dtype(np.float64): 1}


class Tensor:
    """A dense tensor in the engine's arena (shape () = scalar)."""

    def __init__(self, mem, shape, dtype=np.float32, transposed=False, managed=True,
                 needs_iterator=False, col_major=False):
        self.mem = int(mem)
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self.transposed = transposed
        self.managed = managed
        self.needs_iterator = needs_iterator
        self.col_major = col_major   # DataOrder.IsColMajor: element (i, j) of an (r, c) matrix at j * r + i

    @property
    def size(self):
        return int(np.prod(self.shape)) if self.shape else 1

    @property
    def nbytes(self):
        return self.size * self.dtype.itemsize

    def T(self):
        """Transposed view of a matrix (tensor.T(): shape swapped, data order flagged)."""
        assert len(self.shape) == 2
        return Tensor(self.mem, self.shape[::-1], self.dtype, not self.transposed, self.managed,
                      col_major=self.col_major)

    def desc(self):
        d = GhhTensor()
        d.mem = self.mem
        d.dtype = DTYPES.get(self.dtype, 2)
        d.ndim = len(self.shape)
        for i, s in enumerate(self.shape):
            d.shape[i] = s
        d.flags = ((0 if self.managed else T_NOT_MANAGED) | (T_TRANSPOSED if self.transposed else 0) |
                   (T_NEEDS_ITER if self.needs_iterator else 0) | (T_COL_MAJOR if self.col_major else 0))
        return d


BIN_FN = dict(_ffi.BIN_FN)


class Engine:
    """cuda.Engine stand-in (cuda/engine.go, cuda/external.go, cuda/arena.go,
    cuda/arith.go, cuda/cmp.go, cuda/linalg.go)."""

    def __init__(self, handle=None):
        self.lib = load_host()
        self._own = handle is None
        self.h = handle if handle is not None else self.lib.ghh_engine_new()

    def _check(self, rc):
        if rc != 0:
            raise EngineError(rc, self.lib.ghh_engine_last_error(self.h).decode(errors="replace"))

    # External
    def Init(self, device, size):
        self._check(self.lib.ghh_engine_init(self.h, device, size))

    def Close(self):
        if self.h:
            self._check(self.lib.ghh_engine_close(self.h))

    def destroy(self):
        if self.h and self._own:
            self.lib.ghh_engine_destroy(self.h)
        self.h = None

    def HasFunc(self, name):
        return bool(self.lib.ghh_engine_has_func(self.h, name.encode()))

    def ElemGridSize(self, n):
        out = (C.c_int32 * 6)()
        self.lib.ghh_engine_elem_grid_size(self.h, n, C.byref(out))
        return tuple(out)

    def DoWork(self):
        self._check(self.lib.ghh_engine_do_work(self.h))

    Signal = DoWork

    def AllocAccessible(self):
        return bool(self.lib.ghh_engine_alloc_accessible(self.h))

    def AllocFlags(self):
        """(manually managed, column-major tag): cuda/engine.go:81-83."""
        out = (C.c_int32 * 2)()
        self.lib.ghh_engine_alloc_flags(self.h, C.byref(out))
        return bool(out[0]), bool(out[1])

    def Memset(self, mem, val=None):
        self._check(self.lib.ghh_engine_memset(self.h, int(mem), None))

    def Memclr(self, mem):
        self._check(self.lib.ghh_engine_memclr(self.h, int(mem)))

    def Accessible(self, mem):
        out = C.c_uint64(0)
        self._check(self.lib.ghh_engine_accessible(self.h, int(mem), C.byref(out)))
        return out.value

    def NonStdAlloc(self):
        pass

    def WorksWith(self, order=None):
        return True

    def pending(self):
        return self.lib.ghh_engine_pending(self.h)

    def submit_calls(self):
        return self.lib.ghh_engine_submit_calls(self.h)

    # Arena
    def Get(self, size):
        mem = C.c_uint64()
        self._check(self.lib.ghh_engine_get(self.h, size, C.byref(mem)))
        return mem.value

    def Put(self, mem, size):
        self.lib.ghh_engine_put(self.h, mem, size)

    def ResetAllocator(self):
        self.lib.ghh_engine_reset_allocator(self.h)

    def Memcpy(self, dst, src):
        self._check(self.lib.ghh_engine_memcpy(self.h, dst.mem, dst.nbytes, src.mem, src.nbytes))

    # Transfer (ExternMetadata.Transfer, cuda.go:179-215)
    def to_device(self, arr, shape=None):
        arr = np.ascontiguousarray(arr)
        t = Tensor(self.Get(max(arr.nbytes, 1)), arr.shape if shape is None else shape, arr.dtype)
        if arr.nbytes:
            self._check(self.lib.ghh_engine_h2d(self.h, t.mem, arr.ctypes.data_as(C.c_void_p), arr.nbytes))
        return t

    def to_host(self, t):
        out = np.empty(t.shape, dtype=t.dtype)
        self._check(self.lib.ghh_engine_d2h(self.h, out.ctypes.data_as(C.c_void_p), t.mem, out.nbytes))
        return out

    def new_tensor(self, shape, dtype=np.float32):
        dtype = np.dtype(dtype)
        n = int(np.prod(shape)) if len(shape) else 1
        return Tensor(self.Get(max(n * dtype.itemsize, 1)), shape, dtype)

    # arith / cmp
    def _binop(self, fn, a, b, reuse=None, unsafe=False, incr=False):
        ret = C.c_uint64()
        r = C.byref(reuse.desc()) if reuse is not None else None
        self._check(self.lib.ghh_engine_binop(self.h, BIN_FN[fn], C.byref(a.desc()), C.byref(b.desc()), r,
                                              0 if unsafe else 1, int(incr), C.byref(ret)))
        return reuse if reuse is not None else a

    def _binop_scalar(self, fn, a, b_mem, leftTensor, reuse=None, unsafe=False):
        ret = C.c_uint64()
        r = C.byref(reuse.desc()) if reuse is not None else None
        b = b_mem.mem if isinstance(b_mem, Tensor) else (0 if b_mem is None else int(b_mem))
        self._check(self.lib.ghh_engine_binop_scalar(self.h, BIN_FN[fn], C.byref(a.desc()), b,
                                                     int(leftTensor), r, 0 if unsafe else 1, C.byref(ret)))
        return reuse if reuse is not None else a

    def Unary(self, op_name, a, dst=None):
        self._check(self.lib.ghh_engine_unary(self.h, op_name.encode(), C.byref(a.desc()),
                                              dst.mem if dst is not None else 0))
        return dst if dst is not None else a

    def MatMul(self, a, b, prealloc):
        self._check(self.lib.ghh_engine_matmul(self.h, C.byref(a.desc()), C.byref(b.desc()),
                                               C.byref(prealloc.desc())))

    def MatVecMul(self, a, b, prealloc):
        self._check(self.lib.ghh_engine_matvecmul(self.h, C.byref(a.desc()), C.byref(b.desc()),
                                                  C.byref(prealloc.desc())))

    def Outer(self, a, b, prealloc):
        self._check(self.lib.ghh_engine_outer(self.h, C.byref(a.desc()), C.byref(b.desc()),
                                              C.byref(prealloc.desc())))

    def HasNaN(self, a):
        out = C.c_int()
        self._check(self.lib.ghh_engine_has_nan(self.h, C.byref(a.desc()), C.byref(out)))
        return bool(out.value)

    def HasInf(self, a):
        out = C.c_int()
        self._check(self.lib.ghh_engine_has_inf(self.h, C.byref(a.desc()), C.byref(out)))
        return bool(out.value)


def _mk(fn):
    def tt(self, a, b, reuse=None, unsafe=False, incr=False):
        return self._binop(fn, a, b, reuse, unsafe, incr)

    def ts(self, a, b, leftTensor, reuse=None, unsafe=False):
        return self._binop_scalar(fn, a, b, leftTensor, reuse, unsafe)
    return tt, ts


for _go, _fn in [("Add", "add"), ("Sub", "sub"), ("Mul", "mul"), ("Div", "div"), ("Pow", "pow"),
                 ("Lt", "lt"), ("Lte", "lte"), ("Gt", "gt"), ("Gte", "gte"), ("ElEq", "eq"),
                 ("ElNe", "ne"), ("Mod", "mod")]:
    _tt, _ts = _mk(_fn)
    setattr(Engine, _go, _tt)
    setattr(Engine, _go + "Scalar", _ts)


class BFC:
    """cuda/bfc.go arena bookkeeping (host only)."""

    def __init__(self, alignment=32):
        self.lib = load_host()
        self.h = self.lib.ghh_bfc_new(alignment)

    def __del__(self):
        if getattr(self, "h", None):
            self.lib.ghh_bfc_destroy(self.h)
            self.h = None

    def reserve(self, start, size):
        self.lib.ghh_bfc_reserve(self.h, start, size)

    def release(self):
        return self.lib.ghh_bfc_release(self.h)

    def alloc(self, size):
        addr = C.c_uint64()
        oom = (C.c_int64 * 2)()
        rc = self.lib.ghh_bfc_alloc(self.h, size, C.byref(addr), oom)
        if rc == 1:
            raise ValueError("Cannot allocate memory with size 0 or less")
        if rc == 2:
            raise MemoryError(f"allocated/reserved: {oom[1]}/{oom[0]}")
        return addr.value

    def free(self, addr):
        self.lib.ghh_bfc_free(self.h, addr)

    def coalesce(self):
        self.lib.ghh_bfc_coalesce(self.h)

    def reset_allocator(self):
        self.lib.ghh_bfc_reset_allocator(self.h)

    def freelist_len(self):
        return self.lib.ghh_bfc_freelist_len(self.h)

    def freelist(self):
        n = self.freelist_len()
        offs = (C.c_uint64 * max(n, 1))()
        sizes = (C.c_int64 * max(n, 1))()
        self.lib.ghh_bfc_freelist(self.h, offs, sizes, n)
        return [(offs[i], sizes[i]) for i in range(n)]

    def align(self, size):
        return self.lib.ghh_bfc_align(self.h, size)

    def allocated(self):
        return self.lib.ghh_bfc_allocated(self.h)

    def used_count(self):
        return self.lib.ghh_bfc_used_count(self.h)
