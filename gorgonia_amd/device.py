"""Thin Python view of the device C ABI: a context, raw device buffers and
command builders.  Used by the tests, the benchmark and the Python mirror of
the engine; it adds no numerics of its own - every result comes from the HIP
library."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _ffi
from ._ffi import GhCmd


class DeviceError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"{_ffi.ERR_NAMES.get(code, code)}: {msg}")
        self.code = code


def make_cmd(opcode, flags=0, ptrs=(), dims=(), f=()):
    c = GhCmd()
    c.opcode = opcode
    c.flags = flags
    for i, p in enumerate(ptrs):
        c.ptr[i] = int(p)
    for i, d in enumerate(dims):
        c.dim[i] = int(d)
    for i, v in enumerate(f):
        c.f[i] = float(v)
    return c


class Context:
    """One gh_ctx: a device, its stream and (optionally) an arena reservation."""

    def __init__(self, device=0, arena_bytes=0):
        self.lib = _ffi.load()
        h = C.c_void_p()
        rc = self.lib.gh_init(device, arena_bytes, C.byref(h))
        if rc != 0:
            raise DeviceError(rc, f"gh_init(device={device}, arena_bytes={arena_bytes}) failed")
        self.h = h
        self._owned = []

    # -- lifetime -----------------------------------------------------------
    def close(self):
        if self.h:
            self.lib.gh_close(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    # -- errors ---------------------------------------------------------------
    def check(self, rc):
        if rc != 0:
            buf = C.create_string_buffer(512)
            self.lib.gh_last_error(self.h, buf, 512)
            raise DeviceError(rc, buf.value.decode(errors="replace"))

    def clear_error(self):
        self.lib.gh_clear_error(self.h)

    def info(self):
        d = _ffi.GhDevInfo()
        self.check(self.lib.gh_device_info(self.h, C.byref(d)))
        return d

    # -- memory -----------------------------------------------------------------
    def malloc(self, nbytes):
        p = C.c_uint64()
        self.check(self.lib.gh_malloc(self.h, max(int(nbytes), 1), C.byref(p)))
        return p.value

    def free(self, ptr):
        self.check(self.lib.gh_free(self.h, ptr))

    def arena(self):
        return self.lib.gh_arena_base(self.h), self.lib.gh_arena_size(self.h)

    def h2d(self, dptr, arr):
        arr = np.ascontiguousarray(arr)
        self.check(self.lib.gh_memcpy_h2d(self.h, dptr, arr.ctypes.data_as(C.c_void_p), arr.nbytes))
        self.sync()  # pageable numpy memory: do not return before the copy is done

    def d2h(self, dptr, shape, dtype=np.float32):
        out = np.empty(shape, dtype=dtype)
        self.check(self.lib.gh_memcpy_d2h(self.h, out.ctypes.data_as(C.c_void_p), dptr, out.nbytes))
        self.sync()
        return out

    def upload(self, arr):
        """Allocate a device buffer holding `arr`; returns its address."""
        arr = np.ascontiguousarray(arr)
        p = self.malloc(arr.nbytes)
        if arr.nbytes:
            self.h2d(p, arr)
        return p

    # -- work ---------------------------------------------------------------------
    def submit(self, cmds):
        if isinstance(cmds, GhCmd):
            cmds = [cmds]
        n = len(cmds)
        arr = (GhCmd * n)(*cmds)
        self.check(self.lib.gh_submit(self.h, arr, n))

    def sync(self):
        self.check(self.lib.gh_sync(self.h))

    def run(self, cmds):
        self.submit(cmds)
        self.sync()

    def event(self, slot):
        self.check(self.lib.gh_event_record(self.h, slot))

    def elapsed_ms(self, a, b):
        ms = C.c_float()
        self.check(self.lib.gh_event_elapsed_ms(self.h, a, b, C.byref(ms)))
        return ms.value

    # -- graphs ---------------------------------------------------------------------
    def graph_begin(self):
        self.check(self.lib.gh_graph_begin(self.h))

    def graph_end(self):
        gid = C.c_int()
        self.check(self.lib.gh_graph_end(self.h, C.byref(gid)))
        return gid.value

    def graph_launch(self, gid):
        self.check(self.lib.gh_graph_launch(self.h, gid))

    def graph_destroy(self, gid):
        self.check(self.lib.gh_graph_destroy(self.h, gid))


# ---- command builders -------------------------------------------------------------

def cmd_bin(fn, mode, a, b, n, dtype=_ffi.F32, dst=0):
    fl = _ffi.flag_fn(_ffi.BIN_FN[fn]) | _ffi.flag_mode(_ffi.MODE[mode]) | _ffi.flag_dtype(dtype)
    return make_cmd(_ffi.OP_ELEM_BIN, fl, (a, b, dst), (n,))


def cmd_unary(fn, a, n, dtype=_ffi.F32, dst=0):
    fl = _ffi.flag_fn(_ffi.UNARY_FN[fn]) | _ffi.flag_dtype(dtype)
    return make_cmd(_ffi.OP_ELEM_UNARY, fl, (a, dst), (n,))


def cmd_bcast(fn, dst, big, small, outer, mid, inner, small_left=False, dtype=_ffi.F32):
    fl = _ffi.flag_fn(_ffi.BIN_FN[fn]) | _ffi.flag_dtype(dtype) | (_ffi.FLAG_SMALL_LEFT if small_left else 0)
    return make_cmd(_ffi.OP_BCAST_BIN, fl, (dst, big, small), (outer, mid, inner))


def cmd_copy(dst, src, nbytes):
    return make_cmd(_ffi.OP_MEMCPY_D2D, 0, (dst, src), (nbytes,))


def cmd_gemm(a, b, c, m, n, k, lda=None, ldb=None, ldc=None, trans_a=False, trans_b=False,
             batch=1, stride_a=0, stride_b=0, stride_c=0, act=None, alpha=0.0, dtype=_ffi.F32, softmax=False,
             bias=0):
    lda = lda if lda is not None else (m if trans_a else k)
    ldb = ldb if ldb is not None else (k if trans_b else n)
    ldc = ldc if ldc is not None else n
    fl = (_ffi.FLAG_TRANS_A if trans_a else 0) | (_ffi.FLAG_TRANS_B if trans_b else 0)
    fl |= {None: 0, "relu": _ffi.FLAG_ACT_RELU, "leaky": _ffi.FLAG_ACT_LEAKY}[act] | _ffi.flag_dtype(dtype)
    if softmax:
        fl |= _ffi.FLAG_GEMM_SOFTMAX
    if bias:
        fl |= _ffi.FLAG_GEMM_BIAS
    return make_cmd(_ffi.OP_GEMM, fl, (a, b, c, bias), (m, n, k, lda, ldb, ldc, batch, stride_a, stride_b,
                                                  stride_c), (alpha,))


def cmd_gemv(a, x, y, m, n, lda=None, trans=False, dtype=_ffi.F32):
    return make_cmd(_ffi.OP_GEMV, (_ffi.FLAG_TRANS_A if trans else 0) | _ffi.flag_dtype(dtype), (a, x, y),
                    (m, n, lda if lda is not None else n))


def cmd_outer(x, y, a, m, n, dtype=_ffi.F32):
    return make_cmd(_ffi.OP_OUTER, _ffi.flag_dtype(dtype), (x, y, a), (m, n))


def _double_bits(v):
    """A float64 scalar as the int64 a dim slot carries (gh_cmd.f is float32)."""
    return int(np.array([v], dtype=np.float64).view(np.int64)[0])


def cmd_conv2d(x, w, y, B, Cin, H, W, F, kh, kw, pad=(0, 0), stride=(1, 1), dilation=(1, 1),
               act=None, alpha=0.0, bn=None, eps=1e-5, pool2=False, dtype=_ffi.F32, pre=None, keep=None):
    """bn = (mean, var, gamma or 0, beta or 0) device pointers: BatchNorm (eval)
    on the result; pool2: 2x2 stride-2 MaxPool2D on the result (y is then
    B x F x oh/2 x ow/2).  Order: conv, bn, activation, pool.
    pre = w0 (Cin x 1 x 3 x 3 filters): x holds single-channel images B x 1 x 2H x 2W and the
    convolution's input is MaxPool2D(Rectify(Conv2d(x, w0, pad 1))), never stored.
    keep (with pool2): a B x F x oh x ow tensor that also receives the unpooled result as the
    activation reads it."""
    fl = {None: 0, "relu": _ffi.FLAG_ACT_RELU, "leaky": _ffi.FLAG_ACT_LEAKY}[act] | _ffi.flag_dtype(dtype)
    ptrs = [x, w, y]
    if bn is not None:
        mean, var, gamma, beta = bn
        fl |= _ffi.FLAG_CONV_BN | (_ffi.FLAG_HAS_GAMMA if gamma else 0) | (_ffi.FLAG_HAS_BETA if beta else 0)
        ptrs += [mean, var, gamma, beta]
    if pool2:
        fl |= _ffi.FLAG_CONV_POOL2
    if pre is not None:
        fl |= _ffi.FLAG_CONV_PRE
        ptrs = (ptrs + [0] * 7)[:7] + [pre]
    if keep is not None:
        fl |= _ffi.FLAG_CONV_KEEP
        ptrs = (ptrs + [0] * 7)[:7] + [keep]
    return make_cmd(_ffi.OP_CONV2D, fl, ptrs,
                    (B, Cin, H, W, F, kh, kw, pad[0], pad[1], stride[0], stride[1], dilation[0],
                     dilation[1]), (alpha, eps))


def cmd_maxpool2d(x, y, B, Cn, H, W, kh, kw, pad, stride, dtype=_ffi.F32):
    """pad: 2 values (symmetric H, W) or 4 values (north, south, west, east) as in MaxPool2D."""
    if len(pad) == 4:
        p4, fl = tuple(pad), _ffi.FLAG_EXPLICIT_PAD
    else:
        p4, fl = (pad[0], pad[0], pad[1], pad[1]), 0
    return make_cmd(_ffi.OP_MAXPOOL2D, fl | _ffi.flag_dtype(dtype), (x, y), (B, Cn, H, W, kh, kw) + p4 + tuple(stride))


def cmd_bn_infer(x, y, mean, var, B, Cn, S, eps, gamma=0, beta=0, dtype=_ffi.F32):
    fl = (_ffi.FLAG_HAS_GAMMA if gamma else 0) | (_ffi.FLAG_HAS_BETA if beta else 0) | _ffi.flag_dtype(dtype)
    return make_cmd(_ffi.OP_BN_INFER, fl, (x, y, mean, var, gamma, beta), (B, Cn, S, _double_bits(eps)), (eps,))


def cmd_relu(x, y, n, dtype=_ffi.F32):
    return make_cmd(_ffi.OP_RELU, _ffi.flag_dtype(dtype), (x, y), (n,))


def cmd_leaky_relu(x, y, n, alpha, dtype=_ffi.F32):
    return make_cmd(_ffi.OP_LEAKY_RELU, _ffi.flag_dtype(dtype), (x, y), (n, _double_bits(alpha)), (alpha,))


def cmd_softmax(x, y, rows, cols, dtype=_ffi.F32):
    return make_cmd(_ffi.OP_SOFTMAX, _ffi.flag_dtype(dtype), (x, y), (rows, cols))


def cmd_maxpool2d_bwd(x, dy, dx, B, Cn, H, W, kh, kw, pad, stride, dtype=_ffi.F32):
    c = cmd_maxpool2d(x, dy, B, Cn, H, W, kh, kw, pad, stride, dtype=dtype)
    c.opcode = _ffi.OP_MAXPOOL2D_BWD
    c.ptr[2] = int(dx)
    return c


def _conv_dims(B, Cin, H, W, F, kh, kw, pad, stride, dilation):
    return (B, Cin, H, W, F, kh, kw, pad[0], pad[1], stride[0], stride[1], dilation[0], dilation[1])


def cmd_conv2d_bwd_data(dy, w, dx, B, Cin, H, W, F, kh, kw, pad=(0, 0), stride=(1, 1), dilation=(1, 1),
                        dtype=_ffi.F32):
    """dx of Conv2d; B, Cin, H, W describe x (and dx)."""
    return make_cmd(_ffi.OP_CONV2D_BWD_DATA, _ffi.flag_dtype(dtype), (dy, w, dx),
                    _conv_dims(B, Cin, H, W, F, kh, kw, pad, stride, dilation))


def cmd_conv2d_bwd_filter(x, dy, dw, B, Cin, H, W, F, kh, kw, pad=(0, 0), stride=(1, 1), dilation=(1, 1),
                          dtype=_ffi.F32):
    return make_cmd(_ffi.OP_CONV2D_BWD_FILTER, _ffi.flag_dtype(dtype), (x, dy, dw),
                    _conv_dims(B, Cin, H, W, F, kh, kw, pad, stride, dilation))


def cmd_bn_train(x, y, run_mean, run_var, save_mean, save_var, B, Cn, S, eps, momentum, dtype=_ffi.F32):
    return make_cmd(_ffi.OP_BN_TRAIN, _ffi.flag_dtype(dtype), (x, y, run_mean, run_var, save_mean, save_var),
                    (B, Cn, S, _double_bits(eps), _double_bits(momentum)), (eps, momentum))


def cmd_bn_bwd(x, dy, dx, save_mean, save_var, B, Cn, S, eps, training=True, dtype=_ffi.F32):
    return make_cmd(_ffi.OP_BN_BWD, (0 if training else _ffi.FLAG_BN_EVAL) | _ffi.flag_dtype(dtype),
                    (x, dy, dx, save_mean, save_var), (B, Cn, S, _double_bits(eps)), (eps,))


def cmd_softmax_bwd(y, dy, dx, rows, cols, dtype=_ffi.F32):
    return make_cmd(_ffi.OP_SOFTMAX_BWD, _ffi.flag_dtype(dtype), (y, dy, dx), (rows, cols))


SOLVER = {"vanilla": 0, "rmsprop": 1, "adam": 2}


def cmd_solver_step(kind, w, g, n, par, use, cache=0, cache2=0, dtype=_ffi.F32):
    """par: the ten constants of gorgonia_hip.h's SOLVER_STEP row (float32 in f[], or for float64
    tensors as double bit patterns in dim[1..10]); use: option mask."""
    fl = _ffi.flag_fn(SOLVER[kind]) | _ffi.flag_mode(use) | _ffi.flag_dtype(dtype)
    if dtype == _ffi.F64:
        return make_cmd(_ffi.OP_SOLVER_STEP, fl, (w, g, cache, cache2), (n,) + tuple(_double_bits(v) for v in par))
    return make_cmd(_ffi.OP_SOLVER_STEP, fl, (w, g, cache, cache2), (n,), tuple(float(v) for v in par))


def cmd_rand_uniform(out, n, seed, offset=0, state=0, dtype=_ffi.F32):
    return make_cmd(_ffi.OP_RAND_UNIFORM, _ffi.flag_dtype(dtype), (out, state), (n, seed, offset))


def cmd_dropout(x, y, r, n, prob, training=True, dtype=_ffi.F32):
    fl = (0 if training else _ffi.FLAG_BN_EVAL) | _ffi.flag_dtype(dtype)
    return make_cmd(_ffi.OP_DROPOUT, fl, (x, y, r), (n, _double_bits(prob)), (prob,))


def cmd_dropout_bwd(y, dy, dx, n, prob, dtype=_ffi.F32):
    return make_cmd(_ffi.OP_DROPOUT_BWD, _ffi.flag_dtype(dtype), (y, dy, dx), (n, _double_bits(prob)), (prob,))


def cmd_relu_bwd(x, dy, dx, n, dtype=_ffi.F32):
    return make_cmd(_ffi.OP_RELU_BWD, _ffi.flag_dtype(dtype), (x, dy, dx), (n,))


def cmd_has(kind, a, flag, n, dtype=_ffi.F32):
    op = _ffi.OP_HAS_NAN if kind == "nan" else _ffi.OP_HAS_INF
    return make_cmd(op, _ffi.flag_dtype(dtype), (a, flag), (n,))


def cmd_fill(a, n, value):
    return make_cmd(_ffi.OP_FILL, 0, (a,), (n,), (value,))
