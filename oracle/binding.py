"""ctypes binding of oracle/liboracle.so for the parity tests, the smoke check
and the CPU-baseline leg of the benchmark.  TEST INFRASTRUCTURE ONLY: the
product package never imports this module."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "liboracle.so")

BIN = {"mod": 11, "add": 0, "sub": 1, "mul": 2, "div": 3, "pow": 4, "lt": 5, "lte": 6, "gt": 7, "gte": 8,
       "eq": 9, "ne": 10}
MODE = {"vv": 0, "vs": 1, "sv": 2, "ss": 3}
UNARY = {"abs": 0, "sign": 1, "ceil": 2, "floor": 3, "sin": 4, "cos": 5, "exp": 6, "ln": 7,
         "log2": 8, "neg": 9, "square": 10, "sqrt": 11, "inverse": 12, "invsqrt": 13, "cube": 14,
         "tanh": 15, "sigmoid": 16, "log1p": 17, "expm1": 18, "softplus": 19}

_lib = None


def build():
    subprocess.run(["make", "-C", HERE, "-s"], check=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        _lib = C.CDLL(LIB)
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _i64(*v):
    return [C.c_int64(int(x)) for x in v]


def set_threads(n):
    lib().oracle_set_threads(int(n))


def binop(fn, mode, a, b):
    """Returns the array the device kernel writes (A for vv/vs/ss, B for sv)."""
    dt = a.dtype
    A = np.array(a, dtype=dt, copy=True).reshape(-1)
    B = np.array(b, dtype=dt, copy=True).reshape(-1)
    n = B.size if mode == "sv" else A.size
    f = lib().oracle_binop_f32 if dt == np.float32 else lib().oracle_binop_f64
    f(BIN[fn], MODE[mode], _p(A), _p(B), C.c_int64(n))
    return B if mode == "sv" else A


def bcast_binop(fn, big, small, outer, mid, inner, small_left=False):
    dt = np.float64 if np.asarray(big).dtype == np.float64 else np.float32
    big = np.ascontiguousarray(big, dtype=dt)
    small = np.ascontiguousarray(small, dtype=dt)
    dst = np.empty(outer * mid * inner, dtype=dt)
    f = lib().oracle_bcast_binop_f64 if dt == np.float64 else lib().oracle_bcast_binop_f32
    f(BIN[fn], int(small_left), _p(dst), _p(big), _p(small), *_i64(outer, mid, inner))
    return dst


def unary(fn, a):
    A = np.array(a, copy=True).reshape(-1)
    f = lib().oracle_unary_f32 if A.dtype == np.float32 else lib().oracle_unary_f64
    f(UNARY[fn], _p(A), C.c_int64(A.size))
    return A


def _ft(x):
    """float64 arrays keep their type (the *_f64 twins), everything else is float32."""
    return np.float64 if np.asarray(x).dtype == np.float64 else np.float32


def relu(x):
    x = np.ascontiguousarray(x, dtype=_ft(x))
    y = np.empty_like(x)
    (lib().oracle_relu_f64 if x.dtype == np.float64 else lib().oracle_relu_f32)(_p(y), _p(x), C.c_int64(x.size))
    return y


def leaky_relu(x, alpha):
    x = np.ascontiguousarray(x, dtype=_ft(x))
    y = np.empty_like(x)
    if x.dtype == np.float64:
        lib().oracle_leaky_relu_f64(_p(y), _p(x), C.c_double(alpha), C.c_int64(x.size))
    else:
        lib().oracle_leaky_relu_f32(_p(y), _p(x), C.c_float(alpha), C.c_int64(x.size))
    return y


def gemm(A, B, trans_a=False, trans_b=False):
    A = np.ascontiguousarray(A, dtype=np.float32)
    B = np.ascontiguousarray(B, dtype=np.float32)
    m, k = (A.shape[1], A.shape[0]) if trans_a else A.shape
    n = B.shape[0] if trans_b else B.shape[1]
    Cm = np.empty((m, n), dtype=np.float32)
    lib().oracle_gemm_f32(int(trans_a), int(trans_b), *_i64(m, n, k), _p(A), C.c_int64(A.shape[1]),
                          _p(B), C.c_int64(B.shape[1]), _p(Cm), C.c_int64(n))
    return Cm


def gemm_f64acc(A, B, trans_a=False, trans_b=False):
    A = np.ascontiguousarray(A, dtype=np.float32)
    B = np.ascontiguousarray(B, dtype=np.float32)
    m, k = (A.shape[1], A.shape[0]) if trans_a else A.shape
    n = B.shape[0] if trans_b else B.shape[1]
    Cm = np.empty((m, n), dtype=np.float64)
    lib().oracle_gemm_f64acc(int(trans_a), int(trans_b), *_i64(m, n, k), _p(A),
                             C.c_int64(A.shape[1]), _p(B), C.c_int64(B.shape[1]), _p(Cm),
                             C.c_int64(n))
    return Cm


def bmm(A, B, trans_a=False, trans_b=False):
    A = np.ascontiguousarray(A, dtype=np.float32)
    B = np.ascontiguousarray(B, dtype=np.float32)
    batch = A.shape[0]
    m, k = (A.shape[2], A.shape[1]) if trans_a else A.shape[1:]
    n = B.shape[1] if trans_b else B.shape[2]
    Cm = np.empty((batch, m, n), dtype=np.float32)
    lib().oracle_bmm_f32(int(trans_a), int(trans_b), *_i64(batch, m, n, k), _p(A), _p(B), _p(Cm))
    return Cm


def gemv(A, x, trans=False):
    A = np.ascontiguousarray(A, dtype=np.float32)
    x = np.ascontiguousarray(x, dtype=np.float32)
    m, n = A.shape
    y = np.empty(n if trans else m, dtype=np.float32)
    lib().oracle_gemv_f32(int(trans), *_i64(m, n), _p(A), C.c_int64(n), _p(x), _p(y))
    return y


def outer(x, y):
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.ascontiguousarray(y, dtype=np.float32)
    A = np.empty((x.size, y.size), dtype=np.float32)
    lib().oracle_outer_f32(*_i64(x.size, y.size), _p(x), _p(y), _p(A))
    return A


def conv_out_hw(h, w, kh, kw, pad, stride, dil):
    oh, ow = C.c_int64(), C.c_int64()
    lib().oracle_conv_out_hw(*_i64(h, w, kh, kw, pad[0], pad[1], stride[0], stride[1], dil[0],
                                   dil[1]), C.byref(oh), C.byref(ow))
    return oh.value, ow.value


def conv2d(x, w, pad=(0, 0), stride=(1, 1), dil=(1, 1)):
    if _ft(x) == np.float64:
        x = np.ascontiguousarray(x, dtype=np.float64)
        w = np.ascontiguousarray(w, dtype=np.float64)
        B, Cn, H, W = x.shape
        F, _, kh, kw = w.shape
        oh, ow = conv_out_hw(H, W, kh, kw, pad, stride, dil)
        y = np.empty((B, F, oh, ow), dtype=np.float64)
        lib().oracle_conv2d_f64(_p(x), _p(w), _p(y), *_i64(B, Cn, H, W, F, kh, kw, pad[0], pad[1],
                                                           stride[0], stride[1], dil[0], dil[1]))
        return y
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    B, Cn, H, W = x.shape
    F, _, kh, kw = w.shape
    oh, ow = conv_out_hw(H, W, kh, kw, pad, stride, dil)
    y = np.empty((B, F, oh, ow), dtype=np.float32)
    rc = lib().oracle_conv2d_f32(_p(x), _p(w), _p(y), *_i64(B, Cn, H, W, F, kh, kw, pad[0], pad[1],
                                                           stride[0], stride[1], dil[0], dil[1]))
    if rc != 0:
        raise MemoryError("oracle conv2d scratch allocation failed")
    return y


def conv2d_direct_f64(x, w, pad=(0, 0), stride=(1, 1), dil=(1, 1)):
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    B, Cn, H, W = x.shape
    F, _, kh, kw = w.shape
    oh, ow = conv_out_hw(H, W, kh, kw, pad, stride, dil)
    y = np.empty((B, F, oh, ow), dtype=np.float64)
    lib().oracle_conv2d_direct_f64(_p(x), _p(w), _p(y), *_i64(B, Cn, H, W, F, kh, kw, pad[0], pad[1],
                                                             stride[0], stride[1], dil[0], dil[1]))
    return y


def _pad4(pad):
    if len(pad) == 4:
        return np.array(pad, dtype=np.int64), 1
    return np.array([pad[0], pad[0], pad[1], pad[1]], dtype=np.int64), 0


def maxpool_out_hw(h, w, kh, kw, pad, stride):
    p4, _ = _pad4(pad)
    oh, ow = C.c_int64(), C.c_int64()
    lib().oracle_maxpool_out_hw(*_i64(h, w, kh, kw), _p(p4), *_i64(stride[0], stride[1]),
                                C.byref(oh), C.byref(ow))
    return oh.value, ow.value


def maxpool2d(x, kernel, pad, stride):
    x = np.ascontiguousarray(x, dtype=_ft(x))
    B, Cn, H, W = x.shape
    p4, explicit = _pad4(pad)
    oh, ow = maxpool_out_hw(H, W, kernel[0], kernel[1], pad, stride)
    y = np.empty((B, Cn, oh, ow), dtype=x.dtype)
    (lib().oracle_maxpool2d_f64 if x.dtype == np.float64 else lib().oracle_maxpool2d_f32)(_p(x), _p(y), *_i64(B, Cn, H, W, kernel[0], kernel[1]), _p(p4),
                               C.c_int(explicit), *_i64(stride[0], stride[1]))
    return y


def bn_infer(x, mean, var, eps, gamma=None, beta=None):
    dt = _ft(x)
    x = np.ascontiguousarray(x, dtype=dt)
    B, Cn = x.shape[:2]
    S = x.size // (B * Cn)
    y = np.empty_like(x)
    mean = np.ascontiguousarray(mean, dtype=dt)
    var = np.ascontiguousarray(var, dtype=dt)
    g = np.ascontiguousarray(gamma, dtype=dt) if gamma is not None else None
    b = np.ascontiguousarray(beta, dtype=dt) if beta is not None else None
    f, e = (lib().oracle_bn_infer_f64, C.c_double(eps)) if dt == np.float64 else (lib().oracle_bn_infer_f32, C.c_float(eps))
    f(_p(x), _p(y), _p(mean), _p(var), _p(g) if g is not None else None,
      _p(b) if b is not None else None, e, *_i64(B, Cn, S))
    return y


def bn_train(x, run_mean, run_var, momentum, eps):
    """One training-mode forward; returns (y, new_running_mean, new_running_var)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    B, Cn = x.shape[:2]
    S = x.size // (B * Cn)
    y = np.empty_like(x)
    rm = np.array(run_mean, dtype=np.float32, copy=True)
    rv = np.array(run_var, dtype=np.float32, copy=True)
    lib().oracle_bn_train_f32(_p(x), _p(y), _p(rm), _p(rv), C.c_float(momentum), C.c_float(eps),
                              *_i64(B, Cn, S))
    return y, rm, rv


def softmax(x):
    x = np.ascontiguousarray(x)
    rows, cols = int(np.prod(x.shape[:-1])), x.shape[-1]
    y = np.empty_like(x)
    f = lib().oracle_softmax_f32 if x.dtype == np.float32 else lib().oracle_softmax_f64
    f(_p(x), _p(y), *_i64(rows, cols))
    return y


def maxpool2d_bwd(x, dy, kernel, pad, stride):
    x = np.ascontiguousarray(x, dtype=_ft(x))
    dy = np.ascontiguousarray(dy, dtype=x.dtype)
    B, Cn, H, W = x.shape
    p4, explicit = _pad4(pad)
    dx = np.empty_like(x)
    f = lib().oracle_maxpool2d_bwd_f64 if x.dtype == np.float64 else lib().oracle_maxpool2d_bwd_f32
    f(_p(x), _p(dy), _p(dx), *_i64(B, Cn, H, W, kernel[0], kernel[1]), _p(p4), C.c_int(explicit),
      *_i64(stride[0], stride[1]))
    return dx


def conv2d_bwd(x, w, dy, pad=(0, 0), stride=(1, 1), dil=(1, 1)):
    """(dx, dw) of Conv2d as the reference's graph differentiates it (float32), or for float64
    operands from the definition in float64."""
    if np.asarray(x).dtype == np.float64:
        x = np.ascontiguousarray(x, dtype=np.float64)
        w = np.ascontiguousarray(w, dtype=np.float64)
        dy = np.ascontiguousarray(dy, dtype=np.float64)
        B, Cn, H, W = x.shape
        F, _, kh, kw = w.shape
        dx, dw = np.empty_like(x), np.empty_like(w)
        lib().oracle_conv2d_bwd_f64(_p(x), _p(w), _p(dy), _p(dx), _p(dw),
                                    *_i64(B, Cn, H, W, F, kh, kw, pad[0], pad[1], stride[0], stride[1],
                                          dil[0], dil[1]))
        return dx, dw
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    dy = np.ascontiguousarray(dy, dtype=np.float32)
    B, Cn, H, W = x.shape
    F, _, kh, kw = w.shape
    dx, dw = np.empty_like(x), np.empty_like(w)
    rc = lib().oracle_conv2d_bwd_f32(_p(x), _p(w), _p(dy), _p(dx), _p(dw),
                                     *_i64(B, Cn, H, W, F, kh, kw, pad[0], pad[1], stride[0], stride[1],
                                           dil[0], dil[1]))
    if rc != 0:
        raise MemoryError("oracle conv2d backward scratch allocation failed")
    return dx, dw


def conv2d_bwd_direct_f64(x, w, dy, pad=(0, 0), stride=(1, 1), dil=(1, 1)):
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    dy = np.ascontiguousarray(dy, dtype=np.float32)
    B, Cn, H, W = x.shape
    F, _, kh, kw = w.shape
    dx, dw = np.empty(x.shape, np.float64), np.empty(w.shape, np.float64)
    lib().oracle_conv2d_bwd_direct_f64(_p(x), _p(w), _p(dy), _p(dx), _p(dw),
                                       *_i64(B, Cn, H, W, F, kh, kw, pad[0], pad[1], stride[0], stride[1],
                                             dil[0], dil[1]))
    return dx, dw


def bn_train_stats(x, run_mean, run_var, momentum, eps):
    """Training-mode forward; returns (y, running_mean, running_var, save_mean, save_var_sum)."""
    dt = _ft(x)
    x = np.ascontiguousarray(x, dtype=dt)
    B, Cn = x.shape[:2]
    S = x.size // (B * Cn)
    y = np.empty_like(x)
    rm = np.array(run_mean, dtype=dt, copy=True)
    rv = np.array(run_var, dtype=dt, copy=True)
    sm, sv = np.empty(Cn, dt), np.empty(Cn, dt)
    if dt == np.float64:
        lib().oracle_bn_train_stats_f64(_p(x), _p(y), _p(rm), _p(rv), _p(sm), _p(sv), C.c_double(momentum),
                                        C.c_double(eps), *_i64(B, Cn, S))
    else:
        lib().oracle_bn_train_stats_f32(_p(x), _p(y), _p(rm), _p(rv), _p(sm), _p(sv), C.c_float(momentum),
                                        C.c_float(eps), *_i64(B, Cn, S))
    return y, rm, rv, sm, sv


def bn_bwd(x, dy, save_mean, save_var, eps, training=True):
    dt = _ft(x)
    x = np.ascontiguousarray(x, dtype=dt)
    dy = np.ascontiguousarray(dy, dtype=dt)
    B, Cn = x.shape[:2]
    S = x.size // (B * Cn)
    dx = np.empty_like(x)
    sm = np.ascontiguousarray(save_mean, dtype=dt)
    sv = np.ascontiguousarray(save_var, dtype=dt)
    if dt == np.float64:
        lib().oracle_bn_bwd_f64(_p(x), _p(dy), _p(dx), _p(sm), _p(sv), C.c_double(eps), C.c_int(int(training)),
                                *_i64(B, Cn, S))
    else:
        lib().oracle_bn_bwd_f32(_p(x), _p(dy), _p(dx), _p(sm), _p(sv), C.c_float(eps), C.c_int(int(training)),
                                *_i64(B, Cn, S))
    return dx


def softmax_bwd(y, dy):
    y = np.ascontiguousarray(y, dtype=_ft(y))
    dy = np.ascontiguousarray(dy, dtype=y.dtype)
    rows, cols = int(np.prod(y.shape[:-1])), y.shape[-1]
    dx = np.empty_like(y)
    (lib().oracle_softmax_bwd_f64 if y.dtype == np.float64 else lib().oracle_softmax_bwd_f32)(
        _p(y), _p(dy), _p(dx), *_i64(rows, cols))
    return dx


SOLVER = {"vanilla": 0, "rmsprop": 1, "adam": 2}


def solver_params(eta, eps=1e-8, l1reg=0.0, l2reg=0.0, clip=0.0, batch=1.0, decay=0.999, beta1=0.9, beta2=0.999,
                  kind="vanilla", iteration=1, dtype=np.float32):
    """The constants a solver step uses in the tensors' type, computed the way the reference does
    (float64 first, then one cast for float32 tensors; solvers.go:307-314, 492-525, 793-806), and
    its use mask."""
    f = np.dtype(dtype).type
    if kind == "rmsprop":
        a, b = f(decay), f(1.0 - decay)
    else:
        a, b = f(beta1), f(beta2)
    c1 = f(1) / f(1 - beta1 ** iteration)
    c2 = f(1) / f(1 - beta2 ** iteration)
    par = np.array([f(eta), f(eps), f(l1reg), f(l2reg), f(clip), f(1) / f(batch), a, b, c1, c2], dtype=dtype)
    use = (1 if l1reg else 0) | (2 if l2reg else 0) | (4 if clip else 0) | (8 if batch > 1 else 0)
    return par, use


def solver_step(kind, w, g, c1=None, c2=None, **kw):
    """One solver step in place on copies, in w's type (float32 or float64); returns (w, g, c1, c2)."""
    dt = _ft(np.asarray(w))
    par, use = solver_params(kind=kind, dtype=dt, **kw)
    w = np.array(w, dtype=dt, copy=True)
    g = np.array(g, dtype=dt, copy=True)
    c1 = np.zeros_like(w) if c1 is None else np.array(c1, dtype=dt, copy=True)
    c2 = np.zeros_like(w) if c2 is None else np.array(c2, dtype=dt, copy=True)
    (lib().oracle_solver_step_f64 if dt == np.float64 else lib().oracle_solver_step_f32)(
        C.c_int(SOLVER[kind]), _p(w), _p(g), _p(c1), _p(c2), C.c_int64(w.size), C.c_int(use), _p(par))
    return w, g, c1, c2


def dropout(x, r, prob, training=True):
    x = np.ascontiguousarray(x, dtype=_ft(x))
    r = np.ascontiguousarray(r, dtype=x.dtype)
    y = np.empty_like(x)
    (lib().oracle_dropout_f64 if x.dtype == np.float64 else lib().oracle_dropout_f32)(
        _p(x), _p(r), _p(y), C.c_int64(x.size), C.c_double(prob), C.c_int(int(training)))
    return y


def dropout_bwd(y, dy, prob):
    y = np.ascontiguousarray(y, dtype=_ft(y))
    dy = np.ascontiguousarray(dy, dtype=y.dtype)
    dx = np.empty_like(y)
    (lib().oracle_dropout_bwd_f64 if y.dtype == np.float64 else lib().oracle_dropout_bwd_f32)(
        _p(y), _p(dy), _p(dx), C.c_int64(y.size), C.c_double(prob))
    return dx


def uniform01(n, seed, offset=0, dtype=np.float32):
    out = np.empty(n, dtype)
    (lib().oracle_uniform01_f64 if out.dtype == np.float64 else lib().oracle_uniform01_f32)(
        _p(out), C.c_int64(n), C.c_uint64(seed), C.c_uint64(offset))
    return out


def has_nan(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return bool(lib().oracle_has_nan_f32(_p(a), C.c_int64(a.size)))


def has_inf(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return bool(lib().oracle_has_inf_f32(_p(a), C.c_int64(a.size)))
