"""Graph-building API and tape machine, named after the Gorgonia functions they
stand in for (api_gen.go, operations.go, nn.go, ops/nn/api_cuda.go, vm_tape.go).
Only what the device path needs: forward graphs of operators that have a
device implementation.  Nodes are plain handles; all logic is in
libgorgonia_host.so."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _ffi
from .engine import Engine, EngineError, GhhOp, load_host

(K_ELEMBIN, K_ELEMUNARY, K_BCAST, K_MATMUL, K_MATVEC, K_OUTER, K_BMM, K_CONV2D, K_MAXPOOL, K_BN,
 K_RECTIFY, K_LEAKY, K_SOFTMAX, K_RESHAPE, K_MAXPOOL_DIFF, K_CONV_DIFF_DATA, K_CONV_DIFF_FILTER, K_BN_TRAIN,
 K_BN_DIFF, K_SOFTMAX_DIFF, K_SET, K_SOLVER, K_RAND_UNIFORM, K_DROPOUT, K_DROPOUT_DIFF, K_RECTIFY_DIFF) = range(26)


class Node:
    def __init__(self, g, nid):
        self.g, self.id = g, nid

    def Shape(self):
        return self.g.shape_of(self.id)

    def Dtype(self):
        """numpy dtype of the node's value (float32 or float64)."""
        code = self.g.lib.ghh_graph_node_dtype(self.g.h, self.id)
        if code not in (0, 1):
            raise EngineError(1, f"node {self.id}: the device path holds float32 and float64 values only")
        return np.dtype(np.float64 if code == 1 else np.float32)


class ExprGraph:
    def __init__(self):
        self.lib = load_host()
        self.h = self.lib.ghh_graph_new()
        self._keep = []  # host arrays bound to nodes must outlive the graph

    def __del__(self):
        if getattr(self, "h", None):
            self.lib.ghh_graph_destroy(self.h)
            self.h = None

    def _check(self, rc):
        if rc != 0:
            raise EngineError(rc, self.lib.ghh_graph_last_error(self.h).decode(errors="replace"))

    def shape_of(self, nid):
        buf = (C.c_int64 * 8)()
        n = self.lib.ghh_graph_node_shape(self.h, nid, buf, 8)
        return tuple(buf[i] for i in range(n))

    def apply(self, kind, inputs, fn=0, name="", trans_a=False, trans_b=False, ints=(), f0=0.0, f1=0.0, fs=()):
        op = GhhOp()
        op.kind, op.fn, op.name = kind, fn, name.encode()
        op.trans_a, op.trans_b = int(trans_a), int(trans_b)
        op.n_ints = len(ints)
        for i, v in enumerate(ints):
            op.ints[i] = int(v)
        op.f0 = float(f0)
        op.f1 = float(f1)
        for i, v in enumerate(fs):
            op.fs[i] = float(v)
        arr = (C.c_int * len(inputs))(*[n.id for n in inputs])
        out = C.c_int()
        self._check(self.lib.ghh_graph_apply(self.h, C.byref(op), arr, len(inputs), C.byref(out)))
        return Node(self, out.value)


def NewGraph():
    return ExprGraph()


def NewTensor(g, value, resident=False):
    """NewTensor(g, dt, dims, WithShape(...), WithValue(value)): an input node
    bound to a host array.  resident=True keeps it on the device across runs
    (weights); the reference re-uploads every input on every run."""
    value = np.asarray(value)
    if value.ndim:  # ascontiguousarray would turn a 0-d scalar into shape (1,)
        value = np.ascontiguousarray(value)
    g._keep.append(value)
    shp = (C.c_int64 * max(value.ndim, 1))(*value.shape)
    dt = {np.dtype(np.float32): 0, np.dtype(np.float64): 1}.get(value.dtype, 2)
    nid = g.lib.ghh_graph_new_tensor(g.h, shp, value.ndim, dt, value.ctypes.data_as(C.c_void_p),
                                     int(resident))
    if nid < 0:
        raise EngineError(_ffi.GH_EINVAL, g.lib.ghh_graph_last_error(g.h).decode(errors="replace"))
    node = Node(g, nid)
    node.dtype = value.dtype
    return node


def NewScalar(g, value, dtype=np.float32, resident=True):
    return NewTensor(g, np.array(value, dtype=dtype), resident)


def Let(node, value):
    value = np.ascontiguousarray(value)
    node.g._keep.append(value)
    node.g._check(node.g.lib.ghh_graph_let(node.g.h, node.id, value.ctypes.data_as(C.c_void_p)))


def Read(node, dtype=None):
    """gorgonia.Read: returns the host array the value lands in after RunAll.  The array
    has the node's own dtype; asking for another one is an error (the machine copies the
    value's bytes, it does not convert)."""
    want = node.Dtype()
    if dtype is not None and np.dtype(dtype) != want:
        raise EngineError(1, f"Read: node {node.id} holds {want}, not {np.dtype(dtype)}")
    out = np.empty(node.Shape(), dtype=want)
    node.g._keep.append(out)
    node.g._check(node.g.lib.ghh_graph_read(node.g.h, node.id, out.ctypes.data_as(C.c_void_p)))
    return out


class BorrowedRead:
    """A Read whose value stays in the machine's own pinned host buffer: TapeMachine.value(r)
    is a numpy view of it, valid after RunAll and overwritten by the next one."""

    def __init__(self, node):
        self.node = node


def LetBorrowed(node):
    """Let without the host-to-host copy: the input's value is what the caller writes into
    TapeMachine.input(node), the machine's pinned buffer for it."""
    node.g._check(node.g.lib.ghh_graph_let_borrowed(node.g.h, node.id))
    return node


def ReadBorrowed(node):
    """gorgonia.Read without the final host-to-host copy: the machine lends its buffer."""
    node.g._check(node.g.lib.ghh_graph_read_borrowed(node.g.h, node.id))
    return BorrowedRead(node)


def _bin(fn):
    return lambda a, b: a.g.apply(K_ELEMBIN, [a, b], fn=_ffi.BIN_FN[fn])


def _un(name):
    return lambda a: a.g.apply(K_ELEMUNARY, [a], name=name)


def _calc_broadcast_shape(shape, expected_dims, along):
    """calcBroadcastShape (shape.go:38-68): the operand's shape in `expected_dims` dimensions with
    ones at the axes it is repeated along and its own extents, in order, in the free slots."""
    if len(shape) == expected_dims:
        return tuple(shape)
    if len(shape) == 0:
        return (1,) * expected_dims
    new = [0] * expected_dims
    for i in along:
        new[i] = 1
    for s in shape:
        for j in range(expected_dims):
            if new[j] == 0:
                new[j] = s
                break
    return tuple(new)


def _bc(fn):
    def op(a, b, leftPattern=None, rightPattern=None):
        """Broadcast<Op>(a, b, leftPattern, rightPattern) (api_gen.go:129-135 over Broadcast, broadcast.go:69-129):
        a is repeated along the axes of leftPattern and b along those of rightPattern, then the plain operator
        runs.  Here nothing is repeated in memory: the device operator reads the small operand where the
        repeated one would hold its copy.  Without patterns the operand with extents of one is the small one."""
        left, right = list(leftPattern or ()), list(rightPattern or ())
        if not left and not right:
            return a.g.apply(K_BCAST, [a, b], fn=_ffi.BIN_FN[fn])
        ashape, bshape = a.Shape(), b.Shape()
        x, y = a, b
        xs, ys = list(ashape), list(bshape)
        if left:
            for ax in left:
                if ax >= len(bshape):
                    raise EngineError(_ffi.GH_EINVAL, f"Attempting to broadcast a on axis {ax} of b. But b has shape {bshape}")
            xs = list(_calc_broadcast_shape(ashape, len(bshape), left))
            if tuple(xs) != tuple(ashape):
                x = Reshape(a, xs)
        if right:
            for ax in right:
                if ax >= len(ashape):
                    raise EngineError(_ffi.GH_EINVAL, f"Attempting to broadcast b on axis {ax} of a. But a has shape {ashape}")
            ys = list(_calc_broadcast_shape(bshape, len(ashape), right))
            if tuple(ys) != tuple(bshape):
                y = Reshape(b, ys)
        # the shapes the repeats would give (repeatOp multiplies the extent of its axis, op_tensor.go:175-188)
        xr, yr = list(xs), list(ys)
        for ax in left:
            xr[ax] *= bshape[ax]
        for ax in right:
            yr[ax] *= ashape[ax]
        if xr != yr:
            raise EngineError(_ffi.GH_EINVAL, f"Shape mismatch. Expected {tuple(xr)}. Got {tuple(yr)}")
        if left and right and tuple(xs) != tuple(xr) and tuple(ys) != tuple(yr):
            # both operands grow: the left one first, as a product with ones (exact), then the right one
            ones = NewTensor(a.g, np.ones(tuple(xr), dtype=a.Dtype()), resident=True)
            x = a.g.apply(K_BCAST, [ones, x], fn=_ffi.BIN_FN["mul"])
        return a.g.apply(K_BCAST, [x, y], fn=_ffi.BIN_FN[fn])
    return op


# api_gen.go names
Add, Sub, HadamardProd, HadamardDiv, Pow = _bin("add"), _bin("sub"), _bin("mul"), _bin("div"), _bin("pow")
Mod = _bin("mod")


def _cmp(fn):
    plain = _bin(fn)

    def op(a, b, retSame=True):
        """<Cmp>(a, b, retSame) (api_gen.go:80-127).  The device operators write 1 / 0 in the operands' own type
        (cuda/cmp.go:14-701), which is retSame = true; a Bool result does not exist on this path."""
        if not retSame:
            raise EngineError(_ffi.GH_EINVAL, "comparison on the device path returns the operands' type (retSame)")
        return plain(a, b)
    return op


Lt, Lte, Gt, Gte, Eq, Ne = _cmp("lt"), _cmp("lte"), _cmp("gt"), _cmp("gte"), _cmp("eq"), _cmp("ne")


def Div(a, b):
    """operations.go:114-122: HadamardDiv for a scalar operand or equal shapes; matrix division does not exist
    (the reference panics with "Unhandled")."""
    if a.Shape() == () or b.Shape() == () or a.Shape() == b.Shape():
        return HadamardDiv(a, b)
    raise EngineError(_ffi.GH_EINVAL, f"Div: unhandled for shapes {a.Shape()} and {b.Shape()}")


BroadcastAdd, BroadcastSub = _bc("add"), _bc("sub")
BroadcastHadamardProd, BroadcastHadamardDiv, BroadcastPow = _bc("mul"), _bc("div"), _bc("pow")


def _bc_cmp(fn):
    plain = _bc(fn)

    def op(a, b, retSame=True, leftPattern=None, rightPattern=None):
        """Broadcast<Cmp>(a, b, retSame, leftPattern, rightPattern) (api_gen.go:174-227).  The device operators
        write 1 / 0 in the operands' own type (cuda/cmp.go:14-701), which is retSame = true; a Bool result does
        not exist on this path."""
        if not retSame:
            raise EngineError(_ffi.GH_EINVAL, "comparison on the device path returns the operands' type (retSame)")
        return plain(a, b, leftPattern, rightPattern)
    return op


BroadcastLt, BroadcastGt, BroadcastLte, BroadcastGte = _bc_cmp("lt"), _bc_cmp("gt"), _bc_cmp("lte"), _bc_cmp("gte")
BroadcastEq, BroadcastNe = _bc_cmp("eq"), _bc_cmp("ne")
Abs, Sign, Ceil, Floor, Sin, Cos, Exp, Log, Log2 = (_un(n) for n in
                                                     ("abs", "sign", "ceil", "floor", "sin", "cos", "exp", "ln", "log2"))
Neg, Square, Sqrt, Inverse, InverseSqrt, Cube = (_un(n) for n in
                                                 ("neg", "square", "sqrt", "inv", "invSqrt", "cube"))
Tanh, Sigmoid, Log1p, Expm1, Softplus = (_un(n) for n in ("tanh", "sigmoid", "log1p", "expm1", "softplus"))


def Mul(a, b, transA=False, transB=False):
    """operations.go:52-74: scalar operand -> HadamardProd; vector . vector -> the inner product (a scalar);
    vector x matrix -> matVecMul of the transposed matrix; matrix x vector; matrix x matrix.  transA / transB are
    the flags the reference's linAlgBinOp carries when its differentiation builds the gradient products
    (operatorLinAlg.go:14-68)."""
    sa, sb = a.Shape(), b.Shape()
    if sa == () or sb == ():
        return HadamardProd(a, b)
    if len(sa) == 2 and len(sb) == 2:
        return a.g.apply(K_MATMUL, [a, b], trans_a=transA, trans_b=transB)
    if len(sa) == 2 and len(sb) == 1:
        return a.g.apply(K_MATVEC, [a, b], trans_a=transA)
    if len(sa) == 1 and len(sb) == 2:
        return a.g.apply(K_MATVEC, [b, a], trans_a=True)
    if len(sa) == 1 and len(sb) == 1:
        if sa != sb:
            raise EngineError(_ffi.GH_EINVAL, f"Mul: vectors of different lengths {sa} . {sb}")
        # the engine has MatVecMul, MatMul and Outer (cuda/linalg.go:47-260): the inner product is the 1 x n matrix a times b
        return Reshape(a.g.apply(K_MATVEC, [Reshape(a, (1, sa[0])), b]), ())
    raise EngineError(_ffi.GH_EINVAL, f"Mul: not yet implemented for a {sa} b {sb}")


def OuterProd(a, b):
    return a.g.apply(K_OUTER, [a, b])


def BatchedMatMul(a, b, transA=False, transB=False):
    return a.g.apply(K_BMM, [a, b], trans_a=transA, trans_b=transB)


def Conv2d(im, filter, kernelShape, pad=None, stride=(1, 1), dilation=None):
    """nnops.Conv2d (ops/nn/api_cuda.go:10-16; nn.go:211-305)."""
    pad = (0, 0) if pad is None else pad
    dilation = (1, 1) if dilation is None else dilation
    return im.g.apply(K_CONV2D, [im, filter], ints=list(kernelShape) + list(pad) + list(stride) + list(dilation))


def Conv1d(im, filter, kernel, pad, stride, dilation):
    """nnops.Conv1d (ops/nn/api_cuda.go:18-20; nn.go:308-310): a Conv2d over (B, C, 1, W) with
    kernel {1, kernel}, pad {0, pad}, stride {1, stride}, dilation {1, dilation}."""
    return Conv2d(im, filter, (1, kernel), [0, pad], [1, stride], [1, dilation])


def MaxPool2D(x, kernel, pad, stride):
    """nnops.MaxPool2D (nn.go:322-375): pad has 2 values (symmetric) or 4 (N, S, W, E)."""
    return x.g.apply(K_MAXPOOL, [x], ints=list(kernel) + [len(pad)] + list(pad) + list(stride))


def MaxPool1D(x, kernel, pad, stride):
    """nn.go:378-380: MaxPool2D over (B, C, 1, W) with kernel {1, kernel}, pad {0, pad}, stride {1, stride}."""
    return MaxPool2D(x, (1, kernel), (0, pad), (1, stride))


def BatchNorm(x, scale, bias, runningMean, runningVariance, epsilon=1e-5):
    """nnops.BatchNorm in EvalMode with SetStats(runningMean, runningVariance)
    (nn.go:386-441, op_nn.go:1286-1313): y = scale * ((x - mean)/sqrt(var + eps)) + bias."""
    ins = [x, runningMean, runningVariance] + ([scale, bias] if scale is not None else [])
    return x.g.apply(K_BN, ins, f0=epsilon)


def Rectify(x):
    return x.g.apply(K_RECTIFY, [x])


def LeakyRelu(x, alpha):
    return x.g.apply(K_LEAKY, [x], f0=alpha)


def SoftMax(x, *axes):
    """SoftMax(x, axes...) (op_softmax.go:13-17, 33-43): over the last axis, the reference's default, which is
    the only one the device operator has; another axis is refused."""
    if axes and axes[0] not in (-1, len(x.Shape()) - 1):
        raise EngineError(_ffi.GH_EINVAL, f"SoftMax: axis {axes[0]} of a {len(x.Shape())}-d value is not on the device path (last axis only)")
    return x.g.apply(K_SOFTMAX, [x])


def Reshape(x, shape):
    return x.g.apply(K_RESHAPE, [x], ints=list(shape))


# ---- the diff ops symbolic differentiation inserts, for hand-built training graphs ----

def MaxPool2DDiff(x, grad, kernel, pad, stride):
    """maxPoolDiffOp (op_nn.go:962-1093): gradient of MaxPool2D(x, kernel, pad, stride) wrt x."""
    return x.g.apply(K_MAXPOOL_DIFF, [x, grad], ints=list(kernel) + [len(pad)] + list(pad) + list(stride))


def Conv2dDiffImage(grad, filter, imageShape, kernelShape, pad=(0, 0), stride=(1, 1), dilation=(1, 1)):
    """Gradient of Conv2d wrt the image (col2im of grad2d . filter, op_nn.go:267-291, 605-640)."""
    ints = list(kernelShape) + list(pad) + list(stride) + list(dilation) + list(imageShape)
    return grad.g.apply(K_CONV_DIFF_DATA, [grad, filter], ints=ints)


def Conv2dDiffFilter(im, grad, kernelShape, pad=(0, 0), stride=(1, 1), dilation=(1, 1)):
    """Gradient of Conv2d wrt the filter (grad2d^T . im2col(im))."""
    return im.g.apply(K_CONV_DIFF_FILTER, [im, grad], ints=list(kernelShape) + list(pad) + list(stride) + list(dilation))


def BatchNormTrain(x, runningMean, runningVariance, saveMean, saveVariance, momentum=0.9, epsilon=1e-5):
    """nnops.BatchNorm in training mode (op_nn.go:1489-1635): returns the normalised
    value; the four statistics tensors (resident inputs) are updated in place."""
    op_inputs = [x, runningMean, runningVariance, saveMean, saveVariance]
    return x.g.apply(K_BN_TRAIN, op_inputs, f0=epsilon, f1=momentum)


def BatchNormDiff(x, grad, saveMean, saveVariance, epsilon=1e-5):
    """batchnormDiffOp (op_nn.go:1834-1943), training branch."""
    return x.g.apply(K_BN_DIFF, [x, grad, saveMean, saveVariance], f0=epsilon)


def SoftMaxDiff(y, grad):
    """softmaxDiffOp (op_softmax.go:184-279): y = SoftMax(x), returns the gradient wrt x."""
    return y.g.apply(K_SOFTMAX_DIFF, [y, grad])


def Set(a, b):
    """gorgonia.Set(a, b): a's value becomes b's; a keeps its register, so a
    resident input updated this way carries the new value into the next run."""
    return a.g.apply(K_SET, [a, b])


def AdamCorrections(iteration, beta1=0.9, beta2=0.999, dtype=np.float32):
    """The two bias corrections of an Adam step, 1/(1 - beta^t), rounded to the weights' type the
    way the reference rounds them (solvers.go:780-870): the value to bind (Let) before each run
    to the `corrections` input of SolverStep("adam", ...)."""
    f = np.dtype(dtype).type
    return np.array([f(1) / f(1 - beta1 ** iteration), f(1) / f(1 - beta2 ** iteration)], dtype=dtype)


def SolverStep(kind, weights, grad, caches=(), eta=0.001, eps=1e-8, l1reg=0.0, l2reg=0.0, clip=0.0, batch=1.0,
               decay=0.999, beta1=0.9, beta2=0.999, iteration=1, corrections=None):
    """One Step of NewVanillaSolver / NewRMSPropSolver / NewAdamSolver (solvers.go) on one
    weight tensor, on the device: the weights (a resident input) and the solver's caches
    (resident inputs, zero at the start) are updated in place.  The constants are
    rounded to the weights' type the way the reference rounds them (float64 weights keep
    them in double).  Adam's bias corrections depend on the iteration: given as `iteration`
    they are constants of the command (one graph per step); given as `corrections` - an input
    node holding AdamCorrections(t), rebound before each run - they are read from memory and
    the same command, and the same captured segment, serves every step."""
    f = np.float64 if getattr(weights, "dtype", None) == np.float64 else np.float32
    a, b = (f(decay), f(1.0 - decay)) if kind == "rmsprop" else (f(beta1), f(beta2))
    fs = [f(eta), f(eps), f(l1reg), f(l2reg), f(clip), f(1) / f(batch), a, b,
          f(1) / f(1 - beta1 ** iteration), f(1) / f(1 - beta2 ** iteration)]
    use = (1 if l1reg else 0) | (2 if l2reg else 0) | (4 if clip else 0) | (8 if batch > 1 else 0)
    fn = {"vanilla": 0, "rmsprop": 1, "adam": 2}[kind]
    extra = [corrections] if corrections is not None else []
    if extra and kind != "adam":
        raise EngineError(1, "only Adam takes bias corrections")
    return weights.g.apply(K_SOLVER, [weights, grad] + list(caches) + extra, fn=fn, ints=[use], fs=fs)


def RandUniform(g, shape, seed, offset=0, counter=None):
    """The uniform [0, 1) numbers gorgonia.Dropout draws (nn.go:71-77), generated on the
    device: element i is a function of (seed, offset + i) only.  With `counter` (from
    NewCounter) the offset lives on the device and moves on by the tensor's size every
    run, so a replayed tape draws fresh numbers each time."""
    inputs = [] if counter is None else [counter]
    return g.apply(K_RAND_UNIFORM, inputs, ints=[int(seed), int(offset)] + [int(d) for d in shape])


def NewCounter(g, start=0):
    """One 8-byte position of a random stream, resident on the device."""
    return NewTensor(g, np.array([start], dtype=np.uint64).view(np.float64), resident=True)


def Dropout(x, prob, rand=None, seed=0, training=True):
    """gorgonia.Dropout(x, dropProb) (nn.go:71-77, op_dropout.go:107-132):
    y = r < 1-p ? x/(1-p) : 0 with r uniform in [0, 1).  `rand` supplies the numbers
    (a node of x's size); without it a device generator seeded with `seed` and its own
    counter is added to the graph.  The reference seeds from the wall clock."""
    if rand is None:
        rand = RandUniform(x.g, x.Shape(), seed, counter=NewCounter(x.g))
    return x.g.apply(K_DROPOUT, [x, rand], fn=int(training), f0=float(prob))


def DropoutDiff(y, grad, prob):
    """dropoutDiffOp (op_dropout.go:205-238): dx = dy/p where y is non-zero, else 0."""
    return y.g.apply(K_DROPOUT_DIFF, [y, grad], f0=float(prob))


def RectifyDiff(x, grad):
    """The gradient of Rectify(x) as one operator, where the reference's device build calls the
    activation backward of ops/nn/activation_cuda.go:130-153: grad * (x >= 0), the bits of
    HadamardProd(grad, Gte(x, 0))."""
    return x.g.apply(K_RECTIFY_DIFF, [x, grad])


class TapeMachine:
    """NewTapeMachine(g, ...) / RunAll / Reset / Close (vm_tape.go:45-249)."""

    def __init__(self, g, graph_replay=False, reupload_resident=False, fuse_activations=False,
                 device=0, compile_only=False, engine=None, node_at_a_time=False, watch_nan=False, watch_inf=False):
        self.g = g
        self.lib = g.lib
        # a watched machine checks every operator's own value, so nothing is folded into its producer (a pool
        # drops the NaN its input held: the folded command's result would hide it)
        self.fused = self.lib.ghh_graph_fuse_activations(g.h) if fuse_activations and not (watch_nan or watch_inf) else 0
        self._shared_engine = engine  # WithEngine(e) (vm.go:318-329): kept alive, never closed here
        # graph_replay: False, True (capture on the second run, replay from then on) or
        # "measured" (time plain submits against replays first, keep the quicker)
        mode = 2 if graph_replay == "measured" else int(bool(graph_replay))
        if node_at_a_time:
            self.h = self.lib.ghh_lisp_new(g.h, int(reupload_resident))
        elif engine is not None:
            self.h = self.lib.ghh_tape_new_with_engine(g.h, engine.h, mode, int(reupload_resident))
        else:
            self.h = self.lib.ghh_tape_new(g.h, mode, int(reupload_resident))
        if watch_nan or watch_inf:
            self._check(self.lib.ghh_tape_watch(self.h, int(watch_nan), int(watch_inf)))
        if compile_only:
            self._check(self.lib.ghh_tape_compile_only(self.h))
        else:
            self._check(self.lib.ghh_tape_init(self.h, device))

    def _check(self, rc):
        if rc != 0:
            if not self.h:
                raise EngineError(rc, "the machine is closed")
            raise EngineError(rc, self.lib.ghh_tape_last_error(self.h).decode(errors="replace"))

    def RunAll(self):
        self._check(self.lib.ghh_tape_run_all(self.h))

    def RunAllN(self, n):
        """n RunAll calls in one call into the library (no interpreter between the steps)."""
        self._check(self.lib.ghh_tape_run_all_n(self.h, int(n)))

    def Reset(self):
        self._check(self.lib.ghh_tape_reset(self.h))

    def Close(self):
        if self.h:
            self.lib.ghh_tape_close(self.h)
            self.lib.ghh_tape_destroy(self.h)
            self.h = None

    def engine(self):
        return Engine(self.lib.ghh_tape_engine(self.h))

    def gpumem(self):
        return self.lib.ghh_tape_gpumem(self.h)

    def segments(self):
        return self.lib.ghh_tape_segments(self.h)

    def graph_launches(self):
        return self.lib.ghh_tape_graph_launches(self.h)

    def segment_verdict(self, segment=0):
        """'measuring', 'plain' or 'replay' for a segment of the last run (graph_replay="measured")."""
        return ("measuring", "plain", "replay")[self.lib.ghh_tape_segment_verdict(self.h, segment)]

    def _view(self, ptr, node):
        shape = node.Shape()
        n = int(np.prod(shape)) if len(shape) else 1
        ctype = C.c_double if node.Dtype() == np.float64 else C.c_float
        return np.ctypeslib.as_array((ctype * n).from_address(ptr)).reshape(shape)

    def input(self, node):
        """The numpy view of a LetBorrowed input's pinned buffer: write the next value there."""
        ptr = self.lib.ghh_tape_input_buffer(self.h, node.id)
        if not ptr:
            raise EngineError(1, f"input: node {node.id} is not a borrowed input of this machine")
        return self._view(ptr, node)

    def value(self, borrowed):
        """The numpy view of a ReadBorrowed value (no copy; the next RunAll overwrites it)."""
        node = borrowed.node
        ptr = self.lib.ghh_tape_read_buffer(self.h, node.id)
        if not ptr:
            raise EngineError(1, f"value: node {node.id} is not a borrowed read of this machine")
        return self._view(ptr, node)

    def phase_ns(self):
        """Host nanoseconds of the last RunAll: (whole call, launching, waiting for the device)."""
        out = (C.c_int64 * 3)()
        self.lib.ghh_tape_phase_ns(self.h, out)
        return tuple(out)

    def submit_calls(self):
        return self.lib.ghh_tape_submit_calls(self.h)

    def register_address(self, node):
        return self.lib.ghh_tape_register_address(self.h, node.id)

    def program(self):
        n = self.lib.ghh_tape_program_string(self.h, None, 0)
        buf = C.create_string_buffer(n + 1)
        self.lib.ghh_tape_program_string(self.h, buf, n + 1)
        return buf.value.decode()


def NewLispMachine(g, *opts, **kw):
    """NewLispMachine(g) (vm_genera.go:43-120), forward execution: every node is run and waited for
    on its own.  The reference's tests run one graph on both machines and compare."""
    for o in opts:
        kw.update(o)
    return TapeMachine(g, node_at_a_time=True, **kw)


def WithEngine(e):
    """VMOpt of the reference (vm.go:318-329): NewTapeMachine(g, WithEngine(e))."""
    return {"engine": e}


def WithNaNWatch():
    """VMOpt of the reference (vm.go:138-151): watch for NaNs when executing; this slows the execution down."""
    return {"watch_nan": True}


def WithInfWatch():
    """VMOpt of the reference (vm.go:153-166): watch for +Inf and -Inf when executing."""
    return {"watch_inf": True}


def NewTapeMachine(g, *opts, **kw):
    for o in opts:
        kw.update(o)
    return TapeMachine(g, **kw)
