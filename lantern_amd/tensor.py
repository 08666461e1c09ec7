"""Tensor / TensorR front end over a Backend: the op surface models are written against.

Reference: src/main/scala/lantern/TensorDifferentiation.scala -- `Tensor` (386-1138), `TensorR`
(1146-1506), `gradR` / `gradR_loss` (1750-1780).  The reference gets reverse mode from delimited
continuations (`shift`/`reset`): each TensorR op runs forward, calls the continuation, then runs
its gradient code.  Here each op records its gradient code on a tape that `gradR*` replays in
reverse, which issues the same backend calls in the same order.

Every TensorR method below issues exactly the backend calls its Scala original stages, one per trait method, with every
buffer from `mallocArray` (zero-filled) and every gradient accumulated: nothing is fused or reordered on this side.  What
makes such a call sequence fast (conv -> batchNorm -> relu as one chain, gradients written instead of cleared and added,
one launch for the optimizer) happens inside the backend's library.
"""
import ctypes
import math

import numpy as np

from . import backend as B
from .backend import Buf, dim_broadcast, conv_size

_backend = None
_tape = []
_libc = ctypes.CDLL(None)
_libc.rand.restype = ctypes.c_int


def set_backend(b):
    """`backend = BackendXxx()` of the reference (TD:384)."""
    global _backend
    _backend = b
    return b


def get_backend():
    if _backend is None:
        raise RuntimeError("no backend set: call set_backend(BackendHIP(...)) and backend.setup() first")
    return _backend


def _prod(dims):
    p = 1
    for d in dims:
        p *= int(d)
    return p


def resize_dim(scalar_count, dims):
    """resizeDim (TD:36-49): at most one -1."""
    dims = [int(d) for d in dims]
    neg = [d for d in dims if d < 0]
    prod = _prod([d for d in dims if d >= 0])
    if len(neg) >= 2:
        raise ValueError("cannot have 2 or more -1s in resize!!")
    if not neg and prod != scalar_count:
        raise ValueError("must same size!!")
    return tuple(d if d > 0 else scalar_count // prod for d in dims)


class Random:
    """Random.rand / srand (TD:66-69): glibc rand(), `(float)rand()/RAND_MAX`."""

    @staticmethod
    def srand(seed):
        _libc.srand(ctypes.c_uint(seed))

    @staticmethod
    def rand_array(n):
        r = np.fromiter((_libc.rand() for _ in range(n)), dtype=np.int64, count=n)
        return r.astype(np.float32) / np.float32(2147483647)


class Tensor:
    """Dense row-major fp32 tensor: a backend buffer plus dims (TD:386-398)."""

    def __init__(self, data, dims):
        self.data = data
        if type(dims) is not tuple:
            dims = tuple(dims)
        n = 1
        for d in dims:
            n *= d
        if type(n) is not int:              # numpy integers in the shape: normalise once
            dims = tuple(int(d) for d in dims)
            n = int(n)
        self.shape = dims
        self.scalarCount = n
        self.rank = len(dims)

    # -- shape helpers ----------------------------------------------------------------------
    @property
    def strides(self):
        st, s = [], 1
        for d in reversed(self.shape):
            st.append(s); s *= d
        return tuple(reversed(st))

    @property
    def isScalar(self): return self.scalarCount == 1

    def __call__(self, i):
        """x(i): the i-th slice along dim 0 (TD:419-421)."""
        sub = self.shape[1:]
        return Tensor(self.data.offset(i * _prod(sub)), sub if sub else (1,))

    def resize(self, *dims):
        return Tensor(self.data, resize_dim(self.scalarCount, dims))

    # -- constructors (TD:1040-1123) ------------------------------------------------------------
    @staticmethod
    def zeros(*dims):
        return Tensor(get_backend().mallocArray(_prod(dims)), dims)

    @staticmethod
    def zeros_like(t):
        return Tensor(get_backend().mallocArray(t.scalarCount), t.shape)

    @staticmethod
    def fill(dims, value):
        be = get_backend()
        data = be.mallocArray(_prod(dims), zero=False)
        be.fillInPlace(data, _prod(dims), float(value))
        return Tensor(data, dims)

    @staticmethod
    def ones(*dims): return Tensor.fill(dims, 1.0)

    @staticmethod
    def scalar(v): return Tensor.fill((1,), v)

    @staticmethod
    def fromData(dims, *scalars):
        assert len(scalars) == _prod(dims)
        return Tensor.fromNumpy(np.asarray(scalars, dtype=np.float32).reshape(dims))

    @staticmethod
    def fromNumpy(arr):
        arr = np.ascontiguousarray(arr, dtype=np.float32)
        return Tensor(get_backend().fromHost(arr), arr.shape if arr.ndim else (1,))

    @staticmethod
    def fillWithBias(dims, bias, dim):
        return Tensor(get_backend().fillWithBias(tuple(dims), bias.data, dim), dims)

    @staticmethod
    def randseed(seed): Random.srand(seed)

    @staticmethod
    def randinit(dims, scale=1.0, seed=None):
        """(rand() - 0.5) * scale drawn on the host, then uploaded (CPU:101-110, CUB:154-155)."""
        if seed is not None:
            Random.srand(seed)
        r = (Random.rand_array(_prod(dims)) - np.float32(0.5)) * np.float32(scale)
        return Tensor.fromNumpy(r.reshape(dims))

    @staticmethod
    def rand(*dims, scale=1.0):
        if len(dims) == 2 and isinstance(dims[0], (tuple, list)):   # Tensor.rand(Seq(..), scale)
            dims, scale = tuple(dims[0]), dims[1]
        return Tensor.randinit(tuple(dims), scale)

    # -- host access ---------------------------------------------------------------------------
    def toCPU(self):
        """Contents as a numpy array (toCPU, CUB:68-107)."""
        return get_backend().toHost(self.data, self.scalarCount).reshape(self.shape)

    def copy_data(self, src):
        assert self.scalarCount == src.scalarCount
        get_backend().copyFloatArray(self.data, src.data, self.scalarCount)

    def clear(self): get_backend().fillInPlace(self.data, self.scalarCount, 0.0)
    def setAsOne(self): get_backend().fillInPlace(self.data, self.scalarCount, 1.0)
    def fillInPlace(self, v): get_backend().fillInPlace(self.data, self.scalarCount, float(v))
    def clipAt(self, bound): get_backend().clipAt(self.data, self.scalarCount, float(bound))

    @staticmethod
    def assertEqual(a, b, mes="", tal=0.0001):
        """Tensor.assertEqual (TD:1125-1138): same shape, |a-b| < tal element-wise."""
        assert a.shape == b.shape, "tensor not of the same dims %s vs %s %s" % (a.shape, b.shape, mes)
        x, y = a.toCPU(), b.toCPU()
        bad = ~(np.abs(x - y) < tal)
        assert not bad.any(), "%s not equal at %s: %s vs %s" % (mes, np.argwhere(bad)[0], x[bad][0], y[bad][0])

    # -- arithmetic ------------------------------------------------------------------------------
    def _bin(self, op, that):
        be = get_backend()
        if isinstance(that, Tensor):
            a, b, o = dim_broadcast(self.shape, that.shape)
            return Tensor(be.bcast_op(op, self.data, a, that.data, b, o), o), a, b
        return Tensor(be.scalar_op(op, self.data, float(that), self.scalarCount), self.shape)

    def _first(self, r): return r[0] if isinstance(r, tuple) else r
    def __add__(self, t): return self._first(self._bin(B.ADD, t))
    def __sub__(self, t): return self._first(self._bin(B.SUB, t))
    def __mul__(self, t): return self._first(self._bin(B.MUL, t))
    def __truediv__(self, t): return self._first(self._bin(B.DIV, t))

    def _ibin(self, op, that):
        be = get_backend()
        if isinstance(that, Tensor):
            if self.shape == that.shape:
                if op == B.ADD:             # the gradient accumulation of every operator: no shape arrays to pass
                    be.geam(self.data, 1.0, that.data, 1.0, self.data, self.scalarCount)
                    return self
                a = b = self.shape
            else:
                r = max(self.rank, that.rank)
                a = (1,) * (r - self.rank) + self.shape
                b = (1,) * (r - that.rank) + that.shape
            be.bcast_update(op, self.data, a, that.data, b)
        else:
            be.scalar_op(op, self.data, float(that), self.scalarCount, out=self.data)
        return self

    def __iadd__(self, t): return self._ibin(B.ADD, t)
    def __isub__(self, t): return self._ibin(B.SUB, t)
    def __imul__(self, t): return self._ibin(B.MUL, t)
    def __itruediv__(self, t): return self._ibin(B.DIV, t)

    def plusBias(self, bias): return self._ibin(B.ADD, bias)        # TD:265
    def plusEqual(self, adder): return self._ibin(B.ADD, adder)    # TD:269

    def addMul(self, a, b):
        """this += a * b with host scalar a (TD:757-764)."""
        get_backend().geam(self.data, 1.0, b.data, float(a), self.data, self.scalarCount)

    def dot(self, that):
        be = get_backend()
        if self.rank == 1 and that.rank == 1:
            assert self.shape[0] == that.shape[0], "vector vector dot not the same %d %d" % (self.shape[0], that.shape[0])
            return Tensor(be.vectorVectorDot(self.data, that.data, self.shape[0]), (1,))
        if self.rank == 2 and that.rank == 1:
            assert self.shape[1] == that.shape[0]
            return Tensor(be.matrixVectorDot(self.data, that.data, self.shape[0], self.shape[1]), (self.shape[0],))
        if self.rank == 2 and that.rank == 2:
            assert self.shape[1] == that.shape[0]
            return Tensor(be.matrixMatrixDot(self.data, that.data, self.shape[0], self.shape[1], that.shape[1]), (self.shape[0], that.shape[1]))
        raise ValueError("Incompatible shapes: %s, %s" % (self.shape, that.shape))

    @staticmethod
    def _gemm_dims(xs, tx, ys, ty):
        d1, d2 = (xs[1], xs[0]) if tx else (xs[0], xs[1])
        k2, d3 = (ys[1], ys[0]) if ty else (ys[0], ys[1])
        assert d2 == k2, "gemm dims don't match, got %s, %s" % (xs, ys)
        return d1, d2, d3

    def gemm(self, that, transX, transY, alpha):
        d1, d2, d3 = Tensor._gemm_dims(self.shape, transX, that.shape, transY)
        return Tensor(get_backend().gemm(self.data, transX, that.data, transY, float(alpha), d1, d2, d3), (d1, d3))

    def trans(self):
        assert self.rank == 2, "transpose is only for matrix. Tensor transpose is not supported here"
        return Tensor(get_backend().trans(self.data, self.shape[0], self.shape[1]), (self.shape[1], self.shape[0]))

    def permute(self, *dims):
        assert sorted(dims) == list(range(self.rank))
        return Tensor(get_backend().permute(self.data, self.shape, dims), tuple(self.shape[d] for d in dims))

    # -- activations -------------------------------------------------------------------------------
    def _unary(self, op, inPlace=False, lo=-1.0, hi=1.0):
        return Tensor(get_backend().unary(op, self.data, self.scalarCount, inPlace, lo, hi), self.shape)

    def relu(self, inPlace=False): return self._unary(B.RELU, inPlace)
    def tanh(self): return self._unary(B.TANH)
    def sigmoid(self): return self._unary(B.SIGMOID)
    def exp(self): return self._unary(B.EXP)
    def log(self): return self._unary(B.LOG)
    def sqrt(self): return self._unary(B.SQRT)
    def square(self): return self._unary(B.SQUARE)
    def hardTanh(self, min_val=-1.0, max_val=1.0, inPlace=False): return self._unary(B.HARDTANH, inPlace, min_val, max_val)

    # -- softmax / loss ------------------------------------------------------------------------------
    def _softmax_view(self, dim):
        dim = dim + self.rank if dim < 0 else dim
        return _prod(self.shape[:dim]), self.shape[dim], _prod(self.shape[dim + 1:])

    def softmax_batch(self, dim=1):
        o, c, i = self._softmax_view(dim)
        return Tensor(get_backend().softmax(False, self.data, o, c, i), self.shape)

    def logSoftmaxB(self, dim=1):
        o, c, i = self._softmax_view(dim)
        return Tensor(get_backend().softmax(True, self.data, o, c, i), self.shape)

    def nllLossB(self, target):
        assert self.rank == 2, "Input must be a 2-D tensor"
        return Tensor(get_backend().nllLoss(self.data, target, self.shape[0], self.shape[1]), (self.shape[0],))

    # -- reductions -----------------------------------------------------------------------------------
    def sum(self, dim=None):
        be = get_backend()
        if dim is None:
            return Tensor(be.sum(self.data, self.scalarCount), (1,))
        assert 0 <= dim < self.rank, "dim should be within range of this.nbDims"
        outer, d, inner = _prod(self.shape[:dim]), self.shape[dim], _prod(self.shape[dim + 1:])
        res = self.shape[:dim] + self.shape[dim + 1:]
        return Tensor(be.sum_dim(self.data, outer, d, inner), res if res else (1,))

    def mean(self):
        return Tensor(get_backend().mean(self.data, self.scalarCount), (1,))

    def batchNormAv(self):
        """Per-channel mean over (N,H,W) of a 4-D tensor (TD:523-538), as [C,1,1]."""
        assert self.rank == 4, "tensor for batch normal averaging should have 4 dimensions"
        n, c, h, w = self.shape
        be = get_backend()
        per_nc = Tensor(be.sum_dim(self.data, n * c, h * w, 1), (n, c))
        s = Tensor(be.sum_dim(per_nc.data, 1, n, c), (c, 1, 1))
        return s / float(n * h * w)

    # -- conv / pool / bn ---------------------------------------------------------------------------------
    @staticmethod
    def _pads2(pads):
        if len(pads) == 1: return pads[0], pads[0]
        if len(pads) == 2: return pads[0], pads[1]
        if len(pads) == 4: return pads[0], pads[2]
        raise ValueError("pads must have 1, 2 or 4 entries")

    def conv2D_batch(self, kernel, bias, strides, pads):
        assert self.rank == 4 and kernel.rank == 4 and self.shape[1] == kernel.shape[1]
        N, C, H, W = self.shape; K, _, R, S = kernel.shape
        sH, sW = strides[0], strides[1]; pH, pW = Tensor._pads2(pads)
        y, finput = get_backend().conv2D_batch(self.data, kernel.data, bias.data if bias is not None else None,
                                               N, C, H, W, K, R, S, sH, sW, pH, pW)
        return Tensor(y, (N, K, conv_size(H, R, sH, pH), conv_size(W, S, sW, pW))), finput

    def maxPool2D_batch(self, kernels, strides, pads=None):
        assert self.rank == 4, "the input for maxPool (with batch) should have 4 dimensions"
        assert len(kernels) == 2 and len(strides) == 2, "kernels and strides should be size 2"
        pad = 0
        if pads is not None:
            assert len(pads) == 4, "paddings should be size 4 for maxPool_k_batch"
            assert len(set(pads)) == 1 and pads[0] >= 0, "pad should be the same"
            pad = pads[0]
        N, C, H, W = self.shape
        y, idx = get_backend().maxPool2D_batch(self.data, N, C, H, W, kernels[0], kernels[1], strides[0], strides[1], pad)
        return Tensor(y, (N, C, conv_size(H, kernels[0], strides[0], pad), conv_size(W, kernels[1], strides[1], pad))), idx

    def averagePool2D_batch(self, kernels, strides, pads=None):
        """pads = (top, bottom, left, right) as ONNX orders them; the vertical pad is pads[0] and the horizontal one pads[2]
        (CDN:884-889), the divisor counts only elements inside the image (CDN:975-978)."""
        assert self.rank == 4
        pH, pW = _avg_pads(pads)
        N, C, H, W = self.shape
        y = get_backend().averagePool2D_batch(self.data, N, C, H, W, kernels[0], kernels[1], strides[0], strides[1], pH, pW)
        return Tensor(y, (N, C, conv_size(H, kernels[0], strides[0], pH), conv_size(W, kernels[1], strides[1], pW)))

    def _bn_view(self):
        if self.rank == 4: return self.shape[0], self.shape[1], self.shape[2] * self.shape[3]
        if self.rank == 2: return self.shape[0], self.shape[1], 1
        raise ValueError("batch norm expects a rank-4 (spatial) or rank-2 (per-activation) tensor")

    def batchNormInference(self, scale, bias, runningMean, runningVar):
        N, C, HW = self._bn_view()
        return Tensor(get_backend().batchNormInference(self.data, scale.data, bias.data, runningMean.data, runningVar.data, N, C, HW), self.shape)

    def batchNormTraining(self, scale, bias, runningMean, runningVar):
        N, C, HW = self._bn_view()
        y, sm, si = get_backend().batchNormTraining(self.data, scale.data, bias.data, runningMean.data, runningVar.data, N, C, HW)
        return Tensor(y, self.shape), Tensor(sm, (C,)), Tensor(si, (C,))

    batchNorm1DInference = batchNormInference
    batchNorm1DTraining = batchNormTraining

    def dropout(self, prob=0.5):
        y, mask = get_backend().dropout(self.data, self.scalarCount, float(prob))
        return Tensor(y, self.shape), mask

    def concat(self, dim, *others):
        ts = (self,) + others
        outer, inner = _prod(self.shape[:dim]), _prod(self.shape[dim + 1:])
        sizes = [t.shape[dim] for t in ts]
        res_shape = self.shape[:dim] + (sum(sizes),) + self.shape[dim + 1:]
        return Tensor(get_backend().concat([t.data for t in ts], sizes, outer, inner), res_shape)

    def repeat0(self, context):
        """TD:1446-1451 / CDN:378-386: [rows, ...] -> [rows - context, context + 1, ...], out[i0, i1] = in[i0 + i1]."""
        assert self.rank <= 3, "only support input with no more than 3D, got %d" % self.rank
        rows, inner = self.shape[0], _prod(self.shape[1:])
        assert 0 <= context < rows, "context must be smaller than the first dimension"
        return Tensor(get_backend().repeat0(self.data, rows, context, inner), (rows - context, context + 1) + tuple(self.shape[1:]))

    def mask4D(self, lengths):
        assert self.rank == 4
        get_backend().mask4D(self.data, lengths, *self.shape)
        return self

    def global_ave_batch(self):
        """Mean over H,W of [N,C,H,W] -> [N,C] (TD:880-906)."""
        n, c, h, w = self.shape
        s = Tensor(get_backend().sum_dim(self.data, n * c, h * w, 1), (n, c))
        s *= 1.0 / (h * w)
        return s


def _avg_pads(pads):
    if pads is None:
        return 0, 0
    assert len(pads) == 4, "paddings should be size 4"
    assert pads[0] == pads[1] and pads[2] == pads[3] and min(pads) >= 0, "pads must be symmetric"
    return int(pads[0]), int(pads[2])


def int_array(values):
    """An int32 array in backend memory (labels, lengths): `Array(...)` / `toGPU` of Rep[Array[Int]]."""
    return get_backend().fromHost(np.asarray(values, dtype=np.int32))


class TensorR:
    """A value with its gradient (TD:1146-1506).  `d` accumulates; inputs never receive one."""

    def __init__(self, x, d=None, isInput=False):
        """The gradient is allocated zero-filled at construction; an input gets a 2-element dummy (TD:1509-1514)."""
        self.x = x
        self.isInput = isInput
        self.d = d if d is not None else (Tensor.zeros(2) if isInput else Tensor.zeros_like(x))

    @staticmethod
    def _new(x):
        """Result of an op: `TensorR(x)`."""
        return TensorR(x)

    def __call__(self, i): return TensorR(self.x(i), self.d(i))

    def resize(self, *dims):
        nd = resize_dim(self.x.scalarCount, dims)
        return TensorR(Tensor(self.x.data, nd), Tensor(self.d.data, nd), self.isInput)     # a view: shares x and d

    def clip_grad(self, bound): self.d.clipAt(bound)
    def clear_grad(self): self.d.clear()

    # -- in-place adds --------------------------------------------------------------------------
    def plusBias(self, bias):
        self.x.plusBias(bias.x)
        def back():
            if not bias.isInput:
                bias.d += self.d                 # reduce main.d into bias.d (CPU:286-288)
        _tape.append(back)
        return self

    def plusEqual(self, that):
        self.x.plusEqual(that.x)
        def back():
            if not that.isInput:
                that.d += self.d
        _tape.append(back)
        return self

    # -- arithmetic --------------------------------------------------------------------------------
    def _bin(self, op, that):
        be = get_backend()
        if isinstance(that, TensorR):
            ya, a, b = self.x._bin(op, that.x)
            y = TensorR._new(ya)
            # add_grad / minus_grad / mul_grad / div_grad (TD:1171-1206): both operands' gradients in one backend call
            _tape.append(lambda: be.bcast_op_grad(op, self.x.data, self.d.data, a, self.isInput, that.x.data, that.d.data, b, that.isInput, y.d.data, ya.shape))
            return y
        s = float(that)
        y = TensorR._new(self.x._bin(op, s))
        def back():
            if self.isInput: return
            if op in (B.ADD, B.SUB): self.d += y.d                                   # TD:1167-1181
            elif op == B.MUL: be.geam(self.d.data, 1.0, y.d.data, s, self.d.data, self.d.scalarCount)   # TD:1190-1193
            else: self.d.addMul(1.0 / s, y.d)                                         # TD:1202-1205
        _tape.append(back)
        return y

    def __add__(self, t): return self._bin(B.ADD, t)
    def __sub__(self, t): return self._bin(B.SUB, t)
    def __mul__(self, t): return self._bin(B.MUL, t)
    def __truediv__(self, t): return self._bin(B.DIV, t)

    def dot(self, that):
        be = get_backend()
        y = TensorR._new(self.x.dot(that.x))
        def back():                                                                   # dot_grad (CPU:171-184)
            xr, yr = self.x.rank, that.x.rank
            if xr == 1 and yr == 1:
                if not self.isInput: be.addMul_scalar(self.d.data, y.d.data, that.x.data, self.x.scalarCount)
                if not that.isInput: be.addMul_scalar(that.d.data, y.d.data, self.x.data, that.x.scalarCount)
            elif xr == 2 and yr == 1:
                m, n = self.x.shape
                if not self.isInput: be.add_cartesian(self.d.data, that.x.data, y.d.data, m, n)
                if not that.isInput: be.add_composition(that.d.data, self.x.data, y.d.data, m, n)
            else:
                d1, d2 = self.x.shape; d3 = that.x.shape[1]
                if not self.isInput: be.add_dotTrans2(self.d.data, y.d.data, that.x.data, d1, d2, d3)
                if not that.isInput: be.add_dotTrans1(that.d.data, self.x.data, y.d.data, d1, d2, d3)
        _tape.append(back)
        return y

    def gemm(self, that, transX, transY, alpha):
        be = get_backend()
        d1, d2, d3 = Tensor._gemm_dims(self.x.shape, transX, that.x.shape, transY)
        y = TensorR._new(self.x.gemm(that.x, transX, transY, alpha))
        _tape.append(lambda: be.gemm_grad(self.x.data, self.d.data, self.isInput, transX, that.x.data, that.d.data, that.isInput, transY, float(alpha), y.d.data, d1, d2, d3))
        return y

    def trans(self):
        y = TensorR._new(self.x.trans())
        _tape.append(lambda: get_backend().trans_grad(self.d.data, y.d.data, self.x.shape[0], self.x.shape[1]))
        return y

    def permute(self, *dims):
        y = TensorR._new(self.x.permute(*dims))
        _tape.append(lambda: get_backend().permute_grad(self.d.data, y.d.data, self.x.shape, dims))
        return y

    # -- activations ----------------------------------------------------------------------------------
    def _unary(self, op, inPlace=False, lo=-1.0, hi=1.0):
        be = get_backend()
        if inPlace:
            self.x._unary(op, True, lo, hi)
            _tape.append(lambda: be.unary_grad(op, self.x.data, self.x.data, self.d.data, self.d.data, self.x.scalarCount, True, lo, hi))
            return self
        y = TensorR._new(self.x._unary(op, False, lo, hi))
        _tape.append(lambda: be.unary_grad(op, self.x.data, y.x.data, y.d.data, self.d.data, self.x.scalarCount, False, lo, hi))
        return y

    def relu(self, inPlace=False): return self._unary(B.RELU, inPlace)
    def hardTanh(self, min_val=-1.0, max_val=1.0, inPlace=False): return self._unary(B.HARDTANH, inPlace, min_val, max_val)
    def tanh(self): return self._unary(B.TANH)
    def sigmoid(self): return self._unary(B.SIGMOID)
    def exp(self): return self._unary(B.EXP)
    def log(self): return self._unary(B.LOG)
    def sqrt(self): return self._unary(B.SQRT)
    def square(self): return self._unary(B.SQUARE)

    def mask4D(self, lengths):
        self.x.mask4D(lengths)
        return self

    # -- reductions ---------------------------------------------------------------------------------------
    def sum(self, dim=None):
        be = get_backend()
        if dim is None:
            y = TensorR(self.x.sum(), Tensor.zeros(1))
            _tape.append(lambda: be.add_scalar_from(self.d.data, y.d.data, 1.0, self.x.scalarCount))
            return y
        y = TensorR._new(self.x.sum(dim))
        sh = self.x.shape
        outer, d, inner = _prod(sh[:dim]), sh[dim], _prod(sh[dim + 1:])
        _tape.append(lambda: be.sum_dim_grad(self.d.data, y.d.data, outer, d, inner))
        return y

    def mean(self):
        be = get_backend()
        y = TensorR(self.x.mean(), Tensor.zeros(1))
        _tape.append(lambda: be.add_scalar_from(self.d.data, y.d.data, 1.0 / self.x.scalarCount, self.x.scalarCount))
        return y

    # -- bn / softmax / loss ----------------------------------------------------------------------------------
    def batchNorm(self, scale, bias, runningMean, runningVar):
        """TD:1367-1372: batchNormTraining, then batchNorm_grad with the saved statistics."""
        be = get_backend()
        N, C, HW = self.x._bn_view()
        yv, sm, si = self.x.batchNormTraining(scale.x, bias.x, runningMean, runningVar)
        y = TensorR._new(yv)
        _tape.append(lambda: be.batchNorm_grad(self.x.data, None if self.isInput else self.d.data, y.d.data, scale.x.data, scale.d.data, bias.d.data,
                                               sm.data, si.data, N, C, HW))
        return y

    batchNorm1D = batchNorm

    def softmax_batch(self, dim=1):
        be = get_backend()
        o, c, i = self.x._softmax_view(dim)
        y = TensorR._new(self.x.softmax_batch(dim))
        _tape.append(lambda: be.softmax_grad(False, y.x.data, y.d.data, self.d.data, o, c, i))
        return y

    def logSoftmaxB(self, dim=1):
        be = get_backend()
        o, c, i = self.x._softmax_view(dim)
        y = TensorR._new(self.x.logSoftmaxB(dim))
        _tape.append(lambda: be.softmax_grad(True, y.x.data, y.d.data, self.d.data, o, c, i))
        return y

    def nllLossB(self, target):
        be = get_backend()
        assert self.x.rank == 2, "nllLossB() function only takes tensor of rank 2, got %s" % (self.x.shape,)
        y = TensorR._new(self.x.nllLossB(target))
        _tape.append(lambda: be.nllLoss_grad(self.d.data, target, y.d.data, self.x.shape[0], self.x.shape[1]))
        return y

    # -- conv / pool ----------------------------------------------------------------------------------------------
    def convBBP(self, kernel, bias, strides, pads):
        be = get_backend()
        assert self.isInput or self.d.scalarCount == self.x.scalarCount, "For convBBP, THIS is either input or intermediate stage"
        assert self.x.rank == 4, "For convBBP, THIS is dim 4: batch, channel, row, col"
        assert kernel.x.rank == 4 and self.x.shape[1] == kernel.x.shape[1]
        N, C, H, W = self.x.shape; K, _, R, S = kernel.x.shape
        sH, sW = strides[0], strides[1]; pH, pW = Tensor._pads2(pads)
        yv, finput = self.x.conv2D_batch(kernel.x, bias.x if bias is not None else None, strides, pads)
        y = TensorR._new(yv)
        be.convs_open += 1                  # forward convolutions whose gradient is still to come (a backend may run filter gradients beside the ones that follow)
        def back():
            be.convs_open -= 1
            be.conv2D_batch_grad(self.x.data, None if self.isInput else self.d.data, self.isInput, finput, kernel.x.data, kernel.d.data, y.d.data,
                                 bias.d.data if bias is not None else None, N, C, H, W, K, R, S, sH, sW, pH, pW)
        _tape.append(back)
        return y

    def maxPoolBK(self, kernels, strides, pads=None):
        be = get_backend()
        yv, idx = self.x.maxPool2D_batch(kernels, strides, pads)
        y = TensorR._new(yv)
        N, C, H, W = self.x.shape
        geom = (N, C, H, W, kernels[0], kernels[1], strides[0], strides[1], pads[0] if pads else 0)
        _tape.append(lambda: be.maxPool2D_batch_grad(self.d.data, y.d.data, idx, yv.scalarCount, geom))
        return y

    def averagePoolBK(self, kernels, strides, pads=None):
        be = get_backend()
        y = TensorR._new(self.x.averagePool2D_batch(kernels, strides, pads))
        N, C, H, W = self.x.shape
        pH, pW = _avg_pads(pads)
        _tape.append(lambda: be.averagePool2D_batch_grad(self.d.data, y.d.data, N, C, H, W, kernels[0], kernels[1], strides[0], strides[1], pH, pW))
        return y

    def global_ave_batch(self):
        be = get_backend()
        y = TensorR._new(self.x.global_ave_batch())
        n, c, h, w = self.x.shape
        def back():                                  # TD:1454-1479: d += ty.d * (1/HW) broadcast over H,W
            scaled = y.d * (1.0 / (h * w))
            be.sum_dim_grad(self.d.data, scaled.data, n * c, h * w, 1)
        _tape.append(back)
        return y

    def concat(self, dim, *others):
        be = get_backend()
        ts = (self,) + others
        y = TensorR._new(self.x.concat(dim, *[t.x for t in others]))
        outer, inner = _prod(self.x.shape[:dim]), _prod(self.x.shape[dim + 1:])
        sizes = [t.x.shape[dim] for t in ts]
        _tape.append(lambda: be.concat_grad([None if t.isInput else t.d.data for t in ts], sizes, y.d.data, outer, inner))
        return y

    # -- recurrent layer, CTC ----------------------------------------------------------------------------
    def rnn(self, mode, params, hidden, bidirectional, offset=0, hx=None, cx=None):
        """RNNBase.apply (NN:392-415): one layer over [seqLength, batch, inputSize];
        `params` is the packed parameter buffer (a TensorR), this layer's parameters starting `offset` elements in.
        mode 0 = relu, 1 = tanh, 2 = LSTM, 3 = GRU (cuDNN's numbering).  `hx`, `cx`: this layer's initial hidden and cell
        state as plain data [numDirections, batch, hidden] (None = zeros); they receive no gradient (CDN:1843-1844 pass NULL)."""
        be = get_backend()
        assert self.x.rank == 3, "RNN input should have rank 3: [seqLength x batchSize x inputSize]"
        T, Bn, I = self.x.shape
        D = 2 if bidirectional else 1
        w, dw = (params.x.data, params.d.data) if offset == 0 else (params.x.data.offset(offset), params.d.data.offset(offset))
        assert cx is None or mode == 2, "only the LSTM has a cell state"
        if mode >= 2:
            ybuf, reserve = be.rnn_gated_forward(mode, self.x.data, w, T, Bn, I, hidden, bidirectional, hx=hx, cx=cx)
        else:
            ybuf = be.rnn_forward(mode, self.x.data, w, T, Bn, I, hidden, bidirectional, hx=hx)
        y = TensorR._new(Tensor(ybuf, (T, Bn, D * hidden)))
        def back():
            xd = None if self.isInput else self.d.data
            if mode >= 2:
                be.rnn_gated_backward(mode, self.x.data, ybuf, y.d.data, w, reserve, xd, dw, T, Bn, I, hidden, bidirectional, hx=hx, cx=cx)
            else:
                be.rnn_backward(mode, self.x.data, ybuf, y.d.data, w, xd, dw, T, Bn, I, hidden, bidirectional, hx=hx)
        _tape.append(back)
        return y

    def ctcLoss(self, inputLengths, labels, labelLengths):
        """TD:1381-1382 + CDN:1895-1938: `self` holds softmax outputs [T, B, A]; the per-sample costs are
        averaged into the returned 1-element Tensor and the gradient is written into self.d right away
        (there is no tape entry: the result is a plain Tensor, as in the reference)."""
        be = get_backend()
        assert self.x.rank == 3, "Probability tensor should have rank 3: [inputLength, batchSize, alphabetSize]"
        T, Bn, A = self.x.shape
        assert Bn <= 256, "'cudnnGetCTCLossWorkspaceSize' requires batch size less than 256, got %d" % Bn
        costs = be.ctcLoss(self.x.data, self.d.data, inputLengths, labels, labelLengths, T, Bn, A)
        return Tensor(costs, (Bn,)).mean()

    def repeat0(self, context):
        be = get_backend()
        y = TensorR._new(self.x.repeat0(context))
        rows, inner = self.x.shape[0], _prod(self.x.shape[1:])
        def back():
            if not self.isInput: be.repeat0_grad(self.d.data, y.d.data, rows, context, inner)
        _tape.append(back)
        return y

    def dropout(self, prob):
        be = get_backend()
        yv, mask = self.x.dropout(prob)
        y = TensorR._new(yv)
        _tape.append(lambda: be.dropout_grad(self.d.data, y.d.data, mask, self.x.scalarCount))
        return y


def _run_tape(start):
    while len(_tape) > start:
        _tape.pop()()


def gradR(f):
    """gradR (TD:1750-1758): returns the gradient of the input; the output gradient is seeded with ones."""
    def run(x):
        x1 = TensorR(x, Tensor.zeros_like(x))
        start = len(_tape)
        y = f(x1)
        y.d.setAsOne()
        _run_tape(start)
        return x1.d
    return run


def gradR_loss(f):
    """gradR_loss (TD:1763-1780): returns the loss value; gradients land in the closed-over TensorRs."""
    def run(x):
        x1 = TensorR(x)
        be = get_backend()
        res = be.mallocArray(1)
        start = len(_tape)
        y = f(x1)
        assert y.x.scalarCount == 1, "Loss function must return a Tensor of size 1, got %d" % y.x.scalarCount
        y.d.setAsOne()
        be.copyFloatArray(res, y.x.data, 1)
        _run_tape(start)
        return Tensor(res, (1,))
    return run
