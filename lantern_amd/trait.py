"""The reference's `Backend` trait by its own method names.

`lantern_amd.backend.Backend` groups the trait's methods by kernel family (one `unary_grad` for the eight activation
gradients, one `bcast_op_grad` for the four arithmetic ones, `softmax(is_log, ...)`, `batchNorm*` for both ranks).  Code
written against the trait (src/main/scala/lantern/TensorDifferentiation.scala:137-379) finds the remaining names here, with
the trait's argument lists (`Tensor` / `TensorR` objects, not raw buffers), each a line or two over the grouped method:

    t = Trait()                      # over the current backend
    t.relu_grad(x, y, inPlace=True); t.add_grad(a, b, out, a.x.shape, b.x.shape); t.logSoftmax_grad(x, y, 1) ...

The host-lambda methods (`map`, `fold`, `mutate`, `mapInPlace`, `changeTo`) are `???` in the reference's GPU backends
(TensorDslCublas.scala:164-168) and raise here as well.
"""
import numpy as np

from . import backend as B
from .tensor import Tensor, TensorR, get_backend, _prod


def _padded(shape, rank):
    shape = tuple(int(d) for d in shape)
    return (1,) * (rank - len(shape)) + shape


class Trait:
    def __init__(self, backend=None):
        self._be = backend

    @property
    def be(self):
        return self._be if self._be is not None else get_backend()

    # -- construction and copies (TD:145-160) --------------------------------------------------------
    def copyTensorData(self, dest, src):
        assert dest.scalarCount == src.scalarCount, "Tensors do not have same scalar count"
        self.be.copyFloatArray(dest.data, src.data, dest.scalarCount)

    def arrayToTensor(self, array, *dims):
        return Tensor(array, tuple(dims))

    def makeTensor(self, dims, *scalars):
        return Tensor.fromNumpy(np.asarray(scalars, dtype=np.float32).reshape(tuple(dims)))

    def _host_lambda(self, *a, **k):
        raise NotImplementedError("a host function over device elements: ??? in the reference's GPU backends as well (TensorDslCublas.scala:164-168)")

    mutate = mapInPlace = changeTo = map = fold = _host_lambda

    # -- arithmetic gradients (TD:213-262) -------------------------------------------------------------
    def _bin_grad(self, op, x, y, output, xShape, yShape):
        rank = output.x.rank
        self.be.bcast_op_grad(op, x.x.data, x.d.data, _padded(xShape, rank), x.isInput,
                              y.x.data, y.d.data, _padded(yShape, rank), y.isInput, output.d.data, output.x.shape)

    def add_grad(self, x, y, output, xShape, yShape): self._bin_grad(B.ADD, x, y, output, xShape, yShape)
    def minus_grad(self, x, y, output, xShape, yShape): self._bin_grad(B.SUB, x, y, output, xShape, yShape)
    def mul_grad(self, x, y, output, xShape, yShape): self._bin_grad(B.MUL, x, y, output, xShape, yShape)
    def div_grad(self, x, y, output, xShape, yShape): self._bin_grad(B.DIV, x, y, output, xShape, yShape)

    def plusBias_grad(self, main, bias):
        if not bias.isInput: bias.d += main.d                      # main.d reduced over the broadcast axes (CPU:286-288)

    def plusEqual_grad(self, base, adder):
        if not adder.isInput: adder.d += base.d

    def dot_grad(self, x, y, output):                              # CPU:171-184
        be, xr, yr = self.be, x.x.rank, y.x.rank
        if xr == 1 and yr == 1:
            if not x.isInput: be.addMul_scalar(x.d.data, output.d.data, y.x.data, x.x.scalarCount)
            if not y.isInput: be.addMul_scalar(y.d.data, output.d.data, x.x.data, y.x.scalarCount)
        elif xr == 2 and yr == 1:
            m, n = x.x.shape
            if not x.isInput: be.add_cartesian(x.d.data, y.x.data, output.d.data, m, n)
            if not y.isInput: be.add_composition(y.d.data, x.x.data, output.d.data, m, n)
        else:
            d1, d2 = x.x.shape; d3 = y.x.shape[1]
            if not x.isInput: be.add_dotTrans2(x.d.data, output.d.data, y.x.data, d1, d2, d3)
            if not y.isInput: be.add_dotTrans1(y.d.data, x.x.data, output.d.data, d1, d2, d3)

    # -- activations (TD:319-335) ------------------------------------------------------------------------
    def _act_grad(self, op, input, res, inPlace=False, lo=-1.0, hi=1.0):
        self.be.unary_grad(op, input.x.data, res.x.data, res.d.data, input.d.data, input.x.scalarCount, inPlace, lo, hi)

    def relu_grad(self, input, res, inPlace=False): self._act_grad(B.RELU, input, res, inPlace)
    def tanh_grad(self, input, res): self._act_grad(B.TANH, input, res)
    def sigmoid_grad(self, input, res): self._act_grad(B.SIGMOID, input, res)
    def exp_grad(self, input, res): self._act_grad(B.EXP, input, res)
    def log_grad(self, input, res): self._act_grad(B.LOG, input, res)
    def sqrt_grad(self, input, res): self._act_grad(B.SQRT, input, res)
    def square_grad(self, input, res): self._act_grad(B.SQUARE, input, res)
    def hardTanh_grad(self, input, res, min_val=-1.0, max_val=1.0, inPlace=False): self._act_grad(B.HARDTANH, input, res, inPlace, min_val, max_val)

    # -- softmax, reductions (TD:337-347) --------------------------------------------------------------
    def logSoftmax(self, x, dim=1):
        return x.logSoftmaxB(dim)

    def logSoftmax_grad(self, input, res, dim=1):
        o, c, i = input.x._softmax_view(dim)
        self.be.softmax_grad(True, res.x.data, res.d.data, input.d.data, o, c, i)

    def sum_grad(self, input, res, dim=None):
        if dim is None:
            self.be.add_scalar_from(input.d.data, res.d.data, 1.0, input.x.scalarCount)
        else:
            sh = input.x.shape
            self.be.sum_dim_grad(input.d.data, res.d.data, _prod(sh[:dim]), sh[dim], _prod(sh[dim + 1:]))

    def mean_grad(self, input, res):
        self.be.add_scalar_from(input.d.data, res.d.data, 1.0 / input.x.scalarCount, input.x.scalarCount)

    # -- batch norm over [N, C] (TD:309-315): the rank-2 case of the batchNorm* methods ------------------------------
    def batchNorm1DInference(self, x, scale, bias, runningMean, runningVar):
        assert x.rank == 2, "batchNorm1D expects [batch, features]"
        return x.batchNormInference(scale, bias, runningMean, runningVar)

    def batchNorm1DTraining(self, x, scale, bias, runningMean, runningVar):
        assert x.rank == 2, "batchNorm1D expects [batch, features]"
        y, sm, si = x.batchNormTraining(scale, bias, runningMean, runningVar)
        return y, sm, si, 0

    def batchNorm1D_grad(self, input, res, scale, bias, saveMean, saveInvVariance, counterId=0):
        N, C = input.x.shape
        self.be.batchNorm_grad(input.x.data, None if input.isInput else input.d.data, res.d.data, scale.x.data, scale.d.data, bias.d.data,
                               saveMean.data, saveInvVariance.data, N, C, 1)

    # -- repeat0 (TD:348-349) ------------------------------------------------------------------------------
    def repeat0(self, x, context):
        return x.repeat0(context)

    def repeat0_grad(self, input, out, context):
        if not input.isInput:
            self.be.repeat0_grad(input.d.data, out.d.data, input.x.shape[0], context, _prod(input.x.shape[1:]))
