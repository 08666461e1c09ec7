"""The trait's own method names (lantern_amd/trait.py over src/main/scala/lantern/TensorDifferentiation.scala:137-379): every
name the reference's `Backend` declares exists on the mirror, and the ones that are thin views of a grouped method give what
the tape gives.  Runs on the oracle backend without a GPU and on the device."""
import os
import re

import numpy as np
import pytest

import lantern_amd as la
from lantern_amd.tensor import Tensor, TensorR, gradR
from lantern_amd.trait import Trait

# the 89 method names of the trait, as declared between TensorDifferentiation.scala:137 and :379
TRAIT_METHODS = """setup cleanup mallocArray copyFloatArray copyTensorData arrayToTensor makeTensor fill fillWithBias fillInPlace randinit clipAt
mutate mapInPlace changeTo map fold vectorVectorDot matrixVectorDot matrixMatrixDot dot_grad add_cartesian add_composition add_dotTrans1
add_dotTrans2 gemm gemm_grad trans trans_grad permute permute_grad geam add_grad minus_grad mul_grad div_grad plusBias plusBias_grad
plusEqual plusEqual_grad conv2D_batch conv2D_batch_grad mask4D maxPool2D_batch maxPool2D_batch_grad averagePool2D_batch
averagePool2D_batch_grad batchNormInference batchNormTraining batchNorm_grad batchNorm1DInference batchNorm1DTraining batchNorm1D_grad
dropout dropout_grad relu tanh sigmoid hardTanh exp log sqrt square relu_grad tanh_grad sigmoid_grad hardTanh_grad exp_grad log_grad
sqrt_grad square_grad softmax logSoftmax softmax_grad logSoftmax_grad sum sum_grad mean mean_grad concat concat_grad repeat0 repeat0_grad
nllLoss nllLoss_grad ctcLoss adagrad_update momentum_update""".split()


def test_every_trait_method_has_a_home():
    """By its own name on the trait view, on the grouped backend, or as the Tensor / TensorR method that issues it."""
    from lantern_amd.backend import Backend, BackendHIP
    homes = (Trait, BackendHIP, Backend, Tensor, TensorR)
    alias = {"vectorVectorDot": "dot", "matrixVectorDot": "dot", "matrixMatrixDot": "dot", "randinit": "rand", "clipAt": "clipAt",
             "fillWithBias": "fillWithBias", "plusBias": "plusBias", "plusEqual": "plusEqual", "gemm_grad": "gemm", "relu": "relu"}
    missing = [m for m in TRAIT_METHODS if not any(hasattr(h, m) or hasattr(h, alias.get(m, m)) for h in homes)]
    assert not missing, missing


def _vals(*ts):
    return [t.toCPU().copy() for t in ts]


def test_trait_named_gradients_match_the_tape(be):
    t = Trait()
    rng = np.random.RandomState(61)
    a = rng.randn(3, 4).astype(np.float32); b = (rng.rand(4) + 0.5).astype(np.float32); g = rng.randn(3, 4).astype(np.float32)

    # arithmetic with broadcasting: tape vs the trait-named call on hand-made TensorRs
    for name, fn in (("add_grad", lambda x, y: x + y), ("minus_grad", lambda x, y: x - y), ("mul_grad", lambda x, y: x * y), ("div_grad", lambda x, y: x / y)):
        x1, y1 = TensorR(Tensor.fromNumpy(a)), TensorR(Tensor.fromNumpy(b))
        from lantern_amd.tensor import _tape, _run_tape
        start = len(_tape)
        out = fn(x1, y1)
        be.upload(out.d.data, g)
        _run_tape(start)
        x2, y2 = TensorR(Tensor.fromNumpy(a)), TensorR(Tensor.fromNumpy(b))
        out2 = TensorR(Tensor.fromNumpy(out.x.toCPU()), Tensor.fromNumpy(g))
        getattr(t, name)(x2, y2, out2, x2.x.shape, y2.x.shape)
        np.testing.assert_allclose(x2.d.toCPU(), x1.d.toCPU(), rtol=1e-6, err_msg=name)
        np.testing.assert_allclose(y2.d.toCPU(), y1.d.toCPU(), rtol=1e-5, err_msg=name)

    # activations
    pos = (np.abs(a) + 0.5).astype(np.float32)
    for name, method, src in (("relu_grad", "relu", a), ("tanh_grad", "tanh", a), ("sigmoid_grad", "sigmoid", a), ("exp_grad", "exp", a),
                              ("log_grad", "log", pos), ("sqrt_grad", "sqrt", pos), ("square_grad", "square", a)):
        x1 = TensorR(Tensor.fromNumpy(src))
        start = len(_tape)
        out = getattr(x1, method)()
        be.upload(out.d.data, g)
        _run_tape(start)
        x2 = TensorR(Tensor.fromNumpy(src))
        out2 = TensorR(Tensor.fromNumpy(out.x.toCPU()), Tensor.fromNumpy(g))
        getattr(t, name)(x2, out2)
        np.testing.assert_allclose(x2.d.toCPU(), x1.d.toCPU(), rtol=1e-6, err_msg=name)

    # logSoftmax, sum, mean
    x1 = TensorR(Tensor.fromNumpy(a))
    start = len(_tape); out = x1.logSoftmaxB(1); be.upload(out.d.data, g); _run_tape(start)
    x2 = TensorR(Tensor.fromNumpy(a))
    ls = t.logSoftmax(x2.x, 1)
    np.testing.assert_allclose(ls.toCPU(), out.x.toCPU(), rtol=1e-6)
    t.logSoftmax_grad(x2, TensorR(ls, Tensor.fromNumpy(g)), 1)
    np.testing.assert_allclose(x2.d.toCPU(), x1.d.toCPU(), rtol=1e-5)
    x3 = TensorR(Tensor.fromNumpy(a)); t.sum_grad(x3, TensorR(Tensor.fromNumpy(np.zeros(1, np.float32)), Tensor.fromNumpy(np.array([2.0], np.float32))))
    np.testing.assert_allclose(x3.d.toCPU(), np.full(a.size, 2.0, np.float32).reshape(x3.d.toCPU().shape))
    x4 = TensorR(Tensor.fromNumpy(a)); t.mean_grad(x4, TensorR(Tensor.fromNumpy(np.zeros(1, np.float32)), Tensor.fromNumpy(np.array([6.0], np.float32))))
    np.testing.assert_allclose(x4.d.toCPU(), np.full(a.size, 0.5, np.float32).reshape(x4.d.toCPU().shape))
    x5 = TensorR(Tensor.fromNumpy(a)); t.sum_grad(x5, TensorR(Tensor.fromNumpy(np.zeros(3, np.float32)), Tensor.fromNumpy(np.array([1, 2, 3], np.float32))), 1)
    np.testing.assert_allclose(x5.d.toCPU().reshape(3, 4), np.repeat(np.array([[1.], [2.], [3.]], np.float32), 4, axis=1))

    # construction, copies, batchNorm1D, repeat0, the ??? methods
    m = t.makeTensor((2, 2), 1.0, 2.0, 3.0, 4.0)
    assert m.shape == (2, 2) and m.toCPU().ravel().tolist() == [1.0, 2.0, 3.0, 4.0]
    c = Tensor.zeros(2, 2); t.copyTensorData(c, m)
    assert np.array_equal(c.toCPU(), m.toCPU()) and t.arrayToTensor(m.data, 4).shape == (4,)
    xb = Tensor.fromNumpy(rng.randn(6, 4).astype(np.float32))
    sc, bi, rm, rv = Tensor.ones(4), Tensor.zeros(4), Tensor.zeros(4), Tensor.ones(4)
    y, sm, si, counter = t.batchNorm1DTraining(xb, sc, bi, rm, rv)
    yv = y.toCPU().reshape(6, 4)
    np.testing.assert_allclose(yv.mean(axis=0), 0.0, atol=1e-6); np.testing.assert_allclose(yv.var(axis=0), 1.0, rtol=1e-3)
    xr = TensorR(xb); scr, bir = TensorR(sc), TensorR(bi)
    t.batchNorm1D_grad(xr, TensorR(y, Tensor.fromNumpy(np.ones((6, 4), np.float32))), scr, bir, sm, si, counter)
    np.testing.assert_allclose(bir.d.toCPU(), 6.0, rtol=1e-6); np.testing.assert_allclose(xr.d.toCPU(), 0.0, atol=1e-5)   # a constant gradient is projected out
    assert t.batchNorm1DInference(xb, sc, bi, Tensor.zeros(4), Tensor.ones(4)).shape == (6, 4)
    r = t.repeat0(Tensor.fromNumpy(np.arange(8, dtype=np.float32).reshape(4, 2)), 1)
    assert r.shape == (3, 2, 2) and r.toCPU().ravel().tolist() == [0, 1, 2, 3, 2, 3, 4, 5, 4, 5, 6, 7]
    for name in ("map", "fold", "mutate", "mapInPlace", "changeTo"):
        with pytest.raises(NotImplementedError):
            getattr(t, name)(m, lambda v: v)
