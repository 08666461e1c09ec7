"""Known-answer vectors held by the reference's own unit tests, replayed through the same
Tensor/TensorR programs on the CPU oracle (always) and on BackendHIP (-m gpu).

Each test names the reference test it restates.  T/ = src/test/scala/lantern/.
These vectors are what pins the oracle: a dropped term, a wrong sign or a transposed operand in
oracle/lantern_cpu.c fails one of them.
"""
import json
import os

import numpy as np
import pytest

import lantern_amd as la
from lantern_amd import Tensor, TensorR, gradR, gradR_loss, int_array

HERE = os.path.dirname(os.path.abspath(__file__))


def T(dims, *vals):
    return Tensor.fromData(dims, *vals)


def eq(expected, got, tol=1e-4):
    Tensor.assertEqual(expected, got, tal=tol)


def test_vector_vector_dot(be):  # T/TestTensorDifferentiation.scala:61-75
    eq(Tensor.scalar(-30), T((4,), 1, 2, 3, 4).dot(T((4,), -1, -2, -3, -4)))


def test_matrix_vector_dot(be):  # T/TestTensorDifferentiation.scala:77-100; T/TestCublas.scala:25-52
    m, v = T((2, 4), 1, 2, 3, 4, 5, 6, 7, 8), T((4,), -1, -2, -3, -4)
    eq(T((2,), -30, -70), m.dot(v))
    mm, vv = TensorR(m), TensorR(v)
    gradR_loss(lambda dummy: mm.dot(vv).sum())(Tensor.zeros(1))
    eq(T((2, 4), -1, -2, -3, -4, -1, -2, -3, -4), mm.d)
    eq(T((4,), 6, 8, 10, 12), vv.d)


def test_matrix_matrix_dot(be):  # T/TestTensorDifferentiation.scala:102-124
    m1, m2 = T((2, 3), 1, 2, 3, 4, 5, 6), T((3, 2), 2, 3, 4, 2, 3, 4)
    eq(T((2, 2), 19, 19, 46, 46), m1.dot(m2))
    a, b = TensorR(m1), TensorR(m2)
    gradR_loss(lambda dummy: a.dot(b).sum())(Tensor.zeros(1))
    eq(T((2, 3), 5, 6, 7, 5, 6, 7), a.d)
    eq(T((3, 2), 5, 5, 7, 7, 9, 9), b.d)


def test_vector_vector_dot_grad(be):  # dot_grad rank (1,1): CPU:173-175
    a, b = TensorR(T((3,), 1, 2, 3)), TensorR(T((3,), 4, 5, 6))
    loss = gradR_loss(lambda dummy: a.dot(b))(Tensor.zeros(1))
    eq(Tensor.scalar(32), loss)
    eq(T((3,), 4, 5, 6), a.d)
    eq(T((3,), 1, 2, 3), b.d)


def test_gemm_equals_dot_trans(be):  # T/TestTensorDifferentiation.scala:126-150 (property on rand inputs)
    Tensor.randseed(7)
    m1, m2, m3, m4 = Tensor.rand(2, 3), Tensor.rand(3, 4), Tensor.rand(4, 3), Tensor.rand(3, 2)
    eq(m1.dot(m2) * 0.5, m1.gemm(m2, False, False, 0.5))
    eq(m1.dot(m3.trans()) * 0.5, m1.gemm(m3, False, True, 0.5))
    eq(m4.trans().dot(m2) * 0.5, m4.gemm(m2, True, False, 0.5))
    eq(m4.trans().dot(m3.trans()) * 0.5, m4.gemm(m3, True, True, 0.5))


def test_gemm_grad_equals_dot_grad(be):  # T/TestTensorDifferentiation.scala:152-194
    Tensor.randseed(8)
    m1, m2, m3, m4 = Tensor.rand(2, 3), Tensor.rand(3, 4), Tensor.rand(4, 3), Tensor.rand(3, 2)
    cases = [(m1, m2, False, False), (m1, m3, False, True), (m4, m2, True, False), (m4, m3, True, True)]
    for x, y, tx, ty in cases:
        a, b, c, d = TensorR(x), TensorR(y), TensorR(x), TensorR(y)
        gradR(lambda _: ((a.trans() if tx else a).dot(b.trans() if ty else b)) * 0.5)(Tensor.zeros(1))
        gradR(lambda _: c.gemm(d, tx, ty, 0.5))(Tensor.zeros(1))
        eq(a.d, c.d)
        eq(b.d, d.d)


def test_softmax(be):  # T/TestTensorDifferentiation.scala:196-221; T/TestCudnn.scala:751-773
    r = T((2, 3), 1, 2, 3, 4, 5, 6).softmax_batch()
    eq(T((2, 3), 0.0900305733, 0.2447284758, 0.6652409434, 0.0900305733, 0.2447284758, 0.6652409434), r)


def test_softmax_grad(be):  # T/TestCudnn.scala:751-773 (grad of sum-seeded softmax is ~0)
    g = gradR(lambda x: x.softmax_batch())(T((2, 3), 1, 2, 3, 4, 5, 6))
    eq(Tensor.zeros(2, 3), g, tol=1e-6)


def test_log_softmax(be):  # T/TestTensorDifferentiation.scala:223-243; T/TestCudnn.scala:775-795
    inp = T((2, 3), 1, 2, 3, 4, 5, 6)
    eq(T((2, 3), -2.4076058865, -1.4076058865, -0.4076058865, -2.4076061249, -1.4076061249, -0.4076061249), inp.logSoftmaxB())
    g = gradR(lambda x: x.logSoftmaxB())(inp)
    eq(T((2, 3), 0.7299082279, 0.2658145428, -0.9957230091, 0.7299083471, 0.2658147216, -0.9957225323), g)


def test_nll_loss(be):  # T/TestTensorDifferentiation.scala:245-266; T/TestCudnn.scala:917-938
    inp, tgt = T((2, 3), 1, 2, 3, 4, 5, 6), int_array([1, 0])
    eq(T((2,), 1.4076058865, 2.4076061249), inp.logSoftmaxB().nllLossB(tgt))
    g = gradR(lambda x: x.logSoftmaxB().nllLossB(tgt))(inp)
    eq(T((2, 3), 0.0900305808, -0.7552714944, 0.6652410030, -0.9099694490, 0.2447284311, 0.6652408242), g)


def test_maxpool_first_max_and_grad(be):  # T/TestTensorDifferentiation.scala:986-1040 (ones: first max wins)
    x = TensorR(Tensor.ones(1, 2, 8, 10))
    loss = gradR_loss(lambda d: x.maxPoolBK((2, 2), (2, 2)).sum())(Tensor.scalar(0))
    eq(Tensor.scalar(2 * 4 * 5), loss)
    exp = np.zeros((1, 2, 8, 10), np.float32); exp[:, :, ::2, ::2] = 1
    eq(Tensor.fromNumpy(exp), x.d)


def test_maxpool_k2s1(be):  # T/TestCudnn.scala:797-836
    inp = T((1, 1, 3, 3), 1, 2, 3, 4, 5, 6, 7, 8, 9)
    out, idx = inp.maxPool2D_batch((2, 2), (1, 1), None)
    eq(T((1, 1, 2, 2), 5, 6, 8, 9), out)
    assert list(be.toHost(idx, 4, np.int32)) == [4, 5, 7, 8]
    x = TensorR(inp)
    gradR(lambda d: x.maxPoolBK((2, 2), (1, 1), None))(Tensor.zeros(1))
    eq(T((1, 1, 3, 3), 0, 0, 0, 0, 1, 1, 0, 1, 1), x.d)


def test_avgpool(be):  # T/TestCudnn.scala:838-877; T/TestTensorDifferentiation.scala:1246-1271
    inp = T((1, 1, 3, 3), 1, 2, 3, 4, 5, 6, 7, 8, 9)
    eq(T((1, 1, 2, 2), 3, 4, 6, 7), inp.averagePool2D_batch((2, 2), (1, 1), None))
    x = TensorR(inp)
    gradR(lambda d: x.averagePoolBK((2, 2), (1, 1), None))(Tensor.zeros(1))
    eq(T((1, 1, 3, 3), 0.25, 0.5, 0.25, 0.5, 1, 0.5, 0.25, 0.5, 0.25), x.d)
    y = TensorR(Tensor.ones(1, 1, 4, 4))
    gradR_loss(lambda d: y.averagePoolBK((2, 2), (2, 2), None).sum())(Tensor.zeros(1))
    eq(Tensor.fill((1, 1, 4, 4), 0.25), y.d)
    y.clear_grad()
    gradR_loss(lambda d: y.averagePoolBK((2, 2), (1, 1), None).sum())(Tensor.zeros(1))
    eq(T((1, 1, 4, 4), 0.25, 0.5, 0.5, 0.25, 0.5, 1, 1, 0.5, 0.5, 1, 1, 0.5, 0.25, 0.5, 0.5, 0.25), y.d)


def test_dropout_p0(be):  # T/TestTensorDifferentiation.scala:1042-1092; T/TestCudnn.scala:879-915
    Tensor.randseed(3)
    inp = Tensor.rand(2, 16, 20)
    res, mask = inp.dropout(0.0)
    eq(inp, res)
    assert (be.toHost(mask, inp.scalarCount) == 1.0).all()
    x = TensorR(inp)
    gradR_loss(lambda d: x.dropout(0.0).sum())(Tensor.zeros(1))
    eq(Tensor.ones(2, 16, 20), x.d)


def test_conv_forward(be):  # T/TestTensorDifferentiation.scala:1096-1115; T/TestCudnn.scala:641-661
    inp = T((1, 1, 4, 4), 1, 2, 3, 4, 5, 6, 7, 8, 1, 2, 3, 4, 5, 6, 7, 8)
    ker = T((1, 1, 2, 2), 1, 2, 3, 4)
    out, _ = inp.conv2D_batch(ker, Tensor.zeros(1), (2, 2), (0, 0, 0, 0))
    eq(T((1, 1, 2, 2), 44, 64, 44, 64), out)
    out, _ = inp.conv2D_batch(ker, Tensor.ones(1), (2, 2), (0, 0, 0, 0))
    eq(T((1, 1, 2, 2), 45, 65, 45, 65), out)


def test_conv_pad(be):  # T/TestTensorDifferentiation.scala:1117-1176
    ones, ker = Tensor.ones(1, 1, 4, 4), Tensor.ones(1, 1, 3, 3)
    out, _ = ones.conv2D_batch(ker, Tensor.zeros(1), (3, 3), (1, 1, 1, 1))
    eq(Tensor.fill((1, 1, 2, 2), 4.0), out)
    inp = T((1, 1, 4, 4), 1, 2, 3, 4, 5, 6, 7, 8, 2, 3, 4, 5, 6, 7, 8, 9)
    out, _ = inp.conv2D_batch(ker, Tensor.zeros(1), (3, 3), (1, 1, 1, 1))
    eq(T((1, 1, 2, 2), 14, 22, 18, 26), out)
    out, _ = ones.conv2D_batch(ker, None, (3, 3), (1, 1, 1, 1))
    eq(Tensor.fill((1, 1, 2, 2), 4.0), out)


def test_conv_backprop(be):  # T/TestTensorDifferentiation.scala:1178-1206
    inp, ker, bias = TensorR(Tensor.ones(1, 1, 3, 3)), TensorR(Tensor.ones(1, 1, 2, 2)), TensorR(Tensor.zeros(1))
    gradR_loss(lambda x: inp.convBBP(ker, bias, (1, 1), (0, 0, 0, 0)).sum())(Tensor.zeros(1))
    eq(T((1, 1, 3, 3), 1, 2, 1, 2, 4, 2, 1, 2, 1), inp.d)
    eq(Tensor.fill((1, 1, 2, 2), 4.0), ker.d)
    eq(T((1,), 4.0), bias.d)


def test_conv_backprop_pad(be):  # T/TestTensorDifferentiation.scala:1208-1244
    inp, ker, bias = TensorR(Tensor.ones(1, 1, 4, 4)), TensorR(Tensor.ones(1, 1, 3, 3)), TensorR(Tensor.zeros(1))
    gradR_loss(lambda x: inp.convBBP(ker, bias, (3, 3), (1, 1, 1, 1)).sum())(Tensor.zeros(1))
    eq(Tensor.ones(1, 1, 4, 4), inp.d)
    eq(T((1, 1, 3, 3), 1, 2, 1, 2, 4, 2, 1, 2, 1), ker.d)
    eq(T((1,), 4.0), bias.d)


def test_conv_backprop_gradR(be):  # T/TestCudnn.scala:663-694 (4x4 * 3x3 pad 1, output grad seeded to 1)
    inp, ker, bias = TensorR(Tensor.ones(1, 1, 4, 4)), TensorR(Tensor.ones(1, 1, 3, 3)), TensorR(Tensor.zeros(1))
    gradR(lambda x: inp.convBBP(ker, bias, (1, 1), (0, 0, 0, 0)))(Tensor.zeros(1))
    eq(T((1, 1, 4, 4), 1, 2, 2, 1, 2, 4, 4, 2, 2, 4, 4, 2, 1, 2, 2, 1), inp.d)
    eq(Tensor.fill((1, 1, 3, 3), 4.0), ker.d)
    eq(T((1,), 4.0), bias.d)


def test_sum_on_any_dimension(be):  # T/TestTensorDifferentiation.scala:1273-1305
    a = Tensor.ones(3, 4, 5)
    eq(Tensor.fill((4, 5), 3.0), a.sum(0)); eq(Tensor.fill((3, 5), 4.0), a.sum(1)); eq(Tensor.fill((3, 4), 5.0), a.sum(2))
    r = TensorR(a)
    for k, dim in enumerate((0, 1, 2)):
        gradR_loss(lambda d: r.sum(dim).sum())(Tensor.zeros(1))
        eq(Tensor.fill((3, 4, 5), float(k + 1)), r.d)
    b = Tensor.ones(2, 4, 5, 5)
    eq(b.sum(3).sum(2).sum(0).resize(4, 1, 1), b.batchNormAv() * 2 * 5 * 5)
    i5, i6 = TensorR(T((2,), 2.0, 3.0)), TensorR(T((2,), 2.0, 3.0))
    gradR_loss(lambda d: (i5 * i5).sum())(Tensor.zeros(1))
    gradR_loss(lambda d: i6.square().sum())(Tensor.zeros(1))
    eq(i5.d, i6.d)


def test_sum_dim_with_relu_grad(be):  # T/TestCudnn.scala:621-639
    inp = T((2, 3, 2), -1, 2, -3, 4, -5, 6, -7, 8, -9, 10, -11, 12)
    eq(T((2, 2), -9, 12, -27, 30), inp.sum(1))
    eq(T((2, 3, 2), 0, 1, 0, 1, 0, 1, 0, 1, 0, 1, 0, 1), gradR(lambda x: x.sum(1).relu(False))(inp))


def test_sum_all(be):  # T/TestCudnn.scala:1012-1030
    inp = T((1, 1, 2, 3), 1, 2, 3, 4, 5, 6)
    eq(Tensor.scalar(21), inp.sum())
    eq(Tensor.ones(1, 1, 2, 3), gradR(lambda x: x.sum())(inp))


BCAST = [  # T/TestBroadcast.scala:51-148 (add_broadcast1..5): (dims1, vals1, dims2, vals2, result, d2)
    ((2, 3), [1, 2, 3, 4, 5, 6], (2, 3), [6, 5, 4, 3, 2, 1], [7] * 6, [1] * 6),
    ((2, 3), [1, 2, 3, 4, 5, 6], (2, 1), [1, 2], [2, 3, 4, 6, 7, 8], [3, 3]),
    ((2, 3), [1, 2, 3, 4, 5, 6], (1, 3), [3, 4, 5], [4, 6, 8, 7, 9, 11], [2, 2, 2]),
    ((2, 2, 2), [1, 2, 3, 4, 5, 6, 7, 8], (2,), [1, 2], [2, 4, 4, 6, 6, 8, 8, 10], [4, 4]),
    ((2, 2, 2), [1, 2, 3, 4, 5, 6, 7, 8], (2, 1, 2), [1, 2, 3, 4], [2, 4, 4, 6, 8, 10, 10, 12], [2, 2, 2, 2]),
]


@pytest.mark.parametrize("case", range(len(BCAST)))
def test_add_broadcast(be, case):
    d1, v1, d2, v2, res, g2 = BCAST[case]
    t1, t2 = T(d1, *v1), T(d2, *v2)
    eq(T(d1, *res), t1 + t2); eq(T(d1, *res), t2 + t1)
    a, b = TensorR(t1), TensorR(t2)
    gradR_loss(lambda d: (a + b).sum())(Tensor.zeros(1))
    eq(Tensor.ones(*d1), a.d); eq(T(d2, *g2), b.d)


def test_minus_mult_div_broadcast(be):  # T/TestBroadcast.scala:150-225
    v1 = [1, 2, 3, 4, 5, 6, 7, 8]
    def run(op, v2, res, g1, g2):
        t1, t2 = T((2, 2, 2), *v1), T((2, 1, 2), *v2)
        eq(T((2, 2, 2), *res), op(t1, t2))
        a, b = TensorR(t1), TensorR(t2)
        gradR_loss(lambda d: op(a, b).sum())(Tensor.zeros(1))
        eq(T((2, 2, 2), *g1), a.d); eq(T((2, 1, 2), *g2), b.d)
    run(lambda x, y: x - y, [1, 2, 3, 4], [0, 0, 2, 2, 2, 2, 4, 4], [1] * 8, [-2] * 4)
    run(lambda x, y: x * y, [1, 2, 3, 4], [1, 4, 3, 8, 15, 24, 21, 32], [1, 2, 1, 2, 3, 4, 3, 4], [4, 6, 12, 14])
    run(lambda x, y: x / y, [1, 2, 2, 4], [1, 1, 3, 2, 2.5, 1.5, 3.5, 2], [1, .5, 1, .5, .5, .25, .5, .25], [-4, -1.5, -3, -0.875])


def test_binary_ops_tensor_scalar(be):  # T/TestCublas.scala:228-246
    x = T((3, 1, 2), 1, 2, 3, 4, 5, 6)
    x += 4; x -= 4; x *= -8; x /= -8
    eq(T((3, 1, 2), 1, 2, 3, 4, 5, 6), x)


def test_unary_ops(be):  # T/TestCublas.scala:248-341; T/TestTensorDifferentiation.scala:1307-1378
    x = Tensor.fill((3, 2, 3, 3), 16)
    eq(Tensor.fill((3, 2, 3, 3), 4.0), x.sqrt())
    eq(Tensor.fill((3, 2, 3, 3), 0.125), gradR(lambda t: t.sqrt())(x))
    x = Tensor.fill((3, 2, 3, 3), 3)
    eq(Tensor.fill((3, 2, 3, 3), 9.0), x.square())
    eq(Tensor.fill((3, 2, 3, 3), 6.0), gradR(lambda t: t.square())(x))
    x = Tensor.fill((2, 3), 0.5)
    eq(Tensor.fill((2, 3), float(np.exp(np.float32(0.5)))), x.exp())
    eq(Tensor.fill((2, 3), float(np.exp(np.float32(0.5)))), gradR(lambda t: t.exp())(x))
    x = Tensor.fill((2, 3), 2.0)
    eq(Tensor.fill((2, 3), float(np.log(2.0))), x.log())
    eq(Tensor.fill((2, 3), 0.5), gradR(lambda t: t.log())(x))


def test_concat_and_grad(be):  # T/TestCudnn.scala:963-987
    i1 = T((2, 3, 2, 2), 1, 2, 3, 4, 5, 6, 7, 8, 1, 2, 3, 4, 5, 6, 7, 8, 1, 2, 3, 4, 5, 6, 7, 8)
    i2 = T((2, 4, 2, 2), *([3, 4, 5, 6] * 4 + [6, 7, 8, 9] * 4))
    exp = [1, 2, 3, 4, 5, 6, 7, 8, 1, 2, 3, 4] + [3, 4, 5, 6] * 4 + [5, 6, 7, 8, 1, 2, 3, 4, 5, 6, 7, 8] + [6, 7, 8, 9] * 4
    eq(T((2, 7, 2, 2), *exp), i1.concat(1, i2))
    a, b = TensorR(i1), TensorR(i2)
    gradR(lambda x: a.concat(1, b))(Tensor.zeros(1))
    eq(Tensor.ones(2, 3, 2, 2), a.d); eq(Tensor.ones(2, 4, 2, 2), b.d)


def test_concat_big(be):  # T/TestCudnn.scala:989-1010
    i1, i2 = Tensor.ones(100, 3, 32, 32), Tensor.ones(100, 3, 32, 32)
    eq(Tensor.ones(100, 6, 32, 32), i1.concat(1, i2))
    a, b = TensorR(i1), TensorR(i2)
    gradR(lambda x: a.concat(1, b))(Tensor.zeros(1))
    eq(Tensor.ones(100, 3, 32, 32), a.d); eq(Tensor.ones(100, 3, 32, 32), b.d)


def test_permute_2d(be):  # T/TestCudnn.scala:174-191
    x = T((4, 3), -1, 2, -3, -4, 5, 6, -7, 8, -9, -10, 11, -12)
    eq(T((3, 4), -1, -4, -7, -10, 2, 5, 8, 11, -3, 6, -9, -12), x.permute(1, 0))
    eq(T((4, 3), 0, 1, 0, 0, 1, 1, 0, 1, 0, 0, 1, 0), gradR(lambda t: t.permute(1, 0).relu(False))(x))


@pytest.mark.parametrize("dims", [(2, 2, 3), (2, 3, 4, 5)])
def test_permute_all_orders(be, dims):  # T/TestCudnn.scala:193-619: every order of 3-D and 4-D equals an index shuffle
    import itertools
    n = int(np.prod(dims))
    vals = np.arange(n, dtype=np.float32) - n // 2 + 0.5     # no exact zeros: relu grad at 0 differs between the two forms
    x = Tensor.fromNumpy(vals.reshape(dims))
    for perm in itertools.permutations(range(len(dims))):
        np.testing.assert_array_equal(x.permute(*perm).toCPU(), vals.reshape(dims).transpose(perm))
        for inplace in (False, True):
            g = gradR(lambda t: t.permute(*perm).relu(inplace))(x).toCPU()
            np.testing.assert_array_equal(g, (vals.reshape(dims) > 0).astype(np.float32))


def test_batchnorm_inference(be):  # T/TestCudnn.scala:1032-1049
    inp = Tensor.ones(3, 2, 3, 3)
    r = inp.batchNormInference(T((2,), 3, 3), T((2,), 2, 2), T((2,), 3, 3), T((2,), 4, 4))
    eq(Tensor.fill((3, 2, 3, 3), -1.0), r)


def test_batchnorm_training_vector(be):  # T/TestCudnn.scala:1051-1118 (54 outputs + 54 input grads, 5 decimals)
    g = json.load(open(os.path.join(HERE, "golden", "bn_training.json")))
    Tensor.randseed(g["seed"])
    inp = Tensor.rand(*g["shape"])
    scale, bias = TensorR(T((2,), g["scale"], g["scale"])), TensorR(T((2,), g["bias"], g["bias"]))
    rm, rv = Tensor.ones(2), Tensor.ones(2)
    result = Tensor.zeros(*g["shape"])
    def loss(x):
        y = x.batchNorm(scale, bias, rm, rv)
        result.copy_data(y.x)
        return y.relu()
    grad = gradR(loss)(inp)
    eq(T(g["shape"], *g["expected_result"]), result)
    eq(T(g["shape"], *g["expected_grad"]), grad)


def test_mask4d(be):  # T/TestCublas.scala:300-341 semantics: zero x[b,c,d,t] for t >= len[b]
    x = Tensor.ones(2, 2, 2, 4)
    x.mask4D(int_array([1, 3]))
    exp = np.ones((2, 2, 2, 4), np.float32); exp[0, :, :, 1:] = 0; exp[1, :, :, 3:] = 0
    np.testing.assert_array_equal(x.toCPU(), exp)
