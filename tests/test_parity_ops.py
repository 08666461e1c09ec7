"""Every non-convolution operator of the Backend trait, HIP (through the C ABI) against the CPU
oracle on the same seeded inputs, at the shapes the five applications use (ResNet-50, LeNet,
SqueezeNet, TreeLSTM, DeepSpeech2) plus ragged / tiny / empty-ish edge cases.

Bars: bit-exact for integer results (max-pool argmax, dropout mask, nll gather), 1e-4 relative for
floats (tests/util.assert_close), written at each assert."""
import numpy as np
import pytest

import lantern_amd as la
from lantern_amd import backend as B
from lantern_amd._lib import LanternHipError
from tests.util import assert_close

pytestmark = pytest.mark.gpu


class Pair:
    """Runs one snippet on both backends; `up` uploads the same host array to each."""

    def __init__(self, cpu, hip):
        self.bes = (cpu, hip)

    def run(self, fn):
        outs = []
        for be in self.bes:
            la.set_backend(be)
            up = lambda a, be=be: be.fromHost(np.ascontiguousarray(a))
            down = lambda buf, shape, dtype=np.float32, be=be: be.toHost(buf, int(np.prod(shape)), dtype).reshape(shape)
            outs.append(fn(be, up, down))
        return outs


@pytest.fixture
def pair(cpu_backend, on_hip):
    return Pair(cpu_backend, on_hip)


def _random_cases(seed, n, gen):
    """Seeded random geometries appended to the hand-picked tables below: the named cases say which paths the kernels
    take, these look for the ones nobody thought of (the ids in the test report give the geometry)."""
    rng = np.random.RandomState(seed)
    return [gen(rng) for _ in range(n)]


def _ri(rng, lo, hi): return int(rng.randint(lo, hi + 1))
def _pick(rng, xs): return xs[int(rng.randint(len(xs)))]


def _gen_pool(rng):
    kH, kW = _ri(rng, 2, 5), _ri(rng, 2, 5)
    if rng.rand() < 0.6: kW = kH
    pad = _ri(rng, 0, min(kH, kW) // 2)
    return (_ri(rng, 1, 4), _ri(rng, 1, 9), _ri(rng, kH, 40), _ri(rng, kW, 40), kH, kW, _ri(rng, 1, 3), _ri(rng, 1, 3), pad)


def _gen_perm(rng):
    rank = _ri(rng, 2, 4)
    return (tuple(_ri(rng, 1, 9) for _ in range(rank)), tuple(int(v) for v in rng.permutation(rank)))


def check_all(outs, rtol=1e-4, exact=(), elementwise=False):
    """elementwise: every element within rtol of its own magnitude (operators that move or combine single elements: no sum whose terms
    cancel, so the scale of an error is the element itself), instead of the magnitude plus the output's rms; True or the indices
    of such outputs."""
    want, got = outs
    assert len(want) == len(got)
    for i, (w, g) in enumerate(zip(want, got)):
        if i in exact or w.dtype.kind in "iu":
            np.testing.assert_array_equal(g, w, err_msg="output %d" % i)
        elif elementwise is True or (elementwise and i in elementwise):
            np.testing.assert_allclose(g, w, rtol=rtol, atol=1e-30, err_msg="output %d" % i)
        else:
            assert_close(g, w, rtol=rtol, what="output %d" % i)


# ---- batch norm --------------------------------------------------------------------------------------
BN_SHAPES = [(64, 64, 56 * 56), (8, 256, 56 * 56), (16, 128, 112 * 112),      # the third: x and dy beyond the last-level cache, walked from the end
             (16, 512, 28 * 28), (32, 2048, 49), (4, 24, 7), (3, 5, 1), (1, 16, 100), (20, 33, 1), (64, 1024, 1)]
BN_SHAPES += _random_cases(101, 10, lambda r: (_ri(r, 2, 20), _ri(r, 1, 70), _pick(r, [1, 2, 7, 49, 100, 196, 333, 1023])))


@pytest.mark.parametrize("shape", BN_SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("relu", [False, True], ids=["plain", "relu"])
def test_batchnorm_training_and_grad(pair, shape, relu):
    N, Cc, HW = shape
    rng = np.random.RandomState(11)
    x = (rng.randn(N, Cc, HW) * 1.7 + rng.randn(1, Cc, 1) * 3).astype(np.float32)   # per-channel offsets: tests the shifted sums
    g = (rng.rand(Cc) + 0.5).astype(np.float32); b = rng.randn(Cc).astype(np.float32)
    dy = rng.randn(N, Cc, HW).astype(np.float32)
    dx0 = rng.randn(N, Cc, HW).astype(np.float32)
    if N * HW == 1:
        pytest.skip("variance of one sample is undefined")

    def f(be, up, down):
        X, G, Bi, rm, rv = up(x), up(g), up(b), up(np.zeros(Cc, np.float32)), up(np.ones(Cc, np.float32))
        y, sm, si = be.mallocArray(x.size), be.mallocArray(Cc), be.mallocArray(Cc)
        be.batchNormTraining_into(X, G, Bi, rm, rv, y, sm, si, N, Cc, HW, relu)
        outs = [down(y, x.shape), down(sm, (Cc,)), down(si, (Cc,)), down(rm, (Cc,)), down(rv, (Cc,))]
        DY = up(dy); dg, db = be.mallocArray(Cc), be.mallocArray(Cc)
        if relu:
            xd = up(dx0)
            if be.name == "hip":
                be.batchNorm_grad(X, xd, DY, G, dg, db, sm, si, N, Cc, HW, beta_dx=1.0, y_relu=y, bias=Bi)      # mask rebuilt from x
                xd1 = up(dx0); dg1, db1 = be.mallocArray(Cc), be.mallocArray(Cc)
                be.batchNorm_grad(X, xd1, up(dy), G, dg1, db1, sm, si, N, Cc, HW, beta_dx=1.0, y_relu=y)             # mask read from y
                for a, b_ in ((xd, xd1), (dg, dg1), (db, db1)):
                    np.testing.assert_array_equal(be.toHost(a, a.n), be.toHost(b_, b_.n), err_msg="relu mask from x differs from the stored y")
            else:
                _cpu_bn_relu_grad(be, X, xd, DY, y, G, dg, db, sm, si, N, Cc, HW)
        else:
            xd = up(dx0)
            be.batchNorm_grad(X, xd, DY, G, dg, db, sm, si, N, Cc, HW)
        outs += [down(xd, x.shape), down(dg, (Cc,)), down(db, (Cc,))]
        # beta 0 into garbage must equal (accumulated - initial)
        if be.name == "hip":
            xd2 = up(np.full(x.size, 9.0, np.float32)); dg2, db2 = be.mallocArray(Cc), be.mallocArray(Cc)
            be.batchNorm_grad(X, xd2, up(dy), G, dg2, db2, sm, si, N, Cc, HW, beta_dx=0.0, y_relu=y if relu else None)
            assert_close(down(xd2, x.shape) + dx0.reshape(x.shape), outs[5], rtol=2e-4, what="beta 0 vs beta 1")
        return outs

    outs = pair.run(f)
    if relu:   # elements of y within rounding of zero may land on either side of the mask; compare away from them
        x64 = x.astype(np.float64); mu = x64.mean((0, 2), keepdims=True); var = x64.var((0, 2), keepdims=True)
        pre = (x64 - mu) / np.sqrt(var + 1e-5) * g.reshape(1, Cc, 1) + b.reshape(1, Cc, 1)
        edge = np.abs(pre) < 2e-5
        assert edge.mean() < 1e-3 or N * Cc * HW < 5000
        for o in outs:
            o[0][edge & (np.abs(o[0]) < 2e-5)] = 0.0
            o[5][edge] = dx0.reshape(x.shape)[edge]
    check_all(outs, rtol=2e-4 if relu else 1e-4)


def _cpu_bn_relu_grad(be, X, xd, DY, y, G, dg, db, sm, si, N, Cc, HW):
    be.unary_grad(B.RELU, y, y, DY, DY, N * Cc * HW, inPlace=True)
    be.batchNorm_grad(X, xd, DY, G, dg, db, sm, si, N, Cc, HW)


def test_batchnorm_inference(pair):
    N, Cc, HW = 4, 70, 81
    rng = np.random.RandomState(12)
    x = rng.randn(N, Cc, HW).astype(np.float32); g = rng.rand(Cc).astype(np.float32) + .5; b = rng.randn(Cc).astype(np.float32)
    rm = rng.randn(Cc).astype(np.float32); rv = rng.rand(Cc).astype(np.float32) + .1
    check_all(pair.run(lambda be, up, down: [down(be.batchNormInference(up(x), up(g), up(b), up(rm), up(rv), N, Cc, HW), x.shape)]))


# ---- pooling -----------------------------------------------------------------------------------------
POOLS = [(64, 64, 112, 112, 3, 3, 2, 2, 1),     # ResNet stem
         (8, 6, 24, 24, 2, 2, 2, 2, 0),          # LeNet
         (4, 96, 15, 15, 3, 3, 2, 2, 0),         # SqueezeNet (overlapping windows, no pad)
         (2, 3, 9, 7, 3, 2, 2, 1, 1), (1, 1, 2, 2, 2, 2, 2, 2, 0), (3, 5, 7, 7, 7, 7, 1, 1, 0),
         (2, 3, 10, 10, 2, 2, 3, 3, 0),          # stride above the window: pixels no window covers
         (2, 4, 9, 9, 3, 3, 1, 1, 1),            # 3x3 stride 1: three windows per direction over a pixel
         (1, 2, 11, 11, 5, 5, 2, 2, 2),          # 5x5 stride 2
         (2, 2, 70, 70, 3, 3, 2, 2, 1),          # rows wider than a wavefront
         (2, 3, 8, 12, 3, 3, 2, 2, 1), (1, 2, 6, 4, 3, 3, 2, 2, 1), (3, 5, 30, 36, 3, 3, 2, 2, 1)]      # 3x3/2 pad 1 on even maps: the paired-output kernels (as the ResNet stem)


POOLS += _random_cases(102, 16, _gen_pool)


@pytest.mark.parametrize("p", POOLS, ids=lambda s: "x".join(map(str, s)))
def test_maxpool_values_argmax_and_grad(pair, p):
    N, Cc, H, W, kH, kW, sH, sW, pad = p
    P, Q = B.conv_size(H, kH, sH, pad), B.conv_size(W, kW, sW, pad)
    rng = np.random.RandomState(13)
    x = rng.randint(-6, 7, size=(N, Cc, H, W)).astype(np.float32)      # many ties: first maximum in scan order must win
    dy = rng.randn(N, Cc, P, Q).astype(np.float32)

    def f(be, up, down):
        y, idx = be.maxPool2D_batch(up(x), N, Cc, H, W, kH, kW, sH, sW, pad)
        xd = up(np.ones(x.size, np.float32))
        be.maxPool2D_batch_grad(xd, up(dy), idx, N * Cc * P * Q)
        geom = (N, Cc, H, W, kH, kW, sH, sW, pad)
        xg = up(np.ones(x.size, np.float32)); be.maxPool2D_batch_grad(xg, up(dy), idx, N * Cc * P * Q, geom, 1.0)      # gather form, accumulate
        xo = up(np.full(x.size, 7.0, np.float32)); be.maxPool2D_batch_grad(xo, up(dy), idx, N * Cc * P * Q, geom, 0.0)  # gather form, overwrite
        return [down(y, dy.shape), down(idx, dy.shape, np.int32), down(xd, x.shape), down(xg, x.shape), down(xo, x.shape) + (7.0 if be.name == "hip" else 0.0)]

    outs = pair.run(f)
    check_all(outs, exact=(0, 1), rtol=1e-5)     # values and indices bit-exact; overlapping windows sum in any order


@pytest.mark.parametrize("p", [(64, 2048, 7, 7, 7, 7, 1, 1), (4, 10, 13, 13, 13, 13, 1, 1), (2, 3, 8, 6, 2, 3, 2, 3), (2, 3, 9, 9, 3, 3, 2, 2)]
                         + [c[:8] for c in _random_cases(103, 8, _gen_pool)], ids=lambda s: "x".join(map(str, s)))
def test_avgpool_and_grad(pair, p):
    N, Cc, H, W, kH, kW, sH, sW = p
    P, Q = B.conv_size(H, kH, sH), B.conv_size(W, kW, sW)
    rng = np.random.RandomState(14)
    x = rng.randn(N, Cc, H, W).astype(np.float32); dy = rng.randn(N, Cc, P, Q).astype(np.float32)

    def f(be, up, down):
        y = be.averagePool2D_batch(up(x), N, Cc, H, W, kH, kW, sH, sW)
        xd = up(np.ones(x.size, np.float32))
        be.averagePool2D_batch_grad(xd, up(dy), N, Cc, H, W, kH, kW, sH, sW)
        return [down(y, dy.shape), down(xd, x.shape)]

    check_all(pair.run(f))


def _gen_avgpad(r):
    kH, kW = _ri(r, 1, 5), _ri(r, 1, 5)
    pH, pW = _ri(r, 0, kH - 1), _ri(r, 0, kW - 1)
    if pH == 0 and pW == 0: pH = kH - 1 if kH > 1 else 0; pW = 0 if pH else max(kW - 1, 0)
    H, W = _ri(r, max(1, kH - 2 * pH), 20), _ri(r, max(1, kW - 2 * pW), 20)
    return (_ri(r, 1, 4), _ri(r, 1, 9), H, W, kH, kW, _ri(r, 1, 3), _ri(r, 1, 3), pH, pW)


@pytest.mark.parametrize("p", [(2, 3, 8, 8, 3, 3, 1, 1, 1, 1), (4, 16, 7, 7, 3, 3, 2, 2, 1, 1), (1, 2, 5, 9, 2, 4, 2, 3, 1, 2), (2, 2, 13, 13, 3, 3, 2, 2, 0, 1),
                               (1, 1, 1, 1, 3, 3, 1, 1, 2, 2), (8, 64, 28, 28, 3, 3, 1, 1, 1, 1)]
                         + [c for c in _random_cases(109, 8, _gen_avgpad) if c[8] or c[9]], ids=lambda s: "x".join(map(str, s)))
def test_avgpool_with_padding_and_grad(pair, p):
    """averagePool2D_batch with pads (CDN:975-982, divisor = elements inside the image): values and the accumulated input gradient."""
    N, Cc, H, W, kH, kW, sH, sW, pH, pW = p
    P, Q = B.conv_size(H, kH, sH, pH), B.conv_size(W, kW, sW, pW)
    rng = np.random.RandomState(16)
    x = rng.randn(N, Cc, H, W).astype(np.float32); dy = rng.randn(N, Cc, P, Q).astype(np.float32)

    def f(be, up, down):
        y = be.averagePool2D_batch(up(x), N, Cc, H, W, kH, kW, sH, sW, pH, pW)
        xd = up(np.ones(x.size, np.float32))
        be.averagePool2D_batch_grad(xd, up(dy), N, Cc, H, W, kH, kW, sH, sW, pH, pW)
        return [down(y, dy.shape), down(xd, x.shape)]

    check_all(pair.run(f))


def test_avgpool_with_padding_through_the_tape(be):
    """TensorR.averagePoolBK with ONNX-ordered pads: a constant image averages to itself whatever the padding, and the
    gradient of the sum of outputs is the number-weighted coverage of each pixel (every pixel's shares add up to the
    number of outputs when summed over the image)."""
    from lantern_amd.tensor import Tensor, TensorR, gradR
    x = Tensor.fromNumpy(np.full((2, 3, 6, 5), 2.5, np.float32))
    g = gradR(lambda t: t.averagePoolBK((3, 3), (2, 2), (1, 1, 1, 1)).sum())(x)
    y = x.averagePool2D_batch((3, 3), (2, 2), (1, 1, 1, 1))
    assert y.shape == (2, 3, 3, 3) and np.allclose(y.toCPU(), 2.5)
    gx = g.toCPU().reshape(2, 3, 6, 5)
    assert np.allclose(gx.sum(axis=(2, 3)), 9.0, rtol=1e-5)
    with pytest.raises(AssertionError):
        x.averagePool2D_batch((3, 3), (2, 2), (1, 0, 1, 1))


# ---- element-wise, broadcast, layout -----------------------------------------------------------------
@pytest.mark.parametrize("n", [1, 3, 64, 1000, 64 * 256 * 56 * 56 // 16 + 5])
def test_unary_ops_and_grads(pair, n):
    rng = np.random.RandomState(15)
    x = (rng.randn(n) * 1.5).astype(np.float32)
    x[np.abs(x) < 1e-3] = 0.5                                   # keep relu / hardTanh away from their kinks
    xp = np.abs(x) + 0.1
    dy = rng.randn(n).astype(np.float32)

    def f(be, up, down):
        outs = []
        for op, src in ((B.RELU, x), (B.TANH, x), (B.SIGMOID, x), (B.EXP, x), (B.LOG, xp), (B.SQRT, xp), (B.SQUARE, x), (B.HARDTANH, x)):
            X = up(src); y = be.unary(op, X, n, lo=-0.8, hi=0.9)
            dx = up(np.full(n, 0.25, np.float32))
            be.unary_grad(op, X, y, up(dy), dx, n, lo=-0.8, hi=0.9)
            outs += [down(y, (n,)), down(dx, (n,))]
        X = up(x); be.unary(B.RELU, X, n, inPlace=True); outs.append(down(X, (n,)))
        return outs

    check_all(pair.run(f), rtol=2e-4)


BCAST = [((64, 256, 7, 7), (64, 256, 7, 7)), ((8, 16, 5, 5), (1, 16, 1, 1)), ((8, 16, 5, 5), (1,)), ((1, 16, 1, 1), (8, 16, 5, 5)),
         ((100, 150), (150,)), ((100, 1), (1, 150)), ((5,), (5,)), ((3, 1, 4), (1, 6, 1)), ((20, 10), (20, 1)), ((1,), (1,))]


@pytest.mark.parametrize("shapes", BCAST, ids=lambda s: "%s_%s" % ("x".join(map(str, s[0])), "x".join(map(str, s[1]))))
def test_broadcast_ops_grads_and_updates(pair, shapes):
    sa, sb = shapes
    A, Bs, O = B.dim_broadcast(sa, sb)
    rng = np.random.RandomState(16)
    a = rng.randn(*sa).astype(np.float32); b = (rng.rand(*sb) + 0.5).astype(np.float32) * np.where(rng.rand(*sb) < .5, -1, 1).astype(np.float32)
    od = rng.randn(*O).astype(np.float32)

    def f(be, up, down):
        outs = []
        for op in (B.ADD, B.SUB, B.MUL, B.DIV):
            Ab, Bb = up(a), up(b)
            outs.append(down(be.bcast_op(op, Ab, A, Bb, Bs, O), O))
            ad, bd = up(np.ones(a.size, np.float32)), up(np.ones(b.size, np.float32))
            be.bcast_op_grad(op, Ab, ad, A, False, Bb, bd, Bs, False, up(od), O)
            outs += [down(ad, sa), down(bd, sb)]
            if tuple(A) == tuple(O):                          # in-place update needs the left side to have the result shape
                be.bcast_update(op, Ab, A, Bb, Bs); outs.append(down(Ab, sa))
        return outs

    check_all(pair.run(f), rtol=2e-4)


def test_scalar_ops_geam_fill_clip(pair):
    n = 70001
    rng = np.random.RandomState(17)
    x = rng.randn(n).astype(np.float32); y = rng.randn(n).astype(np.float32)
    bias = rng.randn(12).astype(np.float32)

    def f(be, up, down):
        outs = [down(be.scalar_op(op, up(x), 1.7, n), (n,)) for op in (B.ADD, B.SUB, B.MUL, B.DIV)]
        o = be.mallocArray(n); be.geam(up(x), 0.3, up(y), -2.0, o, n); outs.append(down(o, (n,)))
        X = up(x); be.geam(X, 1.0, up(y), 1.0, X, n); outs.append(down(X, (n,)))           # aliasing output with an input
        X = up(x); be.fillInPlace(X, n, 2.5); outs.append(down(X, (n,)))
        X = up(x); be.clipAt(X, n, 0.5); outs.append(down(X, (n,)))
        outs.append(down(be.fillWithBias((3, 12, 5, 7), up(bias), 1), (3, 12, 5, 7)))
        outs.append(down(be.fillWithBias((4, 12), up(bias), 1), (4, 12)))
        return outs

    check_all(pair.run(f), rtol=1e-6, elementwise=(0, 1, 2, 3, 6, 7, 8, 9))      # 4 and 5 (geam) add two products that may cancel


@pytest.mark.parametrize("rc", [(1, 1), (3, 5), (64, 64), (100, 257), (2048, 1000), (1, 300)])
def test_transpose_and_grad(pair, rc):
    r, c = rc
    rng = np.random.RandomState(18); x = rng.randn(r, c).astype(np.float32); yd = rng.randn(c, r).astype(np.float32)

    def f(be, up, down):
        y = be.trans(up(x), r, c); xd = up(np.ones(r * c, np.float32)); be.trans_grad(xd, up(yd), r, c)
        return [down(y, (c, r)), down(xd, (r, c))]

    outs = pair.run(f)
    np.testing.assert_array_equal(outs[1][0], x.T)
    check_all(outs, rtol=1e-6, elementwise=True)


@pytest.mark.parametrize("case", [((4, 6, 5), (2, 0, 1)), ((3, 32, 21, 50), (3, 0, 1, 2)), ((2, 3, 4, 5), (0, 2, 3, 1)), ((7, 9), (1, 0)), ((2, 3, 4, 5), (3, 2, 1, 0)),
                                  ((8, 32, 11, 40), (2, 0, 1, 3))] + _random_cases(104, 8, _gen_perm), ids=str)
def test_permute_and_grad(pair, case):
    dims, perm = case
    rng = np.random.RandomState(19); x = rng.randn(*dims).astype(np.float32)
    odims = tuple(dims[p] for p in perm); yd = rng.randn(*odims).astype(np.float32)

    def f(be, up, down):
        y = be.permute(up(x), dims, perm); xd = up(np.ones(x.size, np.float32)); be.permute_grad(xd, up(yd), dims, perm)
        return [down(y, odims), down(xd, dims)]

    outs = pair.run(f)
    np.testing.assert_array_equal(outs[1][0], np.transpose(x, perm))
    check_all(outs, rtol=1e-6, elementwise=True)


def test_concat_and_grad(pair):
    rng = np.random.RandomState(20)
    for outer, sizes, inner in [(4, (64, 64), 13 * 13), (2, (3, 5, 1), 7), (1, (10,), 1), (3, (2, 2), 1), (5, (128, 128), 1)]:
        xs = [rng.randn(outer, s, inner).astype(np.float32) for s in sizes]
        od = rng.randn(outer, sum(sizes), inner).astype(np.float32)

        def f(be, up, down):
            y = be.concat([up(x) for x in xs], list(sizes), outer, inner)
            ds = [up(np.ones(x.size, np.float32)) for x in xs]
            be.concat_grad(ds, list(sizes), up(od), outer, inner)
            outs = [down(y, od.shape)] + [down(d, x.shape) for d, x in zip(ds, xs)]
            if be.name == "hip":      # overwrite form: first input into garbage with beta 0, the others accumulate
                ds2 = [up(np.full(x.size, 9.0 if t == 0 else 1.0, np.float32)) for t, x in enumerate(xs)]
                be.concat_grad(ds2, list(sizes), up(od), outer, inner, [0.0] + [1.0] * (len(xs) - 1))
                np.testing.assert_array_equal(down(ds2[0], xs[0].shape) + 1.0, outs[1])
                for t in range(1, len(xs)):
                    np.testing.assert_array_equal(down(ds2[t], xs[t].shape), outs[1 + t])
            return outs

        outs = pair.run(f)
        np.testing.assert_array_equal(outs[1][0], np.concatenate(xs, 1))
        check_all(outs, rtol=1e-6)


# ---- reductions, softmax, loss -----------------------------------------------------------------------
@pytest.mark.parametrize("n", [1, 7, 4096, 1000003])
def test_sum_mean_and_grads(pair, n):
    rng = np.random.RandomState(21); x = (rng.randn(n) + 0.3).astype(np.float32)

    def f(be, up, down):
        X = up(x); s, m = be.sum(X, n), be.mean(X, n)
        dx = up(np.ones(n, np.float32)); be.add_scalar_from(dx, up(np.array([2.5], np.float32)), 1.0 / n, n)
        return [down(s, (1,)), down(m, (1,)), down(dx, (n,))]

    outs = pair.run(f)
    assert abs(outs[1][0][0] - x.astype(np.float64).sum()) <= 1e-4 * (np.abs(x).sum())   # device sum against the exact one
    check_all(outs, rtol=2e-4)


@pytest.mark.parametrize("oci", [(64, 49, 1), (1, 5, 1), (8, 3, 20), (100, 1, 7), (3, 1000, 1), (2, 64, 3000), (1, 2000, 300), (3, 700, 100), (1, 5920, 1600)]
                         + _random_cases(105, 8, lambda r: (_ri(r, 1, 9), _ri(r, 1, 300), _ri(r, 1, 50))))
def test_sum_dim_and_grad(pair, oci):
    o, d, i = oci
    rng = np.random.RandomState(22); x = rng.randn(o, d, i).astype(np.float32); dy = rng.randn(o, i).astype(np.float32)

    def f(be, up, down):
        y = be.sum_dim(up(x), o, d, i); dx = up(np.ones(x.size, np.float32)); be.sum_dim_grad(dx, up(dy), o, d, i)
        return [down(y, (o, i)), down(dx, x.shape)]

    check_all(pair.run(f))


@pytest.mark.parametrize("oci", [(64, 1000, 1), (100, 10, 1), (1, 1, 1), (5, 29, 1), (3, 29, 150), (7, 5000, 1), (2, 3, 1)]
                         + _random_cases(106, 6, lambda r: (_ri(r, 1, 40), _ri(r, 1, 600), _pick(r, [1, 1, 1, 7, 33]))))
@pytest.mark.parametrize("is_log", [0, 1], ids=["softmax", "logsoftmax"])
def test_softmax_and_grad(pair, oci, is_log):
    o, c, i = oci
    rng = np.random.RandomState(23); x = (rng.randn(o, c, i) * 4).astype(np.float32); dy = rng.randn(o, c, i).astype(np.float32)

    def f(be, up, down):
        y = be.softmax(is_log, up(x), o, c, i); dx = up(np.ones(x.size, np.float32))
        be.softmax_grad(is_log, y, up(dy), dx, o, c, i)
        return [down(y, x.shape), down(dx, x.shape)]

    check_all(pair.run(f), rtol=2e-4)


def test_nll_loss_and_grad(pair):
    rng = np.random.RandomState(24)
    for batch, classes in [(64, 1000), (100, 10), (1, 5), (7, 1)]:
        x = rng.randn(batch, classes).astype(np.float32); t = rng.randint(0, classes, size=batch).astype(np.int32)
        dy = rng.randn(batch).astype(np.float32)

        def f(be, up, down):
            T = up(t); y = be.nllLoss(up(x), T, batch, classes); dx = up(np.ones(x.size, np.float32))
            be.nllLoss_grad(dx, T, up(dy), batch, classes)
            return [down(y, (batch,)), down(dx, x.shape)]

        outs = pair.run(f)
        np.testing.assert_array_equal(outs[1][0], -x[np.arange(batch), t])           # a gather: exact
        check_all(outs, rtol=1e-6)


# ---- dot family --------------------------------------------------------------------------------------
SHAPES_MV = [(150, 300), (5, 150), (1, 1), (1000, 2048), (33, 7), (150, 150), (9, 31), (257, 65), (32, 32)]


def test_dot_family_at_treelstm_and_classifier_shapes(pair):
    rng = np.random.RandomState(25)

    def f(be, up, down):
        outs = []
        for m, n in SHAPES_MV:
            Mx = rng_m[(m, n)]; v = rng_v[n]; w = rng_v2[m]
            outs.append(down(be.matrixVectorDot(up(Mx), up(v), m, n), (m,)))
            outs.append(down(be.vectorVectorDot(up(v), up(v[::-1].copy()), n), (1,)))
            xd = up(np.ones(m * n, np.float32)); be.add_cartesian(xd, up(v), up(w), m, n); outs.append(down(xd, (m, n)))
            vd = up(np.ones(n, np.float32)); be.add_composition(vd, up(Mx), up(w), m, n); outs.append(down(vd, (n,)))
            sd = up(np.ones(n, np.float32)); be.addMul_scalar(sd, up(np.array([0.7], np.float32)), up(v), n); outs.append(down(sd, (n,)))
        for d1, d2, d3 in [(64, 2048, 1000), (100, 320, 50), (3, 4, 5), (20, 1, 7), (1, 33, 1)]:
            X, Y, O = rng_g[(d1, d2)], rng_g[(d2, d3)], rng_g[(d1, d3)]
            outs.append(down(be.matrixMatrixDot(up(X), up(Y), d1, d2, d3), (d1, d3)))
            xd = up(np.ones(d1 * d2, np.float32)); be.add_dotTrans2(xd, up(O), up(Y), d1, d2, d3); outs.append(down(xd, (d1, d2)))
            yd = up(np.ones(d2 * d3, np.float32)); be.add_dotTrans1(yd, up(X), up(O), d1, d2, d3); outs.append(down(yd, (d2, d3)))
        return outs

    rng_m = {s: rng.randn(*s).astype(np.float32) for s in SHAPES_MV}
    rng_v = {n: rng.randn(n).astype(np.float32) for _, n in SHAPES_MV}
    rng_v2 = {m: rng.randn(m).astype(np.float32) for m, _ in SHAPES_MV}
    rng_g = {}
    for d1, d2, d3 in [(64, 2048, 1000), (100, 320, 50), (3, 4, 5), (20, 1, 7), (1, 33, 1)]:
        for s in ((d1, d2), (d2, d3), (d1, d3)):
            rng_g.setdefault(s, rng.randn(*s).astype(np.float32))
    check_all(pair.run(f))


@pytest.mark.parametrize("tx", [False, True])
@pytest.mark.parametrize("ty", [False, True])
def test_gemm_and_grad_all_transposes(pair, tx, ty):
    rng = np.random.RandomState(26)
    for d1, d2, d3 in [(32, 672, 1024), (5, 7, 3), (64, 100, 29)]:
        X = rng.randn(*((d2, d1) if tx else (d1, d2))).astype(np.float32); Y = rng.randn(*((d3, d2) if ty else (d2, d3))).astype(np.float32)
        od = rng.randn(d1, d3).astype(np.float32)

        def f(be, up, down):
            Xb, Yb = up(X), up(Y)
            r = be.gemm(Xb, tx, Yb, ty, 0.5, d1, d2, d3)
            xd, yd = up(np.ones(X.size, np.float32)), up(np.ones(Y.size, np.float32))
            be.gemm_grad(Xb, xd, False, tx, Yb, yd, False, ty, 0.5, up(od), d1, d2, d3)
            return [down(r, (d1, d3)), down(xd, X.shape), down(yd, Y.shape)]

        check_all(pair.run(f))


# ---- dropout, masks ----------------------------------------------------------------------------------
def test_dropout_mask_is_bit_exact_and_scaled(pair):
    n = 100003
    rng = np.random.RandomState(27); x = rng.randn(n).astype(np.float32); dy = rng.randn(n).astype(np.float32)

    def f(be, up, down):
        be.dropout_seed, be.dropout_offset = 1234, 77
        y, mask = be.dropout(up(x), n, 0.3)
        y2, mask2 = be.dropout(up(x), n, 0.3)                  # the stream advances: a different mask
        dx = up(np.ones(n, np.float32)); be.dropout_grad(dx, up(dy), mask, n)
        y0, m0 = be.dropout(up(x), n, 0.0)
        return [down(mask, (n,)), down(y, (n,)), down(mask2, (n,)), down(dx, (n,)), down(m0, (n,)), down(y0, (n,))]

    outs = pair.run(f)
    m = outs[1][0]
    assert abs((m > 0).mean() - 0.7) < 0.01 and not np.array_equal(m, outs[1][2])
    np.testing.assert_array_equal(outs[1][4], np.ones(n, np.float32))
    check_all(outs, exact=(0, 2, 4), rtol=1e-6)
    with pytest.raises(ValueError):
        pair.bes[1].dropout(None, 4, 1.0)


def test_mask4d(pair):
    n, c, d, t = 4, 3, 5, 17
    rng = np.random.RandomState(28); x = rng.randn(n, c, d, t).astype(np.float32); lens = np.array([17, 0, 9, 1], np.int32)

    def f(be, up, down):
        X = up(x); be.mask4D(X, up(lens), n, c, d, t); return [down(X, x.shape)]

    outs = pair.run(f)
    want = x.copy()
    for i, l in enumerate(lens):
        want[i, :, :, l:] = 0
    np.testing.assert_array_equal(outs[1][0], want)
    check_all(outs, exact=(0,))


# ---- optimizers --------------------------------------------------------------------------------------
def test_optimizers_single_and_multi_tensor(pair):
    rng = np.random.RandomState(29)
    sizes = [1, 7, 64, 1000, 9 * 64 * 64, 2048 * 1000 + 3]
    xs = [rng.randn(s).astype(np.float32) for s in sizes]; gs = [(rng.randn(s) * 3).astype(np.float32) for s in sizes]

    def f(be, up, down):
        outs = []
        for nesterov in (False, True):
            X, D, V = up(xs[3]), up(gs[3]), be.mallocArray(sizes[3])
            for _ in range(3):
                be.momentum_update(X, D, V, 0.1, 0.9, 2.0, nesterov, sizes[3]); be.upload(D, gs[3])
            outs += [down(X, (sizes[3],)), down(V, (sizes[3],))]
        X, D, M = up(xs[2]), up(gs[2]), be.mallocArray(sizes[2])
        be.adagrad_update(X, D, M, 0.05, 1.0, sizes[2]); outs += [down(X, (sizes[2],)), down(M, (sizes[2],)), down(D, (sizes[2],))]
        X, D = up(xs[4]), up(gs[4]); be.sgd_update(X, D, 0.01, sizes[4]); outs += [down(X, (sizes[4],)), down(D, (sizes[4],))]
        ps = [(up(x), up(g), be.mallocArray(s), s) for x, g, s in zip(xs, gs, sizes)]
        for _ in range(2):
            be.multi_momentum_update(ps, 0.1, 0.9, 400.0, False)
            for p, g in zip(ps, gs):
                be.copyFloatArray(p[1], up(g), p[3])
        for p in ps:
            outs += [down(p[0], (p[3],)), down(p[2], (p[3],))]
        ps2 = [(up(x), up(g), s) for x, g, s in zip(xs, gs, sizes)]
        be.multi_sgd_update(ps2, 0.05)
        for p in ps2:
            outs += [down(p[0], (p[2],)), down(p[1], (p[2],))]
        return outs

    check_all(pair.run(f), rtol=1e-5)


# ---- fused pairs against their unfused sequences ----------------------------------------------------
def test_add_relu_and_its_gradient(pair):
    n = 64 * 256 * 14 * 14 + 3
    rng = np.random.RandomState(30)
    a = rng.randn(n).astype(np.float32); b = rng.randn(n).astype(np.float32); dy = rng.randn(n).astype(np.float32)
    s = a + b; a[np.abs(s) < 1e-4] += 1.0

    def f(be, up, down):
        o = be.mallocArray(n); be.add_into(up(a), up(b), o, n, True)
        ad = be.mallocArray(n, zero=False) if be.name == "hip" else be.mallocArray(n)
        bd = up(np.ones(n, np.float32))
        if be.name == "hip":
            be.add_relu_grad(o, up(dy), ad, 0.0, bd, 1.0, n)         # first writer overwrites, second accumulates
        else:
            be.add_relu_grad(o, up(dy), ad, 1.0, bd, 1.0, n)
        return [down(o, (n,)), down(ad, (n,)), down(bd, (n,))]

    check_all(pair.run(f), rtol=1e-6, elementwise=True)


@pytest.mark.parametrize("beta", [0.0, 1.0, 0.5])
@pytest.mark.parametrize("tt", [(1, 0), (0, 1), (0, 0), (1, 1)], ids=lambda t: "ta%d_tb%d" % t)
def test_sgemm_few_tiles_long_reduction_with_row_stride(on_hip, tt, beta):
    """Weight-gradient shape: a small output over thousands of rows (the reduction is split over blocks and combined
    with atomic adds onto beta*C); C has a row stride larger than n and the padding must stay untouched."""
    be = on_hip
    ta, tb = tt
    m, n, k, ldc = 200, 136, 3000, 144
    rng = np.random.RandomState(41)
    A = rng.randn(*((k, m) if ta else (m, k))).astype(np.float32); Bm = rng.randn(*((n, k) if tb else (k, n))).astype(np.float32)
    C0 = rng.randn(m, ldc).astype(np.float32)
    a, b, c = be.fromHost(A), be.fromHost(Bm), be.fromHost(C0)
    be.lib.lh_sgemm(ta, tb, m, n, k, 0.75, a.ptr, A.shape[1], b.ptr, Bm.shape[1], beta, c.ptr, ldc)
    from lantern_amd import _lib
    _lib.check()
    got = be.toHost(c, m * ldc).reshape(m, ldc)
    want = 0.75 * ((A.T if ta else A).astype(np.float64) @ (Bm.T if tb else Bm).astype(np.float64)) + beta * C0[:, :n]
    assert_close(got[:, :n], want.astype(np.float32), rtol=1e-4, what="sgemm split")
    np.testing.assert_array_equal(got[:, n:], C0[:, n:])


@pytest.mark.parametrize("beta", [0.0, 1.0, 0.5])
def test_deterministic_mode_sgemm_slices_and_axis_sums(on_hip, beta):
    """lh_set_deterministic(1): a product whose reduction is cut into slices (each into its own scratch block, added in slice
    order onto beta*C), the 10-output classifier shape of the small-product kernel, and a sum over a long middle axis give
    the right values and the same bits on a second call; padding columns of a strided C stay untouched."""
    be = on_hip
    from lantern_amd import _lib
    rng = np.random.RandomState(43)
    be.setDeterministic(True)
    try:
        for (ta, tb, m, n, k, ldc) in ((1, 0, 200, 136, 3000, 144), (0, 1, 64, 10, 2048, 10), (0, 0, 800, 800, 5920, 800)):
            A = rng.randn(*((k, m) if ta else (m, k))).astype(np.float32); Bm = rng.randn(*((n, k) if tb else (k, n))).astype(np.float32)
            C0 = rng.randn(m, ldc).astype(np.float32)
            a, b = be.fromHost(A), be.fromHost(Bm)
            outs = []
            for _ in range(2):
                c = be.fromHost(C0)
                be.lib.lh_sgemm(ta, tb, m, n, k, 0.75, a.ptr, A.shape[1], b.ptr, Bm.shape[1], beta, c.ptr, ldc); _lib.check()
                outs.append(be.toHost(c, m * ldc).reshape(m, ldc))
            want = 0.75 * ((A.T if ta else A).astype(np.float64) @ (Bm.T if tb else Bm).astype(np.float64)) + beta * C0[:, :n]
            assert_close(outs[0][:, :n], want.astype(np.float32), rtol=1e-4, what="deterministic sgemm %dx%dx%d" % (m, n, k))
            np.testing.assert_array_equal(outs[0], outs[1])
            np.testing.assert_array_equal(outs[0][:, n:], C0[:, n:])
        x = rng.randn(2, 5920, 1600).astype(np.float32); xd = be.fromHost(x)
        ys = [be.toHost(be.sum_dim(xd, 2, 5920, 1600), 2 * 1600) for _ in range(2)]
        assert_close(ys[0].reshape(2, 1600), x.astype(np.float64).sum(1).astype(np.float32), rtol=1e-4, what="deterministic sum over the middle axis")
        np.testing.assert_array_equal(ys[0], ys[1])
    finally:
        be.setDeterministic(False)


# ---- arena and error path (the library's own behaviour; no oracle counterpart) -----------------------
def _arena_block(be, n, zero=True):
    """A block straight from the library's arena (BackendHIP.mallocArray cuts small blocks from larger ones itself)."""
    from lantern_amd import _lib
    p = (be.lib.lh_malloc if zero else be.lib.lh_malloc_uninit)(4 * n)
    _lib.check()
    return B.Buf(p, n)


def test_arena_zeroing_alignment_rewind_and_overflow(on_hip):
    be = on_hip
    lib = be.lib
    mark = be.getMallocAddr()
    a = _arena_block(be, 1000)
    assert a.ptr % 256 == 0 and not be.toHost(a, 1000).any()
    be.fillInPlace(a, 1000, 3.0)
    used = lib.lh_heap_used()
    b = _arena_block(be, 10)
    assert b.ptr % 256 == 0 and b.ptr >= a.ptr + 4000 and lib.lh_heap_used() > used
    be.resetMallocAddr(mark)
    c = _arena_block(be, 1000)
    assert c.ptr == a.ptr and not be.toHost(c, 1000).any()        # memory handed out again starts at zero (CUB:22-25 memset on rewind)
    be.resetMallocAddr(mark)
    with pytest.raises(LanternHipError):
        be.mallocArray(be.heap_bytes)                              # 4x the arena: refused, nothing allocated
    assert lib.lh_heap_used() <= used                              # nothing was taken by the refused request
    z = _arena_block(be, 4); assert not be.toHost(z, 4).any()      # the library keeps working after an error
    be.resetMallocAddr(mark)


def test_arena_small_blocks_read_zero_after_dirty_memory_uninit_blocks_and_pops(on_hip):
    """Zero-filled blocks are cleared a window at a time; whatever was written there before (a rewound block, an
    uninitialised block handed out inside the window and popped again) must not show through."""
    be = on_hip
    lib = be.lib
    mark = be.getMallocAddr()
    big = _arena_block(be, 1 << 20, zero=False); be.fillInPlace(big, 1 << 20, 7.0)          # 4 MiB of sevens
    be.resetMallocAddr(mark)
    blocks = [_arena_block(be, n) for n in (3, 150, 45000, 1, 300000, 64, 150)]            # crosses several windows
    for blk, n in zip(blocks, (3, 150, 45000, 1, 300000, 64, 150)):
        assert not be.toHost(blk, n).any()
        be.fillInPlace(blk, n, 5.0)
    top = lib.lh_heap_used()
    s = _arena_block(be, 5000, zero=False); be.fillInPlace(s, 5000, 9.0)                    # scratch inside the cleared window
    lib.lh_free_top(5000 * 4)
    assert lib.lh_heap_used() == top
    z = _arena_block(be, 5000); assert z.ptr == s.ptr and not be.toHost(z, 5000).any()
    u = _arena_block(be, 100, zero=False); be.fillInPlace(u, 100, 2.0)
    z2 = _arena_block(be, 100); assert not be.toHost(z2, 100).any() and (be.toHost(u, 100) == 2.0).all()
    be.resetMallocAddr(mark)


def test_mirror_cuts_small_blocks_from_zeroed_arena_blocks_and_drops_them_at_marks(on_hip):
    """BackendHIP.mallocArray: small blocks come 256-byte aligned out of one 1 MiB arena block, read zero even after the
    memory was dirty, never straddle a mark, and large blocks still come straight from the arena."""
    be = on_hip
    mark = be.getMallocAddr()
    dirty = _arena_block(be, 1 << 19, zero=False); be.fillInPlace(dirty, 1 << 19, 4.0)      # 2 MiB of fours
    be.resetMallocAddr(mark)
    used0 = be.lib.lh_heap_used()
    a = be.mallocArray(150); b = be.mallocArray(1, zero=False); c = be.mallocArray(16000)
    assert be.lib.lh_heap_used() == used0 + be.CHUNK
    assert a.ptr % 256 == 0 and b.ptr == a.ptr + 768 and c.ptr == b.ptr + 256
    for blk, n in ((a, 150), (b, 1), (c, 16000)):
        assert not be.toHost(blk, n).any()
    be.fillInPlace(c, 16000, 1.0)
    m2 = be.getMallocAddr()
    d = be.mallocArray(150)
    assert d.ptr == a.ptr + be.CHUNK and not be.toHost(d, 150).any()                        # a fresh block above the mark
    big = be.mallocArray(1 << 18)
    assert big.ptr == d.ptr + be.CHUNK and not be.toHost(big, 1 << 18).any()
    be.resetMallocAddr(m2)
    e = be.mallocArray(150)
    assert e.ptr == d.ptr and not be.toHost(e, 150).any()
    assert (be.toHost(c, 16000) == 1.0).all()
    be.resetMallocAddr(mark)


def test_shape_errors_are_reported_not_launched(on_hip):
    be = on_hip
    x = be.mallocArray(16)
    for call in (lambda: be.lib.lh_conv2d_fwd(x.ptr, x.ptr, 0, x.ptr, 1, 1, 2, 2, 1, 3, 3, 1, 1, 0, 0),       # kernel larger than the padded input
                 lambda: be.lib.lh_conv2d_fwd(x.ptr, x.ptr, 0, x.ptr, 1, 1, 4, 4, 1, 3, 3, 0, 1, 0, 0),       # stride 0
                 lambda: be.lib.lh_sgemm(0, 0, 4, 4, 4, 1.0, x.ptr, 2, x.ptr, 4, 0.0, x.ptr, 4),              # lda < k
                 lambda: be.lib.lh_unary(99, x.ptr, x.ptr, 16, 0.0, 0.0),                                     # unknown op code
                 lambda: be.lib.lh_permute(x.ptr, x.ptr, B._ints((2, 8)), B._ints((0, 0)), 2),                # not a permutation
                 lambda: be.lib.lh_bcast_op(0, x.ptr, B._ints((2, 8)), x.ptr, B._ints((3, 8)), x.ptr, B._ints((3, 8)), 2),   # 2 against 3 does not broadcast
                 lambda: be.lib.lh_dropout_fwd(x.ptr, x.ptr, x.ptr, 16, 1.0, 1, 0)):                          # rate outside [0, 1)
        call()
        with pytest.raises(LanternHipError):
            from lantern_amd import _lib
            _lib.check()
    be.fillInPlace(x, 16, 1.0)
    assert (be.toHost(x, 16) == 1.0).all()


# ---- recurrent layer and CTC (DeepSpeech2 path) ------------------------------------------------------
@pytest.mark.parametrize("case", [(1, True, 12, 32, 672, 800), (1, True, 6, 8, 96, 1024), (0, False, 5, 3, 7, 37), (1, False, 1, 2, 5, 16), (0, True, 9, 4, 33, 130), (1, True, 4, 5, 20, 300), (0, True, 3, 6, 16, 1100), (1, False, 3, 33, 10, 1030), (1, True, 3, 70, 24, 64)]
                         + _random_cases(107, 6, lambda r: (_ri(r, 0, 1), bool(r.rand() < 0.5), _ri(r, 1, 8), _ri(r, 1, 9), _ri(r, 1, 40), _pick(r, [5, 16, 37, 64, 130, 300]))),
                         ids=lambda c: "mode%d_bi%d_T%d_B%d_I%d_H%d" % c)
def test_rnn_forward_and_backward(pair, case):
    mode, bidir, T, Bn, In, H = case
    D = 2 if bidir else 1
    rng = np.random.RandomState(31)
    per = H * In + H * H + 2 * H
    w = (rng.randn(D * per) * (0.5 / np.sqrt(H))).astype(np.float32)
    x = rng.randn(T, Bn, In).astype(np.float32); dy = rng.randn(T, Bn, D * H).astype(np.float32)
    if mode == 0:
        w[:] = np.abs(w) * np.where(rng.rand(w.size) < 0.3, -1, 1)       # relu: keep most pre-activations away from the kink

    def f(be, up, down):
        X, W = up(x), up(w)
        y = be.rnn_forward(mode, X, W, T, Bn, In, H, bidir)
        dx = up(np.ones(x.size, np.float32)); dw = up(np.ones(w.size, np.float32))
        be.rnn_backward(mode, X, y, up(dy), W, dx, dw, T, Bn, In, H, bidir, 1.0)
        outs = [down(y, dy.shape), down(dx, x.shape), down(dw, w.shape)]
        if be.name == "hip":
            dx0 = up(np.full(x.size, 5.0, np.float32)); dw0 = up(np.zeros(w.size, np.float32))
            be.rnn_backward(mode, X, y, up(dy), W, dx0, dw0, T, Bn, In, H, bidir, 0.0)                 # overwrite form
            assert_close(down(dx0, x.shape) + 1.0, outs[1], rtol=2e-4, what="dx beta 0")
            be.rnn_backward(mode, X, y, up(dy), W, None, dw0, T, Bn, In, H, bidir, 1.0)                # input layer: no dx
            assert_close(down(dw0, w.shape) * 0.5 + 1.0, outs[2], rtol=2e-4, what="dw accumulates")
        return outs

    check_all(pair.run(f), rtol=3e-4)


@pytest.mark.parametrize("case", [(2, True, 7, 5, 20, 48), (3, True, 7, 5, 20, 48), (2, False, 1, 2, 5, 16), (3, False, 1, 2, 5, 16), (2, False, 9, 33, 7, 37),
                                  (3, True, 4, 3, 33, 130), (2, True, 3, 4, 161, 96), (3, False, 12, 8, 64, 256),
                                  (2, True, 3, 32, 40, 800), (3, True, 3, 17, 24, 528), (2, False, 2, 20, 12, 1000)]
                         + _random_cases(108, 6, lambda r: (_ri(r, 2, 3), bool(r.rand() < 0.5), _ri(r, 1, 8), _ri(r, 1, 9), _ri(r, 1, 40), _pick(r, [5, 16, 37, 64, 130]))),
                         ids=lambda c: "mode%d_bi%d_T%d_B%d_I%d_H%d" % c)
def test_gated_rnn_forward_and_backward(pair, case):
    """LSTM (mode 2) and GRU (mode 3) layers against the oracle: outputs, input gradient (accumulate, overwrite, none)
    and the packed weight gradient."""
    mode, bidir, T, Bn, In, H = case
    D, G = (2 if bidir else 1), (4 if mode == 2 else 3) * H
    rng = np.random.RandomState(41)
    per = G * In + G * H + 2 * G
    w = (rng.randn(D * per) * (0.7 / np.sqrt(H))).astype(np.float32)
    x = rng.randn(T, Bn, In).astype(np.float32); dy = rng.randn(T, Bn, D * H).astype(np.float32)

    def f(be, up, down):
        X, W = up(x), up(w)
        y, reserve = be.rnn_gated_forward(mode, X, W, T, Bn, In, H, bidir)
        dx = up(np.ones(x.size, np.float32)); dw = up(np.ones(w.size, np.float32))
        be.rnn_gated_backward(mode, X, y, up(dy), W, reserve, dx, dw, T, Bn, In, H, bidir, 1.0)
        outs = [down(y, dy.shape), down(dx, x.shape), down(dw, w.shape)]
        if be.name == "hip":
            y2, reserve2 = be.rnn_gated_forward(mode, X, W, T, Bn, In, H, bidir)                        # the reserve is used up: run forward again
            dx0 = up(np.full(x.size, 5.0, np.float32)); dw0 = up(np.zeros(w.size, np.float32))
            be.rnn_gated_backward(mode, X, y2, up(dy), W, reserve2, dx0, dw0, T, Bn, In, H, bidir, 0.0)  # overwrite form
            assert_close(down(dx0, x.shape) + 1.0, outs[1], rtol=2e-4, what="dx beta 0")
            y3, reserve3 = be.rnn_gated_forward(mode, X, W, T, Bn, In, H, bidir)
            be.rnn_gated_backward(mode, X, y3, up(dy), W, reserve3, None, dw0, T, Bn, In, H, bidir, 1.0)  # input layer: no dx
            assert_close(down(dw0, w.shape) * 0.5 + 1.0, outs[2], rtol=2e-4, what="dw accumulates")
            assert np.array_equal(down(y2, dy.shape), outs[0]) and np.array_equal(down(y3, dy.shape), outs[0])
        return outs

    check_all(pair.run(f), rtol=3e-4)


@pytest.mark.parametrize("case", [(0, True, 5, 3, 7, 37), (1, False, 4, 5, 20, 64), (1, True, 6, 32, 96, 800), (2, True, 7, 5, 20, 48), (2, False, 1, 2, 5, 16),
                                  (3, True, 4, 3, 33, 130), (3, False, 6, 8, 64, 256)], ids=lambda c: "mode%d_bi%d_T%d_B%d_I%d_H%d" % c)
def test_rnn_with_initial_states(pair, case):
    """RNNBase.apply(input, hx, cx): a layer started from a given hidden (and, for the LSTM, cell) state; outputs, input
    gradient and weight gradients.  The states themselves receive no gradient (CDN:1843-1844)."""
    mode, bidir, T, Bn, In, H = case
    ng = {0: 1, 1: 1, 2: 4, 3: 3}[mode]
    D, G = (2 if bidir else 1), ng * H
    rng = np.random.RandomState(51)
    per = G * In + G * H + 2 * G
    w = (rng.randn(D * per) * (0.5 / np.sqrt(H))).astype(np.float32)
    if mode == 0:
        w[:] = np.abs(w) * np.where(rng.rand(w.size) < 0.3, -1, 1)
    x = rng.randn(T, Bn, In).astype(np.float32); dy = rng.randn(T, Bn, D * H).astype(np.float32)
    hx = rng.randn(D, Bn, H).astype(np.float32); cx = rng.randn(D, Bn, H).astype(np.float32)

    def f(be, up, down):
        X, W, HX = up(x), up(w), up(hx)
        CX = up(cx) if mode == 2 else None
        dx = up(np.ones(x.size, np.float32)); dw = up(np.ones(w.size, np.float32))
        if mode < 2:
            y = be.rnn_forward(mode, X, W, T, Bn, In, H, bidir, hx=HX)
            be.rnn_backward(mode, X, y, up(dy), W, dx, dw, T, Bn, In, H, bidir, 1.0, hx=HX)
            y0 = be.rnn_forward(mode, X, W, T, Bn, In, H, bidir)
        else:
            y, reserve = be.rnn_gated_forward(mode, X, W, T, Bn, In, H, bidir, hx=HX, cx=CX)
            be.rnn_gated_backward(mode, X, y, up(dy), W, reserve, dx, dw, T, Bn, In, H, bidir, 1.0, hx=HX, cx=CX)
            y0, _ = be.rnn_gated_forward(mode, X, W, T, Bn, In, H, bidir)
        assert np.abs(down(y, dy.shape) - down(y0, dy.shape)).max() > 1e-3, "the initial state changed nothing"
        return [down(y, dy.shape), down(dx, x.shape), down(dw, w.shape)]

    check_all(pair.run(f), rtol=3e-4)


@pytest.mark.gpu
def test_gated_rnn_rejects_bad_arguments(hip_backend):
    be = hip_backend
    from lantern_amd import _lib
    mark = be.getMallocAddr()
    x = be.mallocArray(8)
    assert be.lib.lh_rnn_gated_reserve_floats(2, 3, 2, 4, 1) == 2 * 3 * 2 * 5 * 4 and be.lib.lh_rnn_gated_reserve_floats(3, 3, 2, 4, 0) == 3 * 2 * 4 * 4
    assert be.lib.lh_rnn_gated_reserve_floats(1, 3, 2, 4, 0) == 0
    with pytest.raises(LanternHipError, match="mode"):
        be.rnn_gated_forward(1, x, x, 1, 1, 1, 1, False)
    with pytest.raises(LanternHipError, match="shape"):
        be.lib.lh_rnn_gated_fwd(2, x.ptr, x.ptr, x.ptr, x.ptr, 0, 1, 1, 1, 0); _lib.check()
    be.resetMallocAddr(mark)


@pytest.mark.parametrize("case", ["ds2", "ragged", "tiny", "long_labels", "lane_limit"])
def test_ctc_loss_and_gradient(pair, case):
    rng = np.random.RandomState(32)
    if case == "ds2":
        T, Bn, A = 185, 32, 29
        lens = np.full(Bn, 50, np.int32); ilen = np.full(Bn, T, np.int32)
    elif case == "ragged":
        T, Bn, A = 40, 7, 11
        lens = np.array([5, 1, 0, 12, 3, 19, 8], np.int32); ilen = np.array([40, 3, 1, 30, 40, 39, 17], np.int32)
    elif case == "long_labels":          # more than 63 symbols: the block-per-sample kernel with states in a loop
        T, Bn, A = 150, 3, 6
        lens = np.array([70, 64, 10], np.int32); ilen = np.array([150, 149, 30], np.int32)
    elif case == "lane_limit":           # 63 symbols = 127 states: the last lane pair of the one-wavefront kernel
        T, Bn, A = 130, 2, 40
        lens = np.array([63, 62], np.int32); ilen = np.array([130, 128], np.int32)
    else:
        T, Bn, A = 3, 1, 2
        lens = np.array([1], np.int32); ilen = np.array([3], np.int32)
    labels = rng.randint(1, A, size=int(lens.sum())).astype(np.int32)
    if case == "ragged":
        labels[5:9] = labels[5]                                   # repeated labels: the skip transition must be closed
    act = (rng.randn(T, Bn, A) * 2).astype(np.float32)
    e = np.exp(act - act.max(2, keepdims=True)); probs = (e / e.sum(2, keepdims=True)).astype(np.float32)

    def f(be, up, down):
        Pb = up(probs); d = up(np.ones(probs.size, np.float32))
        costs = be.ctcLoss(Pb, d, ilen, labels, lens, T, Bn, A)
        c2 = be.ctcLoss(Pb, None, ilen, labels, lens, T, Bn, A)       # no gradient requested
        return [down(costs, (Bn,)), down(d, probs.shape), down(c2, (Bn,))]

    outs = pair.run(f)
    if case == "tiny":            # one label over three frames: p = sum over the 5 alignments b/l placements
        p = probs[:, 0, :]; bl, lb = p[:, 0], p[:, 1]
        want = lb[0] * lb[1] * lb[2] + bl[0] * lb[1] * lb[2] + lb[0] * lb[1] * bl[2] + bl[0] * bl[1] * lb[2] + bl[0] * lb[1] * bl[2] + lb[0] * bl[1] * bl[2]
        np.testing.assert_allclose(outs[1][0][0], -np.log(want), rtol=1e-5)
    check_all(outs, rtol=1e-4)


# ---- convolution with batch-norm statistics from its epilogue -----------------------------------------
CONV_BN = [(64, 64, 56, 64, 1, 1, 0, False),      # 64-row GEMM, 64x128 tiles
           (8, 64, 56, 256, 1, 1, 0, False),      # 128x128 tiles
           (64, 256, 14, 1024, 1, 1, 0, False),   # 784 tiles: a full round + surplus columns in 64x64 tiles
           (4, 32, 15, 48, 3, 2, 1, False),       # odd sizes, partial tiles in both directions
           (2, 16, 9, 24, 3, 1, 1, True),         # with a bias: statistics come from a pass over y
           (64, 512, 7, 512, 3, 1, 1, False),     # few tiles, long reduction: the shared-tile path, statistics from a pass over y
           (2, 3, 20, 16, 5, 1, 2, False)]        # channels not a multiple of 16: the general loader, pass over y


@pytest.mark.parametrize("case", CONV_BN, ids=lambda c: "N%d_C%d_H%d_K%d_k%d_s%d_p%d_b%d" % c)
@pytest.mark.parametrize("relu", [False, True], ids=["plain", "relu"])
def test_conv_with_batchnorm_statistics(pair, case, relu):
    N, Cc, H, K, k, s, p, with_bias = case
    P = B.conv_size(H, k, s, p)
    dims = (N, Cc, H, H, K, k, k, s, s, p, p)
    rng = np.random.RandomState(33)
    x = rng.randn(N, Cc, H, H).astype(np.float32); w = (rng.randn(K, Cc, k, k) / np.sqrt(Cc * k * k)).astype(np.float32)
    bias = (rng.randn(K) * 2).astype(np.float32) if with_bias else None
    g = (rng.rand(K) + 0.5).astype(np.float32); b = rng.randn(K).astype(np.float32)

    def f(be, up, down):
        n = N * K * P * P
        yconv, ybn, sm, si = be.mallocArray(n), be.mallocArray(n), be.mallocArray(K), be.mallocArray(K)
        rm, rv = up(np.zeros(K, np.float32)), up(np.ones(K, np.float32))
        be.conv2D_batch_bn_into(up(x), up(w), up(bias) if with_bias else None, yconv, dims, up(g), up(b), rm, rv, ybn, sm, si, relu)
        outs = [down(yconv, (N, K, P, P)), down(ybn, (N, K, P, P)), down(sm, (K,)), down(si, (K,)), down(rm, (K,)), down(rv, (K,))]
        if be.name == "hip":     # the one-call form against convolution-with-statistics followed by the apply pass: bit for bit
            y2, z2, sm2, si2 = be.mallocArray(n), be.mallocArray(n), be.mallocArray(K), be.mallocArray(K)
            rm2, rv2 = up(np.zeros(K, np.float32)), up(np.ones(K, np.float32))
            be.lib.lh_conv2d_fwd_bnstats(up(x).ptr, up(w).ptr, up(bias).ptr if with_bias else 0, y2.ptr, *dims, sm2.ptr, si2.ptr, rm2.ptr, rv2.ptr, 1e-5, 0.1)
            be.lib.lh_bn_apply(y2.ptr, up(g).ptr, up(b).ptr, sm2.ptr, si2.ptr, z2.ptr, N, K, P * P, int(relu))
            from lantern_amd import _lib
            _lib.check()
            two = [down(y2, (N, K, P, P)), down(z2, (N, K, P, P)), down(sm2, (K,)), down(si2, (K,)), down(rm2, (K,)), down(rv2, (K,))]
            same_conv = np.array_equal(outs[0], two[0])      # launch plans that share tiles between blocks add with atomics
            for i_, (a_, b_) in enumerate(zip(outs, two)):
                if same_conv:
                    np.testing.assert_array_equal(a_, b_, err_msg="one call vs two calls, output %d" % i_)
                else:
                    assert_close(a_, b_, rtol=1e-4, what="one call vs two calls, output %d" % i_)
            assert same_conv or case[2] <= 7, "only the few-tile shapes may differ between two launches"
        return outs

    outs = pair.run(f)
    if relu:        # values within rounding of zero may land on either side of the relu
        edge = np.abs(outs[0][1]) < 2e-5
        for o in outs:
            o[1][edge & (np.abs(o[1]) < 4e-5)] = 0.0
    check_all(outs, rtol=2e-4)



# ---- command list: small operators recorded and run in order by one workgroup --------------------------
def _small_op_program(be, rng_seed=50, n=150, m=37):
    """A chain of dependent small operators covering every recordable entry point; returns host copies of all results."""
    rng = np.random.RandomState(rng_seed)
    up = lambda a: be.fromHost(np.ascontiguousarray(a, np.float32))
    W = up(rng.randn(m, n) * 0.1); x = up(rng.randn(n)); bias = up(rng.randn(m)); gy = up(rng.randn(m))
    lib = be.lib
    outs = []
    h = be.matrixVectorDot(W, x, m, n)                                        # gemv
    lib.lh_bcast_update(B.ADD, h.ptr, B._ints((m,)), bias.ptr, B._ints((m,)), 1)   # += bias
    s = be.unary(B.SIGMOID, h, m); t = be.unary(B.TANH, h, m)
    prod = be.bcast_op(B.MUL, s, (m,), t, (m,), (m,))
    diff = be.bcast_op(B.SUB, prod, (m,), bias, (m,), (m,))
    sc = be.scalar_op(B.MUL, diff, 0.5, m)
    ge = be.mallocArray(m, zero=False); be.geam(sc, 2.0, t, -1.0, ge, m)
    dotv = be.vectorVectorDot(ge, gy, m)
    outs += [(h, m), (s, m), (prod, m), (diff, m), (sc, m), (ge, m), (dotv, 1)]
    # gradients back through the chain
    dprod = be.mallocArray(m); dbias = be.mallocArray(m); ds = be.mallocArray(m); dt = be.mallocArray(m); dh = be.mallocArray(m)
    be.bcast_op_grad(B.SUB, prod, dprod, (m,), False, bias, dbias, (m,), False, gy, (m,))
    be.bcast_op_grad(B.MUL, s, ds, (m,), False, t, dt, (m,), False, dprod, (m,))
    be.unary_grad(B.SIGMOID, h, s, ds, dh, m); be.unary_grad(B.TANH, h, t, dt, dh, m)
    dW = be.mallocArray(m * n); dx = be.mallocArray(n)
    be.add_cartesian(dW, x, dh, m, n); be.add_composition(dx, W, dh, m, n)
    be.addMul_scalar(dx, dotv, x, n)                                           # dx += dotv[0] * x
    outs += [(dprod, m), (dbias, m), (ds, m), (dt, m), (dh, m), (dW, m * n), (dx, n)]
    # classifier head: rows of 5 classes
    logits = be.mallocArray(3 * 5, zero=False); be.copyFloatArray(logits, h, 15)
    lsm = be.softmax(1, logits, 3, 5, 1); sm = be.softmax(0, logits, 3, 5, 1)
    tgt = be.fromHost(np.array([4, 0, 2], np.int32))
    loss = be.nllLoss(lsm, tgt, 3, 5)
    dl = be.mallocArray(15); dlog = be.mallocArray(15)
    be.nllLoss_grad(dl, tgt, up(np.ones(3)), 3, 5)
    be.softmax_grad(1, lsm, dl, dlog, 3, 5, 1); be.softmax_grad(0, sm, dl, dlog, 3, 5, 1)
    outs += [(lsm, 15), (sm, 15), (loss, 3), (dl, 15), (dlog, 15)]
    # optimizers consume and clear the gradient
    cache = be.mallocArray(m * n)
    lib.lh_adagrad(W.ptr, dW.ptr, cache.ptr, 0.05, 1.0, m * n)
    lib.lh_sgd(x.ptr, dx.ptr, 0.1, n)
    outs += [(W, m * n), (cache, m * n), (x, n), (dW, m * n)]
    return [be.toHost(buf, cnt).copy() for buf, cnt in outs]


@pytest.mark.parametrize("n,m", [(150, 37), (1000, 64), (64, 300), (4100, 16)], ids=["150x37", "1000x64", "64x300", "4100x16"])
def test_command_list_matches_one_launch_per_operator(on_hip, n, m):
    be = on_hip
    direct = _small_op_program(be, n=n, m=m)
    rec0, launches0 = be.cmdlistStats()
    be.batchSmallOps(True)
    try:
        listed = _small_op_program(be, n=n, m=m)
    finally:
        be.batchSmallOps(False)
    rec, launches = be.cmdlistStats()
    assert rec - rec0 >= 25 and 0 < launches - launches0 <= 30, (rec - rec0, launches - launches0)
    # the products sum in another order than the stand-alone kernels: 2e-6 over 150 terms; over 1000 and more the differences reach
    # 1e-6 of a product, and the gradients and the Adagrad step behind them (differences of near-equal terms) carry that to 1e-5
    for i, (a, b_) in enumerate(zip(listed, direct)):
        assert_close(a, b_, rtol=2e-6 if n <= 150 else 1e-4, what="result %d" % i)


def test_command_list_reports_a_barrier_that_gave_up_and_stays_usable(on_hip):
    """A workgroup whose barrier wait runs out sets a flag in pinned host memory and all workgroups leave.  The flag is set
    from the host here (no kernel is made to give up): the next call that waits for the device reports it once, also when
    nothing is pending, the barrier counters start over, and the same commands then run and give the right result."""
    be = on_hip
    lib = be.lib
    one = be.fromHost(np.ones(64, np.float32))
    be.batchSmallOps(True)
    try:
        acc = be.mallocArray(64)
        for _ in range(5):
            lib.lh_bcast_update(B.ADD, acc.ptr, B._ints((64,)), one.ptr, B._ints((64,)), 1)
        be.sync()                                                               # handed over and finished: nothing pending now
        lib.lh_cmdlist_inject_timeout()
        with pytest.raises(LanternHipError, match="timed out"):
            be.sync()                                                           # reported although no command is pending
        be.sync()                                                               # once
        lib.lh_cmdlist_inject_timeout()
        with pytest.raises(LanternHipError, match="timed out"):
            be.toHost(acc, 64)                                                  # a read-back reports it too
        for _ in range(7):                                                      # the library is usable: levels and barriers start over
            lib.lh_bcast_update(B.ADD, acc.ptr, B._ints((64,)), one.ptr, B._ints((64,)), 1)
        assert (be.toHost(acc, 64) == 12.0).all()
        lib.lh_cmdlist_inject_timeout()
        lib.lh_cmdlist_end()                                                    # lh_cmdlist_end reports it as well
        with pytest.raises(LanternHipError, match="timed out"):
            la._lib.check()
    finally:
        be.batchSmallOps(False)
    be.sync()


def test_command_list_keeps_program_order_around_other_kernels_and_wraps_its_buffers(on_hip):
    """Recorded commands, kernels too large to record and copies interleave in program order; more commands than the
    pinned buffers hold in total go through without loss."""
    be = on_hip
    lib = be.lib
    big_n = 1 << 20                                                             # above the recording limit: a normal launch
    big = be.mallocArray(big_n, zero=False); small = be.mallocArray(64); one = be.fromHost(np.ones(64, np.float32))
    be.batchSmallOps(True)
    try:
        lib.lh_fill(small.ptr, 3.0, 64)                                         # recorded
        lib.lh_fill(big.ptr, 2.0, big_n)                                        # launched: the recorded fill must land first
        lib.lh_geam(small.ptr, 1.0, big.ptr, 1.0, small.ptr, 64)                # recorded: reads what the big fill wrote -> 5
        lib.lh_scalar_op(B.MUL, big.ptr, big.ptr, 0.5, big_n)                   # launched after the recorded read
        lib.lh_geam(small.ptr, 1.0, big.ptr, 1.0, small.ptr, 64)                # 5 + 1 = 6
        assert (be.toHost(small, 64) == 6.0).all()
        z = be.mallocArray(300)                                                 # the arena's zero fill is recorded too
        lib.lh_bcast_update(B.ADD, z.ptr, B._ints((64,)), small.ptr, B._ints((64,)), 1)
        assert (be.toHost(z, 300)[:64] == 6.0).all() and not be.toHost(z, 300)[64:].any()
        cnt = be.mallocArray(64)
        for _ in range(10000):                                                  # 10000 dependent commands: five buffers' worth
            lib.lh_bcast_update(B.ADD, cnt.ptr, B._ints((64,)), one.ptr, B._ints((64,)), 1)
        assert (be.toHost(cnt, 64) == 10000.0).all()
    finally:
        be.batchSmallOps(False)
    from lantern_amd import _lib
    _lib.check()


@pytest.mark.parametrize("n_vec,vlen,m", [(12, 150, 24), (10, 1000, 37), (8, 4500, 8), (12, 67, 67)],
                         ids=["150x24", "1000x37", "4500x8_shared_by_all_workgroups", "67x67"])
def test_command_list_reordering_keeps_every_dependence(on_hip, n_vec, vlen, m):
    """The command list runs independent commands of a buffer side by side and dependent ones in order.  A random program of
    several hundred small operations over a few buffers and their sub-ranges (reads after writes, writes after reads, writes
    after writes; vectors inside a matrix another command updates as a whole; a scalar one command leaves for the next) must
    give the bits of the same program issued one launch per operator, whose order is the program's."""
    be = on_hip
    lib = be.lib
    sub = min(64, vlen // 3)                    # length of the sub-range operations, which start a third into a vector

    def program():
        mark = be.getMallocAddr()
        r = np.random.RandomState(5)
        vecs = [be.fromHost((r.rand(vlen) + 0.5).astype(np.float32)) for _ in range(n_vec)]
        mat = be.fromHost((r.rand(m * vlen) * 0.1).astype(np.float32))
        scal = be.mallocArray(1)
        ops = np.random.RandomState(9)
        for step in range(600):
            k = ops.randint(0, 9)
            a, b_, c = (int(v) for v in ops.randint(0, n_vec, 3))
            row = int(ops.randint(0, m))
            if k == 0: lib.lh_geam(vecs[a].ptr, 0.5, vecs[b_].ptr, 0.5, vecs[c].ptr, vlen)                      # c = (a + b) / 2
            elif k == 1: lib.lh_unary(B.TANH, vecs[a].ptr, vecs[c].ptr, vlen, -1.0, 1.0)
            elif k == 2: lib.lh_geam(vecs[a].ptr, 1.0, mat.ptr + 4 * row * vlen, 0.25, vecs[a].ptr, vlen)          # reads a row of the matrix
            elif k == 3: lib.lh_ger(m, vlen, vecs[a].ptr, vecs[b_].ptr, mat.ptr) if a != b_ else None               # updates the whole matrix (u = first m of a)
            elif k == 4: lib.lh_sgemv(0, m, vlen, 0.01, mat.ptr, vlen, vecs[a].ptr, 0.0, vecs[c].ptr)                # first m elements of c
            elif k == 5: lib.lh_sgemv(1, m, vlen, 0.01, mat.ptr, vlen, vecs[a].ptr, 1.0, vecs[c].ptr) if a != c else None
            elif k == 6: lib.lh_fill(mat.ptr + 4 * row * vlen, 0.02 * (step % 7), vlen)                               # overwrites one row
            elif k == 7:
                lib.lh_dot_vv(vecs[a].ptr, vecs[b_].ptr, scal.ptr, vlen)
                lib.lh_scalar_op(B.MUL, scal.ptr, scal.ptr, 1e-3, 1)
                lib.lh_axpy_dev(vecs[c].ptr, scal.ptr, vecs[a].ptr, vlen) if a != c else None
            else: lib.lh_geam(vecs[a].ptr, 1.0, vecs[b_].ptr + 4 * (vlen // 3), -0.5, vecs[a].ptr, sub)              # a[:sub] -= b[third : third + sub] / 2
            # keep the values bounded: the matrix is halved after an update, a vector that was added to goes through tanh (in place)
            if k == 3 and a != b_: lib.lh_scalar_op(B.MUL, mat.ptr, mat.ptr, 0.5, m * vlen)
            if k in (2, 8): lib.lh_unary(B.TANH, vecs[a].ptr, vecs[a].ptr, vlen, -1.0, 1.0)
            if k in (5, 7) and a != c: lib.lh_unary(B.TANH, vecs[c].ptr, vecs[c].ptr, vlen, -1.0, 1.0)
        from lantern_amd import _lib
        _lib.check()
        out = [be.toHost(v, vlen).copy() for v in vecs] + [be.toHost(mat, m * vlen).copy()]
        be.resetMallocAddr(mark)
        return out

    direct = program()
    be.batchSmallOps(True)
    try:
        listed = program()
    finally:
        be.batchSmallOps(False)
    assert all(np.isfinite(a).all() for a in direct)
    # the matrix commands sum in another order than the stand-alone kernels (whose transposed product combines blocks with atomic
    # adds, so its own result moves in the last bits from run to run), and 600 dependent operations carry that along and spread it
    # (differences of 1e-5 to 5e-5 of a value are seen): 1e-3; a command that ran before what it depends on is off by 1e-2 and more
    for i, (a, b_) in enumerate(zip(listed, direct)):
        assert_close(a, b_, rtol=1e-3, what="buffer %d" % i)


def test_command_list_long_element_wise_chains_keep_their_operands_in_lds(on_hip):
    """Chains of element-wise commands on the same vectors (each lane reads what it wrote itself) run inside one level; from four
    commands on, the chain's operands are loaded into LDS slots before its first command and every result is written to the slot and
    to memory.  Several independent chains of 60 commands over shared read-only inputs, in-place updates, operands of different
    lengths at one address, more distinct operands than a workgroup has slots (the rest go through memory), gradient forms, and a
    read of every buffer by a matrix command afterwards must give the bits of the same program issued one launch per operator."""
    be = on_hip
    lib = be.lib
    vlen = 150

    def program():
        mark = be.getMallocAddr()
        r = np.random.RandomState(3)
        const = [be.fromHost((r.rand(vlen) + 0.5).astype(np.float32)) for _ in range(6)]        # read by every chain, written by none
        outs = []
        for chain in range(5):
            n_own = 4 if chain < 4 else 48                                                        # the last chain has more operands than slots
            own = [be.fromHost((r.rand(vlen) * 0.5 + 0.25).astype(np.float32)) for _ in range(n_own)]
            ops = np.random.RandomState(100 + chain)
            for step in range(60):
                k = int(ops.randint(0, 8))
                a, b_, c = (int(v) for v in ops.randint(0, n_own, 3))
                u = const[int(ops.randint(0, len(const)))]
                if k == 0: lib.lh_geam(own[a].ptr, 0.5, u.ptr, 0.25, own[c].ptr, vlen)
                elif k == 1: lib.lh_unary(B.TANH, own[a].ptr, own[c].ptr, vlen, -1.0, 1.0)
                elif k == 2: lib.lh_unary(B.SIGMOID, own[a].ptr, own[a].ptr, vlen, -1.0, 1.0)      # in place
                elif k == 3: lib.lh_geam(own[a].ptr, 1.0, own[b_].ptr, -0.5, own[a].ptr, 40)        # a shorter range at the same address
                elif k == 4: lib.lh_scalar_op(B.MUL, own[a].ptr, own[c].ptr, 0.75, vlen)
                elif k == 5: lib.lh_unary_grad(B.TANH, u.ptr, own[a].ptr, own[b_].ptr, own[c].ptr, vlen, 0, -1.0, 1.0) if c not in (a, b_) else None
                elif k == 6: lib.lh_fill(own[c].ptr, 0.125 * (step % 5), 100)
                else: lib.lh_geam(own[a].ptr, 0.9, own[b_].ptr, 0.1, own[c].ptr, vlen)
                if k == 5 and c not in (a, b_): lib.lh_unary(B.TANH, own[c].ptr, own[c].ptr, vlen, -1.0, 1.0)   # keeps the accumulator bounded
            outs += own
        # a matrix command over all results afterwards (another level: it must see what the chains wrote through to memory)
        acc = be.mallocArray(vlen)
        for v in outs[:8]: lib.lh_ger(1, vlen, const[0].ptr, v.ptr, acc.ptr)
        from lantern_amd import _lib
        _lib.check()
        res = [be.toHost(v, vlen).copy() for v in outs] + [be.toHost(acc, vlen).copy()] + [be.toHost(v, vlen).copy() for v in const]
        be.resetMallocAddr(mark)
        return res

    direct = program()
    be.batchSmallOps(True)
    try:
        listed = program()
    finally:
        be.batchSmallOps(False)
    assert all(np.isfinite(a).all() for a in direct)
    n_chain_buffers = 4 * 4 + 48
    for i, (a, b_) in enumerate(zip(listed, direct)):
        if i == n_chain_buffers: assert_close(a, b_, rtol=2e-6, what="rank-1 updates over the chains' results")      # a + u * v may or may not be fused
        else: assert np.array_equal(a, b_), "buffer %d differs by up to %g" % (i, np.abs(a - b_).max())


# ---- residual join behind a batch norm: out = relu(bn(x) + shortcut) -----------------------------------
@pytest.mark.parametrize("shape", [(8, 16, 28, 28), (3, 5, 7, 7), (4, 32, 1, 1), (16, 128, 112, 112)], ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("beta_sd", [0.0, 1.0, None], ids=["shortcut_grad_fresh", "shortcut_grad_accumulates", "shortcut_is_input"])
def test_batchnorm_add_relu_join_forward_and_backward(pair, shape, beta_sd):
    N, Cc, H, W = shape
    HW, n = H * W, N * Cc * H * W
    rng = np.random.RandomState(60)
    x = rng.randn(*shape).astype(np.float32); s = rng.randn(*shape).astype(np.float32); dout = rng.randn(*shape).astype(np.float32)
    g = (rng.rand(Cc) + 0.5).astype(np.float32); b = (rng.randn(Cc) * 0.3).astype(np.float32)

    pre = (x.astype(np.float64) - x.mean((0, 2, 3), keepdims=True)) / np.sqrt(x.var((0, 2, 3), keepdims=True) + 1e-5) * g.reshape(1, -1, 1, 1) + b.reshape(1, -1, 1, 1) + s
    s[np.abs(pre) < 1e-4] += 0.01               # keep every element away from the relu's kink: a flipped mask changes the whole channel

    def f(be, up, down):
        X, S, G, Bb = up(x), up(s), up(g), up(b)
        rm, rv = up(np.zeros(Cc, np.float32)), up(np.ones(Cc, np.float32))
        out = be.mallocArray(n, zero=False); sm = be.mallocArray(Cc, zero=False); si = be.mallocArray(Cc, zero=False)
        be.batchNormTraining_add_relu_into(X, G, Bb, rm, rv, S, out, sm, si, N, Cc, HW)
        dx = up(np.full(n, 2.0, np.float32)); dg = up(np.ones(Cc, np.float32)); db = up(np.ones(Cc, np.float32))
        sd = None if beta_sd is None else up(np.full(n, 3.0, np.float32))
        D = up(dout)
        be.batchNorm_add_relu_grad(X, dx, 1.0, out, D, G, dg, db, sm, si, sd, beta_sd if beta_sd is not None else 1.0, N, Cc, HW)
        outs = [down(out, shape), down(dx, shape), down(dg, (Cc,)), down(db, (Cc,)), down(rm, (Cc,)), down(rv, (Cc,))]
        if sd is not None:
            outs.append(down(sd, shape))
        return outs

    outs = pair.run(f)
    check_all(outs, rtol=2e-4)


# ---- side stream: filter gradients beside the main chain of kernels -------------------------------------
def test_side_stream_filter_gradients_match_in_line_and_wait_for_their_inputs(on_hip):
    """Through the C ABI: dy is produced on the main stream right before the fork (the side work must wait for it),
    main-stream work that does not touch the operands follows, the optimizer-style join comes last.  Accumulating twice
    into one dw from the side stream, then once in line, must give three times the in-line gradient."""
    be, lib = on_hip, on_hip.lib
    dims = (8, 32, 20, 20, 48, 3, 3, 1, 1, 1, 1)
    N, Cc, H, W, K = dims[:5]
    rng = np.random.RandomState(71)
    x = be.fromHost(rng.randn(N * Cc * H * W).astype(np.float32)); dy0 = be.fromHost(rng.randn(N * K * H * W).astype(np.float32))
    n_dy = N * K * H * W; n_w = K * Cc * 9

    def grads(side):
        lib.lh_set_side_stream(1 if side else 0)
        forks0 = lib.lh_side_forks()
        dy = be.mallocArray(n_dy, zero=False); dw = be.mallocArray(n_w); db = be.mallocArray(K); other = be.mallocArray(1 << 20, zero=False)
        lib.lh_scalar_op(B.MUL, dy0.ptr, dy.ptr, 1.0, n_dy)      # dy written on the main stream just before
        for rep in range(2):
            lib.lh_side_begin()
            lib.lh_conv2d_bwd_filter(x.ptr, dy.ptr, dw.ptr, db.ptr, 1.0, *dims)
            lib.lh_side_end()
            for _ in range(4):                                   # unrelated main-stream work meanwhile
                lib.lh_fill(other.ptr, float(rep), 1 << 20)
        lib.lh_conv2d_bwd_filter(x.ptr, dy.ptr, dw.ptr, db.ptr, 1.0, *dims)     # in line: joins first
        from lantern_amd import _lib
        _lib.check()
        out = (be.toHost(dw, n_w).copy(), be.toHost(db, K).copy())              # the read-back joins too
        lib.lh_set_side_stream(1)
        return out, lib.lh_side_forks() - forks0

    (dw_a, db_a), forks_a = grads(False)
    (dw_b, db_b), forks_b = grads(True)
    assert forks_a == 0 and forks_b == 2
    assert_close(dw_b, dw_a, rtol=1e-5, what="filter gradient from the side stream")
    assert_close(db_b, db_a, rtol=1e-5, what="bias gradient from the side stream")
    assert np.abs(dw_a).max() > 1.0


def test_convolution_applied_twice_accumulates_one_filter_gradient_across_streams(pair):
    """One Conv2D module used deep in the network (its filter gradient goes to the side stream) and again on the
    network input (in line): both accumulate into the same gradient buffer."""
    from lantern_amd.nn import Conv2D
    rng = np.random.RandomState(72)
    x = rng.randn(4, 8, 12, 12).astype(np.float32)
    w0 = (rng.randn(8, 8, 3, 3) * 0.2).astype(np.float32)

    def f(be, up, down):
        conv = Conv2D(8, 8, (3, 3), pad=(1, 1), useBias=True, init=lambda dims: w0)
        xin = la.TensorR(la.Tensor.fromNumpy(x), isInput=True)

        def loss(dummy):
            h = conv(xin).tanh()
            for _ in range(7):
                h = (h * h).tanh()
            h = conv(h)                       # the deep use
            for _ in range(7):
                h = (h * h).tanh()
            return h.sum()
        forks0 = be.lib.lh_side_forks() if be.name == "hip" else 0
        if be.name == "hip":
            keep, be.side_min_convs = be.side_min_convs, 1      # fork as soon as ONE more convolution gradient follows (the default asks for two)
        try:
            lval = la.gradR_loss(loss)(la.Tensor.zeros(1))
        finally:
            if be.name == "hip":
                be.side_min_convs = keep
        if be.name == "hip":
            assert be.lib.lh_side_forks() - forks0 == 1
        return [lval.toCPU().copy(), conv.kernel.d.toCPU().copy(), conv.bias.d.toCPU().copy()]

    outs = pair.run(f)
    check_all(outs, rtol=1e-4)


def test_side_stream_contract_errors_are_reported_and_leave_the_library_usable(on_hip):
    """Nested forks, a join or a zero-filled allocation between lh_side_begin and lh_side_end are refused with a message;
    with the side stream switched off the same calls run in line."""
    be, lib = on_hip, on_hip.lib
    from lantern_amd import _lib
    lib.lh_set_side_stream(1)
    lib.lh_side_begin(); _lib.check()
    for call, text in ((lambda: lib.lh_side_begin(), "already on the side stream"),
                       (lambda: lib.lh_side_join(), "lh_side_join between"),
                       (lambda: lib.lh_malloc(1024), "main-stream order only")):
        call()
        with pytest.raises(LanternHipError, match=text):
            _lib.check()
    u = lib.lh_malloc_uninit(1024); _lib.check()             # scratch without a zero fill is allowed there
    assert u
    lib.lh_fill(u, 3.0, 256); _lib.check()                    # runs on the side stream
    lib.lh_side_end(); _lib.check()
    assert (be.toHost(B.Buf(u, 256), 256) == 3.0).all()       # the read-back joins first
    forks = lib.lh_side_forks()
    lib.lh_set_side_stream(0)
    lib.lh_side_begin(); lib.lh_fill(u, 4.0, 256); lib.lh_side_end(); _lib.check()      # in line
    assert lib.lh_side_forks() == forks and (be.toHost(B.Buf(u, 256), 256) == 4.0).all()
    lib.lh_set_side_stream(1)


@pytest.mark.parametrize("shape,context", [((7, 3, 5), 2), ((5, 4), 4), ((9,), 1), ((30, 2, 16), 20), ((4, 1, 1), 0)], ids=str)
def test_repeat0_and_grad(pair, shape, context):
    """repeat0 (TD:1446-1451): values against numpy's sliding windows bit for bit, gradient against the scatter the
    definition fixes (every window's slice added back to the rows it was cut from)."""
    rng = np.random.RandomState(51)
    x = rng.randn(*shape).astype(np.float32)
    rows, inner = shape[0], int(np.prod(shape[1:]))
    oshape = (rows - context, context + 1) + tuple(shape[1:])
    dy = rng.randn(*oshape).astype(np.float32)
    want_y = np.stack([x[i:i + context + 1] for i in range(rows - context)])
    want_dx = np.ones_like(x)
    for i0 in range(rows - context):
        for i1 in range(context + 1):
            want_dx[i0 + i1] += dy[i0, i1]

    def f(be, up, down):
        y = be.repeat0(up(x), rows, context, inner)
        xd = up(np.ones(x.size, np.float32))
        be.repeat0_grad(xd, up(dy), rows, context, inner)
        return [down(y, oshape), down(xd, x.shape)]

    outs = pair.run(f)
    check_all(outs, exact=(0,), rtol=1e-5)
    for o in outs:
        assert np.array_equal(o[0], want_y)
        np.testing.assert_allclose(o[1], want_dx, rtol=1e-5, atol=1e-6)


def test_lookahead_module_forward_and_gradient(be):
    """Lookahead (DeepSpeech.scala:54-66) through the tape: y[t, b, f] = sum_k x[t + k, b, f] w[f, k] with zero padding, and the
    gradients of sum(y * g) with respect to x and w, against numpy."""
    from lantern_amd.nn import Lookahead
    from lantern_amd.tensor import Tensor, TensorR, _tape, _run_tape
    rng = np.random.RandomState(52)
    T, Bn, F, ctx = 6, 2, 5, 3
    x = rng.randn(T, Bn, F).astype(np.float32); g = rng.randn(T, Bn, F).astype(np.float32)
    Tensor.randseed(3)
    la_mod = Lookahead(F, ctx)
    w = la_mod.weight.x.toCPU().reshape(F, ctx + 1)
    xr = TensorR(Tensor.fromNumpy(x))
    start = len(_tape)
    y = la_mod(xr)
    be.upload(y.d.data, g)
    _run_tape(start)
    xp = np.concatenate([x, np.zeros((ctx, Bn, F), np.float32)])
    want = sum(xp[k:k + T] * w[:, k] for k in range(ctx + 1))
    np.testing.assert_allclose(y.x.toCPU().reshape(T, Bn, F), want, rtol=1e-5, atol=1e-6)
    want_dx = np.zeros_like(xp)
    for k in range(ctx + 1):
        want_dx[k:k + T] += g * w[:, k]
    np.testing.assert_allclose(xr.d.toCPU().reshape(T, Bn, F), want_dx[:T], rtol=1e-5, atol=1e-6)
    want_dw = np.stack([(g * xp[k:k + T]).sum(axis=(0, 1)) for k in range(ctx + 1)], axis=1)
    np.testing.assert_allclose(la_mod.weight.d.toCPU().reshape(F, ctx + 1), want_dw, rtol=1e-4, atol=1e-5)
