"""Host-side logic: shape rules, the tape, that the front end issues one backend call per trait method, and (on both backends)
that the chains the library fuses give what the calls as issued give."""
import numpy as np
import pytest

import lantern_amd as la
from lantern_amd import Tensor, TensorR, gradR, gradR_loss
from lantern_amd.backend import dim_broadcast, conv_size
from lantern_amd.tensor import resize_dim
import lantern_amd.tensor as T


def test_dim_broadcast():  # T/TestBroadcast.scala:14-46 (dimBroadcast cases)
    assert dim_broadcast((2, 3), (2, 3)) == ((2, 3), (2, 3), (2, 3))
    assert dim_broadcast((2, 3), (1, 3)) == ((2, 3), (1, 3), (2, 3))
    assert dim_broadcast((2, 2, 2), (2,)) == ((2, 2, 2), (1, 1, 2), (2, 2, 2))
    assert dim_broadcast((3,), (4, 1)) == ((1, 3), (4, 1), (4, 3))
    with pytest.raises(ValueError):
        dim_broadcast((2, 3), (2, 3, 3)[1:] + (2,))


def test_resize_dim_and_conv_size():  # TD:34-49
    assert resize_dim(320 * 100, (-1, 320)) == (100, 320)
    assert resize_dim(24, (2, 3, 4)) == (2, 3, 4)
    with pytest.raises(ValueError):
        resize_dim(24, (-1, -1))
    with pytest.raises(ValueError):
        resize_dim(24, (5, 5))
    assert conv_size(28, 5, 1) == 24 and conv_size(224, 7, 2, 3) == 112 and conv_size(112, 3, 2, 1) == 56


def test_gradients_accumulate_across_uses(on_cpu):
    # x used twice: d = dL/dx summed over both uses (TD accumulates into d)
    x = TensorR(Tensor.fromData((3,), 1, 2, 3))
    gradR_loss(lambda d: (x * x).sum())(Tensor.zeros(1))
    np.testing.assert_allclose(x.d.toCPU(), [2, 4, 6])
    gradR_loss(lambda d: (x * 3.0).sum())(Tensor.zeros(1))
    np.testing.assert_allclose(x.d.toCPU(), [5, 7, 9])         # accumulated on top


def test_input_gets_no_gradient(on_cpu):  # TD:1510: inputs carry a 2-element dummy d
    x = TensorR(Tensor.ones(1, 1, 4, 4), isInput=True)
    k = TensorR(Tensor.ones(1, 1, 3, 3))
    gradR_loss(lambda d: x.convBBP(k, None, (1, 1), (0, 0)).sum())(Tensor.zeros(1))
    assert x.d.scalarCount == 2 and (x.d.toCPU() == 0).all()
    np.testing.assert_allclose(k.d.toCPU().ravel(), [4] * 9)


def test_gradient_through_add_relu_add(be):
    rng = np.random.RandomState(0)
    a, b = rng.randn(2, 3, 4, 4).astype(np.float32), rng.randn(2, 3, 4, 4).astype(np.float32)

    def run():
        x, y = TensorR(Tensor.fromNumpy(a)), TensorR(Tensor.fromNumpy(b))
        gradR_loss(lambda d: ((x + y).relu(True) + x).sum())(Tensor.zeros(1))
        return x.d.toCPU(), y.d.toCPU()
    gx, gy = run()
    mask = (a + b) > 0
    np.testing.assert_allclose(gx, mask + 1.0)
    np.testing.assert_allclose(gy, mask * 1.0)


class _Recorder:
    """Stands in front of a backend and notes the name of every method the front end calls."""

    def __init__(self, inner):
        self._inner, self.calls = inner, []

    def __getattr__(self, name):
        v = getattr(self._inner, name)
        if not callable(v):
            return v
        def call(*a, **k):
            self.calls.append(name)
            return v(*a, **k)
        return call

    def __setattr__(self, name, value):
        if name in ("_inner", "calls"):
            object.__setattr__(self, name, value)
        else:
            setattr(self._inner, name, value)


def test_front_end_issues_one_backend_call_per_trait_method(on_cpu):
    """The front end fuses nothing: conv -> batchNorm -> relu(inPlace) -> + -> relu(inPlace) reaches the backend as the calls
    the reference stages for it (TD:1171-1176, 1324-1329, 1394-1410; relu in place: TD:1232-1238), gradients in reverse order,
    and the optimizer as one momentum_update per parameter (NN:296-303)."""
    from lantern_amd.nn import Module, Conv2D, BatchNorm2D, SGD_Momentum
    rng = np.random.RandomState(1)

    class Net(Module):
        def __init__(self):
            super().__init__("net")
            self.conv = self.add(Conv2D(3, 3, (3, 3), (1, 1), (1, 1), useBias=False, rng=rng))
            self.bn = self.add(BatchNorm2D(3))

        def __call__(self, x):
            h = self.bn(self.conv(x)).relu(True)
            return (self.bn(self.conv(h)) + h).relu(True)
    net = Net()
    opt = SGD_Momentum(net, 0.1, 0.9)
    x = TensorR(Tensor.fromNumpy(rng.randn(2, 3, 4, 4).astype(np.float32)), isInput=True)
    rec = _Recorder(on_cpu)
    la.set_backend(rec)
    try:
        gradR_loss(lambda d: net(x).sum())(Tensor.zeros(1))
        opt.step()
    finally:
        la.set_backend(on_cpu)
    ops = [c for c in rec.calls if c not in ("mallocArray", "fillInPlace", "copyFloatArray")]
    assert ops == ["conv2D_batch", "batchNormTraining", "unary",
                   "conv2D_batch", "batchNormTraining", "bcast_op", "unary", "sum",
                   "add_scalar_from", "unary_grad", "bcast_op_grad", "batchNorm_grad", "conv2D_batch_grad",
                   "unary_grad", "batchNorm_grad", "conv2D_batch_grad",
                   "momentum_update", "momentum_update", "momentum_update"], ops


def _fusion(be, on):
    """Switch the library's fusion of adjacent calls (the oracle has none to switch)."""
    if be.name == "hip":
        be.lib.lh_set_fusion(1 if on else 0)


def test_fused_and_unfused_relu_gradients_agree(be):
    """batchNorm -> relu(inPlace): the library runs the pair as one kernel (forward) and one fused backward; with a read of
    the batch norm's output in between, or with fusion off, every call runs on its own.  Same values, same gradients."""
    rng = np.random.RandomState(2)
    xs = rng.randn(4, 3, 5, 5).astype(np.float32)

    def run(fused, lib_fusion=True):
        _fusion(be, lib_fusion)
        try:
            x = TensorR(Tensor.fromNumpy(xs)); g = TensorR(Tensor.fromData((3,), 1.5, 0.5, 2.0)); b = TensorR(Tensor.fromData((3,), 0.1, -0.2, 0.0))
            def f(d):
                y = x.batchNorm(g, b, Tensor.zeros(3), Tensor.ones(3))
                if not fused:
                    y.x.toCPU()                 # a read in between: the batch norm has to run before the relu is known
                return (y.relu(True) * 2.0).sum()
            gradR_loss(f)(Tensor.zeros(1))
            return x.d.toCPU(), g.d.toCPU(), b.d.toCPU()
        finally:
            _fusion(be, True)
    want = run(True)
    for other in (run(False), run(True, lib_fusion=False)):
        for u, v in zip(want, other):
            np.testing.assert_allclose(u, v, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("bn_side", ["left", "right"])
def test_residual_join_matches_the_unfused_program(be, bn_side):
    """conv -> batchNorm -> + shortcut -> relu(inPlace): the library runs the chain as one convolution launch and one
    normalise-add-relu pass and never stores the batchNorm's own output; values and every gradient equal the program with
    fusion off, and a later read of the batchNorm's output (and of the gradient buffers the fused backward left unmasked)
    still gives what the calls as issued would have left there."""
    rng = np.random.RandomState(3)
    xs = rng.randn(2, 4, 6, 6).astype(np.float32); ws = (rng.randn(4, 4, 3, 3) * 0.2).astype(np.float32)

    def run(fused):
        _fusion(be, fused)
        try:
            x = TensorR(Tensor.fromNumpy(xs)); w = TensorR(Tensor.fromNumpy(ws))
            g = TensorR(Tensor.fromData((4,), 1.5, 0.5, 2.0, 1.0)); b = TensorR(Tensor.fromData((4,), 0.1, -0.2, 0.0, 0.3))
            kept = {}
            def f(d):
                h = (x * 1.5)                                     # the shortcut has a gradient of its own
                y = h.convBBP(w, None, (1, 1), (1, 1)).batchNorm(g, b, Tensor.zeros(4), Tensor.ones(4))
                kept["bn"] = y
                z = (y + h) if bn_side == "left" else (h + y)
                out = z.relu(True)
                kept["z"] = out
                return (out * out).sum()
            gradR_loss(f)(Tensor.zeros(1))
            res = [kept["z"].x.toCPU(), x.d.toCPU(), w.d.toCPU(), g.d.toCPU(), b.d.toCPU()]
            # read last: what the fused chain did not store (the batch norm's output, its gradient buffer = the masked gradient,
            # and the join's gradient buffer masked in place by relu_grad)
            res += [kept["bn"].x.toCPU(), kept["bn"].d.toCPU(), kept["z"].d.toCPU()]
            return res
        finally:
            _fusion(be, True)
    fused, plain = run(True), run(False)
    for u, v in zip(fused, plain):
        np.testing.assert_allclose(u, v, rtol=1e-5, atol=1e-6)


def test_batchnorm_followed_by_add_without_relu_runs_unfused(be):
    rng = np.random.RandomState(4)
    xs = rng.randn(3, 2, 4, 4).astype(np.float32)
    x = TensorR(Tensor.fromNumpy(xs)); g, b = TensorR(Tensor.ones(2)), TensorR(Tensor.zeros(2))
    s = TensorR(Tensor.fromNumpy(rng.randn(3, 2, 4, 4).astype(np.float32)))
    y = x.batchNorm(g, b, Tensor.zeros(2), Tensor.ones(2))
    z = y + s
    v = z.x.toCPU()                                                   # no relu follows: batchNorm, then the add
    ref = (xs - xs.mean(axis=(0, 2, 3), keepdims=True)) / np.sqrt(xs.var(axis=(0, 2, 3), keepdims=True) + 1e-5)
    np.testing.assert_allclose(v, ref + s.x.toCPU(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(y.x.toCPU(), ref, rtol=1e-4, atol=1e-5)      # and the batchNorm's output exists
    T._tape.clear()


def test_join_whose_shortcut_is_the_batchnorms_own_input(be):
    """relu(bn(h) + h): the batch norm's input is also the shortcut, so the fused backward would be handed one buffer for both of
    its gradient outputs (its first pass adds the masked gradient into what its second pass overwrites, losing the shortcut's
    share).  The library runs this join unfused; values and gradients equal the program with the fusion switched off."""
    rng = np.random.RandomState(5)
    xs = rng.randn(4, 3, 5, 5).astype(np.float32)

    def run(fused):
        _fusion(be, fused)
        try:
            x = TensorR(Tensor.fromNumpy(xs)); g = TensorR(Tensor.fromData((3,), 1.5, 0.5, 2.0)); b = TensorR(Tensor.fromData((3,), 0.1, -0.2, 0.3))
            kept = {}
            def f(d):
                h = x * 1.5
                out = (h.batchNorm(g, b, Tensor.zeros(3), Tensor.ones(3)) + h).relu(True)
                kept["out"] = out
                return (out * out).sum()
            gradR_loss(f)(Tensor.zeros(1))
            return [kept["out"].x.toCPU(), x.d.toCPU(), g.d.toCPU(), b.d.toCPU()]
        finally:
            _fusion(be, True)
    fused, plain = run(True), run(False)
    for u, v in zip(fused, plain):
        np.testing.assert_allclose(u, v, rtol=1e-5, atol=1e-6)
    # and against the definition: d/dh [relu(bn(h) + h)] has the identity term of the shortcut
    h = 1.5 * xs.astype(np.float64)
    mu = h.mean((0, 2, 3), keepdims=True); var = h.var((0, 2, 3), keepdims=True); xhat = (h - mu) / np.sqrt(var + 1e-5)
    gam = np.array([1.5, 0.5, 2.0]).reshape(1, 3, 1, 1); bet = np.array([0.1, -0.2, 0.3]).reshape(1, 3, 1, 1)
    out = np.maximum(gam * xhat + bet + h, 0)
    np.testing.assert_allclose(fused[0], out, rtol=1e-4, atol=1e-5)
    dz = 2 * out * (out > 0)
    dxhat = dz * gam
    dh = (dxhat - dxhat.mean((0, 2, 3), keepdims=True) - xhat * (dxhat * xhat).mean((0, 2, 3), keepdims=True)) / np.sqrt(var + 1e-5) + dz
    np.testing.assert_allclose(fused[1], 1.5 * dh, rtol=2e-4, atol=2e-4)


def test_relu_mask_recording_counts_flips(on_cpu):
    """The tracking tests' relu-mask comparison (tests/test_training_parity.py): `_run(masks=)` records the sign pattern of every
    non-negative tape value per step, `_mask_flips` counts where two runs differ.  Two runs of the same program on the oracle
    record identical masks; one flipped bit in one tensor of one step is reported as exactly that."""
    from tests.test_training_parity import _run, _mask_flips
    from lantern_amd.apps.lenet import Trainer
    mk = lambda: Trainer(batch=4, lr=0.0005)
    m1, m2 = [], []
    l1, _ = _run(mk, on_cpu, 2, masks=m1)
    l2, _ = _run(mk, on_cpu, 2, masks=m2)
    np.testing.assert_array_equal(l1, l2)
    assert len(m1) == 2 and any(m is not None for m in m1[0]), "no relu output was recorded"
    assert _mask_flips(m1, m2) == []
    i = next(k for k, m in enumerate(m2[1]) if m is not None)
    shape, bits = m2[1][i]
    flipped = bits.copy(); flipped[0] ^= 0x80
    m2[1][i] = (shape, flipped)
    assert _mask_flips(m1, m2) == [(1, 1, 1)]
