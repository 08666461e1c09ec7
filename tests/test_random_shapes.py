"""Seeded random geometries against the CPU oracle: the hand-picked cases of the other parity files name the paths the
kernels take; these sweeps look for the ones nobody thought of (partial tiles, odd strides and pads, windows hanging over
the border, reductions shorter than a tile).  Every case is printed before it runs so that a failure names its geometry."""
import ctypes as C
import sys

import numpy as np
import pytest

from oracle.backend_cpu import load as load_oracle
from tests.test_parity_conv import check_conv
from tests.util import Dev, assert_close, cptr

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True); sys.stdout.flush()


def _conv_case(rng):
    R, S = [int(rng.choice([1, 1, 2, 3, 3, 4, 5, 7])) for _ in range(2)]
    if rng.rand() < 0.6: S = R
    sH, sW = [int(rng.choice([1, 1, 1, 2, 2, 3])) for _ in range(2)]
    pH, pW = int(rng.randint(0, R)), int(rng.randint(0, S))             # pad < kernel, as the reference's programs use
    H = int(rng.randint(max(1, R - 2 * pH), 26)); W = int(rng.randint(max(1, S - 2 * pW), 26))
    N = int(rng.randint(1, 6)); Cc = int(rng.choice([1, 2, 3, 4, 7, 8, 16, 17, 32, 40, 64, 96])); K = int(rng.choice([1, 2, 5, 8, 16, 24, 33, 64, 70, 130]))
    return (N, Cc, H, W, K, R, S, sH, sW, pH, pW)


@pytest.mark.parametrize("group", range(8))
def test_random_conv_geometries(on_hip, group):
    dev = Dev(on_hip)
    rng = np.random.RandomState(1000 + group)
    for i in range(8):
        dims = _conv_case(rng); bias = bool(rng.rand() < 0.5)
        _say("conv group %d case %d dims %s bias %s" % (group, i, dims, bias))
        mark = on_hip.getMallocAddr()
        check_conv(dev, dims, bias)
        on_hip.sync(); on_hip.resetMallocAddr(mark)


def _conv_case_for_the_filter_gradient_loaders(rng, wide):
    """Maps of up to 39 x 39 pixels (odd pixel counts of 32 and more take the padded numbering of the filter gradient's reduction);
    wide: no padding and filter rows of 5 to 11 taps (x gathered with the lanes along the columns)."""
    if wide:
        R = int(rng.choice([1, 2, 3, 5, 9])); S = int(rng.choice([5, 6, 7, 11])); sH, sW = int(rng.choice([1, 2, 3])), int(rng.choice([1, 1, 2])); pH = pW = 0
    else:
        R = int(rng.choice([1, 3, 5])); S = int(rng.choice([1, 3, 5])); sH, sW = int(rng.choice([1, 1, 2])), int(rng.choice([1, 1, 2]))
        pH, pW = int(rng.randint(0, R)), int(rng.randint(0, S))
    H = int(rng.randint(max(1, R - 2 * pH) + 3, 40)); W = int(rng.randint(max(1, S - 2 * pW) + 3, 40))
    N = int(rng.choice([1, 2, 3, 5, 8, 16])); Cc = int(rng.choice([1, 2, 3, 4, 7, 16, 17, 32, 40, 64])); K = int(rng.choice([1, 5, 8, 16, 24, 32, 33, 64, 70, 130]))
    return (N, Cc, H, W, K, R, S, sH, sW, pH, pW)


@pytest.mark.parametrize("group", range(4))
def test_random_conv_geometries_odd_maps_and_unpadded_wide_filters(on_hip, group):
    dev = Dev(on_hip)
    rng = np.random.RandomState(4000 + group)
    for i in range(8):
        dims = _conv_case_for_the_filter_gradient_loaders(rng, wide=bool(i & 1)); bias = bool(rng.rand() < 0.5)
        det = group == 3                     # the last group in deterministic mode (slices of the reduction added up by a second kernel)
        _say("conv (filter-gradient loaders) group %d case %d dims %s bias %s deterministic %s" % (group, i, dims, bias, det))
        mark = on_hip.getMallocAddr()
        if det: on_hip.setDeterministic(True)
        try:
            check_conv(dev, dims, bias)
        finally:
            if det: on_hip.setDeterministic(False)
        on_hip.sync(); on_hip.resetMallocAddr(mark)


@pytest.mark.parametrize("group", range(3))
def test_random_conv_geometries_on_32_row_tiles(on_hip, group, monkeypatch):
    """The same sweep with at most 32 channels on either side and the library's test switch that sends every product of at
    most 32 rows to the 32 x 128 tile (forward, input gradient with its strided residue classes, filter gradient)."""
    monkeypatch.setenv("LH_FORCE_M32", "1")
    dev = Dev(on_hip)
    rng = np.random.RandomState(3000 + group)
    for i in range(8):
        d = list(_conv_case(rng))
        d[1] = int(rng.choice([1, 3, 4, 8, 16, 20, 32])); d[4] = int(rng.choice([1, 5, 10, 16, 20, 32]))
        dims = tuple(d); bias = bool(rng.rand() < 0.5)
        _say("conv (32-row tiles) group %d case %d dims %s bias %s" % (group, i, dims, bias))
        mark = on_hip.getMallocAddr()
        check_conv(dev, dims, bias)
        on_hip.sync(); on_hip.resetMallocAddr(mark)


@pytest.mark.parametrize("group", range(4))
def test_random_sgemm_shapes_with_row_strides(on_hip, group):
    """All four transpose forms, leading dimensions larger than the rows (views into wider matrices), alpha/beta."""
    dev = Dev(on_hip); lc = load_oracle()
    rng = np.random.RandomState(2000 + group)
    for i in range(10):
        ta, tb = int(rng.randint(2)), int(rng.randint(2))
        m, n, k = [int(rng.choice([1, 2, 3, 7, 16, 31, 64, 65, 100, 129, 200, 257])) for _ in range(3)]
        pa, pb, pc = [int(rng.choice([0, 0, 1, 4, 13])) for _ in range(3)]
        alpha, beta = float(rng.choice([1.0, 0.5, -2.0])), float(rng.choice([0.0, 1.0, 0.25]))
        _say("sgemm group %d case %d ta%d tb%d m%d n%d k%d pads %d %d %d alpha %g beta %g" % (group, i, ta, tb, m, n, k, pa, pb, pc, alpha, beta))
        ash = (k, m) if ta else (m, k); bsh = (n, k) if tb else (k, n)
        A = rng.randn(ash[0], ash[1] + pa).astype(np.float32); Bm = rng.randn(bsh[0], bsh[1] + pb).astype(np.float32)
        Cm = rng.randn(m, n + pc).astype(np.float32)
        ref = Cm.copy()
        lc.lc_sgemm(C.c_int(ta), C.c_int(tb), C.c_int(m), C.c_int(n), C.c_int(k), C.c_float(alpha), cptr(A), C.c_int(A.shape[1]),
                    cptr(Bm), C.c_int(Bm.shape[1]), C.c_float(beta), cptr(ref), C.c_int(Cm.shape[1]))
        mark = on_hip.getMallocAddr()
        c_ = dev.up(Cm)
        dev.lib.lh_sgemm(ta, tb, m, n, k, alpha, dev.up(A).ptr, A.shape[1], dev.up(Bm).ptr, Bm.shape[1], beta, c_.ptr, Cm.shape[1]); dev.check()
        got = dev.down(c_, Cm.shape)
        assert_close(got[:, :n], ref[:, :n], what="sgemm values")
        np.testing.assert_array_equal(got[:, n:], Cm[:, n:], err_msg="columns beyond n were written")
        on_hip.sync(); on_hip.resetMallocAddr(mark)


# ---- random networks: the library's deferred work against the same calls run as issued -------------------------------------------
class _RandomNet:
    """A stack of blocks drawn at random from what the five applications are made of: conv -> batchNorm -> relu(inPlace), conv with bias
    -> relu(inPlace), a residual block (two such convolutions, the shortcut plain or projected, + and relu), a fire module (squeeze, two
    expands, concat) and max-pooling; then a classifier convolution over what is left of the map.  Every tensor of a step is large
    enough for its clearing to be put off."""

    def __init__(self, rng, classes=7):
        from lantern_amd.nn import Module, Conv2D, BatchNorm2D
        self.m = Module("randomnet")
        self.blocks = []
        c, hw = 3, int(rng.choice([16, 24, 32]))
        self.hw0 = hw
        kinds = ["cbr", "cr", "res", "fire", "pool"]
        for i in range(int(rng.randint(3, 7))):
            kind = kinds[int(rng.randint(len(kinds)))] if i else "cbr"
            if kind == "pool" and hw < 8: kind = "cr"
            co = int(rng.choice([16, 24, 32, 48, 64]))
            k = int(rng.choice([1, 3, 3, 5])); pad = (k // 2, k // 2)
            stride = (2, 2) if (kind in ("cbr", "cr") and hw >= 16 and rng.rand() < 0.3) else (1, 1)
            name = "b%d" % i
            if kind == "cbr":
                conv = self.m.add(Conv2D(c, co, (k, k), stride, pad, useBias=False, name=name + "conv", rng=rng)); bn = self.m.add(BatchNorm2D(co, name + "bn"))
                self.blocks.append(("cbr", conv, bn)); c = co; hw = (hw + 2 * pad[0] - k) // stride[0] + 1
            elif kind == "cr":
                conv = self.m.add(Conv2D(c, co, (k, k), stride, pad, useBias=True, name=name + "conv", rng=rng))
                self.blocks.append(("cr", conv)); c = co; hw = (hw + 2 * pad[0] - k) // stride[0] + 1
            elif kind == "res":
                mid = int(rng.choice([8, 16, 32]))
                c1 = self.m.add(Conv2D(c, mid, (1, 1), useBias=False, name=name + "c1", rng=rng)); b1 = self.m.add(BatchNorm2D(mid, name + "b1"))
                c2 = self.m.add(Conv2D(mid, co, (3, 3), (1, 1), (1, 1), useBias=False, name=name + "c2", rng=rng)); b2 = self.m.add(BatchNorm2D(co, name + "b2"))
                proj = None
                if co != c or rng.rand() < 0.3:
                    proj = (self.m.add(Conv2D(c, co, (1, 1), useBias=False, name=name + "pc", rng=rng)), self.m.add(BatchNorm2D(co, name + "pb")))
                self.blocks.append(("res", c1, b1, c2, b2, proj)); c = co
            elif kind == "fire":
                sq = int(rng.choice([8, 16])); e1, e3 = int(rng.choice([16, 32])), int(rng.choice([16, 32]))
                s = self.m.add(Conv2D(c, sq, (1, 1), name=name + "s", rng=rng)); a = self.m.add(Conv2D(sq, e1, (1, 1), name=name + "e1", rng=rng))
                b = self.m.add(Conv2D(sq, e3, (3, 3), (1, 1), (1, 1), name=name + "e3", rng=rng))
                self.blocks.append(("fire", s, a, b)); c = e1 + e3
            else:
                self.blocks.append(("pool",)); hw = hw // 2
        self.head = self.m.add(Conv2D(c, classes, (hw, hw), name="head", rng=rng))
        self.classes = classes

    def __call__(self, x):
        h = x
        for b in self.blocks:
            if b[0] == "cbr": h = b[2](b[1](h)).relu(True)
            elif b[0] == "cr": h = b[1](h).relu(True)
            elif b[0] == "res":
                o = b[2](b[1](h)).relu(True); o = b[4](b[3](o))
                idt = h if b[5] is None else b[5][1](b[5][0](h))
                h = (o + idt).relu(True)
            elif b[0] == "fire":
                s = b[1](h).relu(True); h = b[2](s).relu(True).concat(1, b[3](s).relu(True))
            else: h = h.maxPoolBK((2, 2), (2, 2), None)
        h = self.head(h)
        return h.resize(h.x.shape[0], -1)


def _random_net_steps(be, seed, steps, fusion):
    """Losses and parameters after `steps` momentum steps of the network drawn from `seed` (deterministic mode set by the caller)."""
    import lantern_amd as la
    from lantern_amd.nn import SGD_Momentum
    from lantern_amd.tensor import Tensor, TensorR, gradR_loss, int_array
    la.set_backend(be)
    if hasattr(be, "lib") and hasattr(be.lib, "lh_set_fusion"): be.lib.lh_set_fusion(1 if fusion else 0)
    mark = be.getMallocAddr()
    rng = np.random.RandomState(seed)
    net = _RandomNet(rng)
    opt = SGD_Momentum(net.m, 0.01, 0.9)
    x = Tensor.fromNumpy(rng.standard_normal((8, 3, net.hw0, net.hw0)).astype(np.float32))
    target = int_array(rng.randint(0, net.classes, size=8).astype(np.int32))
    inner = be.getMallocAddr()
    losses = []
    for _ in range(steps):
        xin = TensorR(x, isInput=True)
        loss = gradR_loss(lambda dummy: net(xin).logSoftmaxB().nllLossB(target).mean())(Tensor.zeros(1))
        opt.step()
        losses.append(float(loss.toCPU()[0]))
        be.resetMallocAddr(inner)
    params = [(n, p.x.toCPU().copy()) for n, p in net.m.namedParameters()]
    if hasattr(be, "sync"): be.sync()
    be.resetMallocAddr(mark)
    return np.array(losses), params, [b[0] for b in net.blocks]


@pytest.mark.parametrize("seed", range(10))
def test_random_networks_fused_and_as_issued_give_the_same_bits_and_track_the_oracle(hip_backend, cpu_backend, seed, monkeypatch):
    """Three momentum steps of a random stack of the applications' blocks, one library call per trait method.  With the library's deferred
    work (chains fused, clears put off, filter copies kept, the optimizer's calls gathered) and with every call run as issued
    (lh_set_fusion(0)) the losses and all parameters are the same bits in deterministic mode, once the one thing that is summed in another
    order is taken out: LH_FORCE_STATS_TILE=4 has a fused convolution leave its batch-norm statistics to the stand-alone pass instead of its
    epilogue.  With the epilogue statistics back in, the fused run tracks the oracle."""
    be = hip_backend
    be.setDeterministic(True)
    try:
        monkeypatch.setenv("LH_FORCE_STATS_TILE", "4")
        l1, p1, kinds = _random_net_steps(be, 500 + seed, 3, fusion=True)
        _say("random network %d: blocks %s, losses %s" % (seed, kinds, l1))
        l0, p0, _ = _random_net_steps(be, 500 + seed, 3, fusion=False)
        monkeypatch.delenv("LH_FORCE_STATS_TILE")
        l2, p2, _ = _random_net_steps(be, 500 + seed, 3, fusion=True)
    finally:
        be.lib.lh_set_fusion(1)
        be.setDeterministic(False)
    np.testing.assert_array_equal(l1, l0)
    for (n, a), (_, b) in zip(p1, p0):
        np.testing.assert_array_equal(a, b, err_msg=n)
    np.testing.assert_allclose(l2, l1, rtol=1e-4, atol=1e-5)            # the statistics from the epilogue: another order of the same sums
    lc, pc, _ = _random_net_steps(cpu_backend, 500 + seed, 3, fusion=True)
    np.testing.assert_allclose(l2, lc, rtol=1e-3, atol=1e-5)
    for (n, a), (_, b) in zip(p2, pc):
        assert_close(a, b, rtol=2e-3, what="against the oracle: " + n)


class _RandomNetTrainer:
    """The random network above behind the applications' trainer protocol (step, end_step, model)."""

    def __init__(self, seed):
        import lantern_amd as la
        from lantern_amd.nn import SGD_Momentum
        from lantern_amd.tensor import Tensor, int_array, get_backend
        rng = np.random.RandomState(seed)
        self.net = _RandomNet(rng); self.model = self.net.m
        self.opt = SGD_Momentum(self.model, 0.01, 0.9)
        self.x = Tensor.fromNumpy(rng.standard_normal((8, 3, self.net.hw0, self.net.hw0)).astype(np.float32))
        self.target = int_array(rng.randint(0, self.net.classes, size=8).astype(np.int32))
        self.mark = get_backend().getMallocAddr()

    def step(self):
        from lantern_amd.tensor import Tensor, TensorR, gradR_loss
        xin = TensorR(self.x, isInput=True)
        loss = gradR_loss(lambda dummy: self.net(xin).logSoftmaxB().nllLossB(self.target).mean())(Tensor.zeros(1))
        self.opt.step()
        return loss

    def end_step(self):
        from lantern_amd.tensor import get_backend
        get_backend().resetMallocAddr(self.mark)


@pytest.mark.parametrize("seed", range(4))
def test_random_networks_graph_replays_give_the_eager_steps_bits(hip_backend, seed):
    """The same random networks with the step recorded into a HIP graph after two eager steps: four replays, with eager work of the
    program's own between them, give the losses and parameters of the same steps run eagerly, bit for bit in deterministic mode."""
    from tests.test_training_parity import _graph_against_eager
    _graph_against_eager(lambda: _RandomNetTrainer(700 + seed), hip_backend, eager_steps=2, replays=4, tol=0.0, per_tensor=1e-12, deterministic=True)
