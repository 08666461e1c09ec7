"""conv2D_batch forward / input gradient / filter gradient: HIP (through the C ABI) against
the CPU oracle on the same seeded inputs.  Tolerance 1e-4 relative (see util.assert_close)."""
import ctypes as C

import numpy as np
import pytest

from oracle.backend_cpu import load as load_oracle
from tests.util import Dev, assert_close, cptr

pytestmark = pytest.mark.gpu

# (N, C, H, W, K, R, S, sH, sW, pH, pW)
SHAPES = [
    (2, 3, 9, 9, 8, 3, 3, 1, 1, 1, 1),        # tiny, channels not a multiple of anything
    (3, 1, 28, 28, 10, 5, 5, 1, 1, 0, 0),     # LeNet conv1
    (3, 10, 12, 12, 20, 5, 5, 1, 1, 0, 0),    # LeNet conv2
    (2, 64, 14, 14, 64, 1, 1, 1, 1, 0, 0),    # 1x1 stride 1 (plain GEMM)
    (2, 64, 14, 14, 128, 1, 1, 2, 2, 0, 0),   # 1x1 stride 2 (ResNet downsample)
    (2, 32, 14, 14, 48, 3, 3, 1, 1, 1, 1),    # 3x3 pad 1
    (2, 32, 15, 13, 40, 3, 3, 2, 2, 1, 1),    # 3x3 stride 2, odd non-square input
    (2, 3, 32, 32, 16, 7, 7, 2, 2, 3, 3),     # 7x7 stride 2 pad 3 (ResNet stem)
    (4, 16, 7, 7, 24, 3, 3, 1, 1, 1, 1),      # 7x7 maps: P*Q = 49 not a multiple of 4
    (2, 130, 8, 8, 136, 3, 3, 1, 1, 1, 1),    # M and K just past one 128 tile
    (1, 1, 41, 30, 8, 11, 5, 2, 2, 0, 0),     # tall DeepSpeech-like kernel, stride (2,2)
    (1, 4, 21, 30, 6, 5, 3, 2, 1, 2, 1),      # anisotropic stride and pad
    (2, 96, 16, 16, 16, 1, 1, 1, 1, 0, 0),    # SqueezeNet squeeze (K = 16)
    (2, 512, 4, 4, 10, 4, 4, 1, 1, 0, 0),     # SqueezeNet head: 4x4 kernel onto 1x1
    (5, 256, 7, 7, 64, 1, 1, 1, 1, 0, 0),     # long reduction, 49-pixel maps
    (3, 20, 9, 7, 24, 3, 3, 1, 1, 1, 1),      # 63-pixel maps: the last group of a sample has three real elements
    (4, 64, 14, 14, 96, 1, 1, 2, 2, 0, 0),    # 1x1 stride 2 onto 7x7 maps (gathered x, padded reduction numbering)
    (2, 4, 21, 37, 32, 5, 3, 2, 1, 0, 1),     # 9x37 maps (333 pixels), 32 output channels: the 32-row tile
    (3, 136, 7, 7, 130, 1, 1, 1, 1, 0, 0),    # 49-pixel maps, rows and columns just past one 128 tile
    (2, 3, 13, 15, 12, 5, 5, 1, 1, 0, 0),     # no padding, 5-wide filter rows (x gathered with the lanes along (c, r, s)), 99-pixel maps
    (2, 2, 31, 24, 32, 7, 6, 2, 1, 0, 0),     # the same with anisotropic stride, 247-pixel maps and the 32-row tile
    (2, 6, 30, 24, 40, 9, 5, 2, 1, 0, 0),     # the same over maps of 220 pixels (a multiple of 4)
]


def _oracle_conv(x, w, b, dy, dims, need_dx=True):
    lc = load_oracle()
    N, Cc, H, W, K, R, S, sH, sW, pH, pW = dims
    P, Q = (H + 2 * pH - R) // sH + 1, (W + 2 * pW - S) // sW + 1
    y = np.zeros((N, K, P, Q), np.float32)
    fin = np.zeros((N, Cc * R * S, P * Q), np.float32)
    ints = [C.c_int(v) for v in dims]
    lc.lc_conv2d_fwd(cptr(x), cptr(w), cptr(b) if b is not None else None, cptr(y), cptr(fin), *ints)
    dx = np.zeros_like(x); dw = np.zeros_like(w); db = np.zeros(K, np.float32)
    scratch = np.zeros_like(fin)
    lc.lc_conv2d_bwd(cptr(fin), cptr(w), cptr(dy), cptr(dx) if need_dx else None, cptr(dw), cptr(db), cptr(scratch), *ints)
    return y, dx, dw, db


@pytest.mark.parametrize("dims", SHAPES, ids=lambda d: "x".join(map(str, d)))
@pytest.mark.parametrize("bias", [False, True], ids=["nobias", "bias"])
def test_conv_fwd_bwd(on_hip, dims, bias):
    check_conv(Dev(on_hip), dims, bias)


def check_conv(dev, dims, bias):
    """Forward, input gradient and filter (+ bias) gradient of one geometry against the oracle, overwrite and accumulate forms."""
    N, Cc, H, W, K, R, S, sH, sW, pH, pW = dims
    P, Q = (H + 2 * pH - R) // sH + 1, (W + 2 * pW - S) // sW + 1
    rng = np.random.RandomState(hash(dims) % (2 ** 31))
    x = rng.randn(N, Cc, H, W).astype(np.float32)
    w = (rng.randn(K, Cc, R, S) / np.sqrt(Cc * R * S)).astype(np.float32)
    b = rng.randn(K).astype(np.float32) if bias else None
    dy = rng.randn(N, K, P, Q).astype(np.float32)
    y_ref, dx_ref, dw_ref, db_ref = _oracle_conv(x, w, b, dy, dims)

    ints = list(dims)
    dx_, dw_ = dev.up(x), dev.up(w)
    db_ = dev.up(b) if bias else None
    y_ = dev.zeros(y_ref.size)
    dev.lib.lh_conv2d_fwd(dx_.ptr, dw_.ptr, db_.ptr if bias else 0, y_.ptr, *ints); dev.check()
    assert_close(dev.down(y_, y_ref.shape), y_ref, what="conv fwd")

    ddy = dev.up(dy)
    # input gradient: overwrite (beta 0) into garbage, then accumulate (beta 1) on top
    gdx = dev.up(np.full(x.shape, 7.0, np.float32))
    dev.lib.lh_conv2d_bwd_data(ddy.ptr, dw_.ptr, gdx.ptr, 0.0, *ints); dev.check()
    assert_close(dev.down(gdx, x.shape), dx_ref, what="conv bwd_data beta=0")
    dev.lib.lh_conv2d_bwd_data(ddy.ptr, dw_.ptr, gdx.ptr, 1.0, *ints); dev.check()
    assert_close(dev.down(gdx, x.shape), 2 * dx_ref, what="conv bwd_data beta=1")

    gdw = dev.up(np.full(w.shape, -3.0, np.float32))
    gdb = dev.up(np.ones(K, np.float32))
    dev.lib.lh_conv2d_bwd_filter(dx_.ptr, ddy.ptr, gdw.ptr, gdb.ptr if bias else 0, 0.0, *ints); dev.check()
    assert_close(dev.down(gdw, w.shape), dw_ref, what="conv bwd_filter beta=0")
    dev.lib.lh_conv2d_bwd_filter(dx_.ptr, ddy.ptr, gdw.ptr, gdb.ptr if bias else 0, 1.0, *ints); dev.check()
    assert_close(dev.down(gdw, w.shape), 2 * dw_ref, what="conv bwd_filter beta=1")
    if bias:
        assert_close(dev.down(gdb, (K,)), 1 + 2 * db_ref, what="conv bias grad")


def test_conv_linearity_at_resnet_shape(on_hip):
    """Size-independent property at a full ResNet-50 layer shape (too slow for the oracle in a unit
    test): conv(a*x1 + x2, w) == a*conv(x1, w) + conv(x2, w), and the sum of the output equals
    the closed form for an all-ones filter on a constant input interior."""
    dev = Dev(on_hip)
    dims = (8, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1)
    N, Cc, H, W, K, R, S = dims[:7]
    rng = np.random.RandomState(5)
    x1 = rng.randn(N, Cc, H, W).astype(np.float32); x2 = rng.randn(N, Cc, H, W).astype(np.float32)
    w = (rng.randn(K, Cc, R, S) / 24).astype(np.float32)
    dw_ = dev.up(w)
    outs = []
    for xin in (x1, x2, (2.5 * x1 + x2).astype(np.float32)):
        y_ = dev.zeros(N * K * H * W)
        dev.lib.lh_conv2d_fwd(dev.up(xin).ptr, dw_.ptr, 0, y_.ptr, *dims); dev.check()
        outs.append(dev.down(y_, (N, K, H, W)))
    assert_close(outs[2], 2.5 * outs[0] + outs[1], rtol=1e-4, what="linearity")
    ones_w = dev.up(np.ones((K, Cc, R, S), np.float32))
    y_ = dev.zeros(N * K * H * W)
    dev.lib.lh_conv2d_fwd(dev.up(np.ones((N, Cc, H, W), np.float32)).ptr, ones_w.ptr, 0, y_.ptr, *dims); dev.check()
    y = dev.down(y_, (N, K, H, W))
    assert (y[:, :, 1:-1, 1:-1] == Cc * 9).all() and (y[:, :, 0, 0] == Cc * 4).all() and (y[:, :, 0, 1:-1] == Cc * 6).all()


GEMMS = [(0, 0, 64, 1000, 2048), (0, 1, 64, 1000, 2048), (1, 0, 70, 130, 257), (1, 1, 33, 65, 129),
         (0, 0, 100, 50, 320), (0, 1, 5, 7, 3), (0, 0, 2, 3, 4), (1, 0, 300, 300, 64),
         (0, 1, 64, 10, 2048), (1, 0, 12, 7, 1500), (0, 0, 5, 3, 700), (1, 1, 9, 15, 513)]      # few outputs over a long reduction: the sliced small kernel


@pytest.mark.parametrize("ta,tb,m,n,k", GEMMS)
def test_sgemm(on_hip, ta, tb, m, n, k):
    dev = Dev(on_hip)
    lc = load_oracle()
    rng = np.random.RandomState(m * 131 + n * 7 + k)
    A = rng.randn(*((k, m) if ta else (m, k))).astype(np.float32)
    B = rng.randn(*((n, k) if tb else (k, n))).astype(np.float32)
    Cm = rng.randn(m, n).astype(np.float32)
    for alpha, beta in ((1.0, 0.0), (0.5, 1.0)):
        ref = Cm.copy()
        lc.lc_sgemm(C.c_int(ta), C.c_int(tb), C.c_int(m), C.c_int(n), C.c_int(k), C.c_float(alpha), cptr(A), C.c_int(A.shape[1]),
                    cptr(B), C.c_int(B.shape[1]), C.c_float(beta), cptr(ref), C.c_int(n))
        c_ = dev.up(Cm)
        dev.lib.lh_sgemm(ta, tb, m, n, k, alpha, dev.up(A).ptr, A.shape[1], dev.up(B).ptr, B.shape[1], beta, c_.ptr, n); dev.check()
        assert_close(dev.down(c_, (m, n)), ref, what="sgemm %d%d a=%g b=%g" % (ta, tb, alpha, beta))


# Shapes large enough for the launch plans to be measured on first use (well above the 1e7-flop floor) and small enough for the oracle.
TUNED_SHAPES = [
    (8, 64, 28, 28, 64, 3, 3, 1, 1, 1, 1),      # tap path, 64-row product
    (4, 256, 14, 14, 256, 3, 3, 1, 1, 1, 1),    # few tiles over a long reduction: the stream-K plans compete
    (16, 128, 14, 14, 512, 1, 1, 1, 1, 0, 0),   # 1x1: the plain filter-gradient loaders
    (8, 64, 28, 28, 128, 3, 3, 2, 2, 1, 1),     # stride 2: four residue classes share a pre-zeroed dx (never timed)
    (6, 96, 15, 15, 160, 3, 3, 1, 1, 1, 1),     # odd map, partial tiles everywhere
    (16, 32, 28, 28, 32, 3, 3, 1, 1, 1, 1),     # 32 channels in and out: the 32-row tiles compete in forward and input gradient (tap path)
    (50, 10, 12, 12, 20, 5, 5, 1, 1, 0, 0),     # LeNet's second convolution: 20- and 10-row products through the general loaders
    (8, 1, 41, 60, 32, 11, 5, 2, 2, 0, 0),      # one input channel, tall filter, stride 2 (DeepSpeech2's first layer in small)
    (64, 512, 4, 4, 10, 4, 4, 1, 1, 0, 0),      # a filter as large as the map (SqueezeNet's classifier): one tile under an 8192-long reduction, the plans with one worker per few slabs compete
    (32, 512, 7, 7, 512, 1, 1, 1, 1, 0, 0),     # 1x1 over 49-pixel maps: the filter gradient's padded numbering, slices by atomic adds or in two passes as measured
    (16, 256, 7, 7, 256, 3, 3, 1, 1, 1, 1),     # 3x3 over 49-pixel maps
    (4, 32, 33, 45, 32, 9, 5, 2, 1, 0, 0),      # DeepSpeech2's second layer in small: 13x41 maps (533 pixels), no padding, x gathered with the lanes along the columns
]


@pytest.mark.parametrize("dims", TUNED_SHAPES, ids=lambda d: "x".join(map(str, d)))
def test_conv_measured_launch_plans_and_their_reuse(on_hip, dims):
    """First calls time several launch plans (repeating the launch), later calls reuse the remembered plan, also with an
    accumulating epilogue; every call must give the oracle's result, with the tuner on and off."""
    dev = Dev(on_hip)
    lib = on_hip.lib
    N, Cc, H, W, K, R, S, sH, sW, pH, pW = dims
    P, Q = (H + 2 * pH - R) // sH + 1, (W + 2 * pW - S) // sW + 1
    rng = np.random.RandomState(77)
    x = rng.randn(N, Cc, H, W).astype(np.float32)
    w = (rng.randn(K, Cc, R, S) / np.sqrt(Cc * R * S)).astype(np.float32)
    dy = rng.randn(N, K, P, Q).astype(np.float32)
    y_ref, dx_ref, dw_ref, _ = _oracle_conv(x, w, None, dy, dims)
    mean_ref = y_ref.astype(np.float64).mean((0, 2, 3)); var_ref = y_ref.astype(np.float64).var((0, 2, 3))
    ints = list(dims)
    xd, wd, dyd = dev.up(x), dev.up(w), dev.up(dy)
    try:
        for tuning in (1, 1, 0, 1):                     # measures, reuses, built-in rule, reuses again
            lib.lh_set_tuning(tuning)
            y = dev.zeros(y_ref.size); lib.lh_conv2d_fwd(xd.ptr, wd.ptr, 0, y.ptr, *ints)
            assert_close(dev.down(y, y_ref.shape), y_ref, what="fwd (tuning %d)" % tuning)
            y2 = dev.zeros(y_ref.size); sm = dev.zeros(K); si = dev.zeros(K); rm = dev.zeros(K); rv = dev.up(np.ones(K, np.float32))
            lib.lh_conv2d_fwd_bnstats(xd.ptr, wd.ptr, 0, y2.ptr, *ints, sm.ptr, si.ptr, rm.ptr, rv.ptr, 1e-5, 0.1)
            assert_close(dev.down(y2, y_ref.shape), y_ref, what="fwd with statistics (tuning %d)" % tuning)
            np.testing.assert_allclose(dev.down(sm, (K,)), mean_ref, rtol=1e-4, atol=1e-5)
            np.testing.assert_allclose(dev.down(si, (K,)), 1.0 / np.sqrt(var_ref + 1e-5), rtol=2e-4)
            np.testing.assert_allclose(dev.down(rm, (K,)), 0.1 * mean_ref, rtol=1e-4, atol=1e-5)      # running statistics updated exactly once
            dx0 = dev.up(np.full(x.size, 9.0, np.float32)); lib.lh_conv2d_bwd_data(dyd.ptr, wd.ptr, dx0.ptr, 0.0, *ints)
            assert_close(dev.down(dx0, x.shape), dx_ref, what="dx, overwriting (tuning %d)" % tuning)
            dx1 = dev.up(np.ones(x.size, np.float32)); lib.lh_conv2d_bwd_data(dyd.ptr, wd.ptr, dx1.ptr, 1.0, *ints)
            assert_close(dev.down(dx1, x.shape) - 1.0, dx_ref, what="dx, accumulating (tuning %d)" % tuning)
            dw1 = dev.zeros(w.size)
            lib.lh_conv2d_bwd_filter(xd.ptr, dyd.ptr, dw1.ptr, 0, 1.0, *ints); lib.lh_conv2d_bwd_filter(xd.ptr, dyd.ptr, dw1.ptr, 0, 1.0, *ints)
            assert_close(dev.down(dw1, w.shape) * 0.5, dw_ref, what="dw, accumulated twice (tuning %d)" % tuning)
            dw0 = dev.up(np.full(w.size, 5.0, np.float32)); lib.lh_conv2d_bwd_filter(xd.ptr, dyd.ptr, dw0.ptr, 0, 0.0, *ints)
            assert_close(dev.down(dw0, w.shape), dw_ref, what="dw, overwriting (tuning %d)" % tuning)
    finally:
        lib.lh_set_tuning(1)
    dev.check()


M32_SHAPES = [(16, 32, 28, 28, 32, 3, 3, 1, 1, 1, 1), (50, 10, 12, 12, 20, 5, 5, 1, 1, 0, 0), (8, 1, 41, 60, 32, 11, 5, 2, 2, 0, 0),
              (4, 32, 21, 30, 32, 5, 3, 2, 1, 2, 1),     # stride (2,1): the residue classes of the input gradient in one grouped launch
              (3, 7, 9, 9, 5, 3, 3, 1, 1, 1, 1), (2, 32, 16, 16, 16, 1, 1, 1, 1, 0, 0)]


@pytest.mark.parametrize("dims", M32_SHAPES, ids=lambda d: "x".join(map(str, d)))
@pytest.mark.parametrize("bias", [False, True], ids=["nobias", "bias"])
def test_conv_32_row_tiles(on_hip, dims, bias, monkeypatch):
    """Layers with at most 32 output (forward, filter gradient) or input (input gradient) channels on the 32 x 128 tile,
    forced through the library's test switch (the measured launch plan may be another one)."""
    monkeypatch.setenv("LH_FORCE_M32", "1")
    check_conv(Dev(on_hip), dims, bias)


@pytest.mark.parametrize("dims", [(8, 64, 28, 28, 64, 3, 3, 1, 1, 1, 1),      # filter gradient cut into 25 slices
                                  (4, 32, 15, 13, 40, 3, 3, 2, 2, 1, 1),      # strided, odd maps, with bias
                                  (16, 256, 7, 7, 512, 3, 3, 1, 1, 1, 1),     # few tiles over a long reduction (stream-K by default)
                                  (3, 10, 12, 12, 20, 5, 5, 1, 1, 0, 0)], ids=lambda d: "x".join(map(str, d)))
def test_conv_deterministic_mode(on_hip, dims):
    """lh_set_deterministic(1): the same results against the oracle (slices of a reduction added by a second kernel in a fixed
    order instead of by atomic adds, no stream-K), and two calls give the same bits."""
    dev = Dev(on_hip)
    on_hip.setDeterministic(True)
    try:
        assert dev.lib.lh_get_deterministic() == 1
        check_conv(dev, dims, bias=True)
        N, Cc, H, W, K, R, S, sH, sW, pH, pW = dims
        P, Q = (H + 2 * pH - R) // sH + 1, (W + 2 * pW - S) // sW + 1
        rng = np.random.RandomState(11)
        x = dev.up(rng.randn(N, Cc, H, W).astype(np.float32)); dy = dev.up(rng.randn(N, K, P, Q).astype(np.float32))
        w = dev.up((rng.randn(K, Cc, R, S) / np.sqrt(Cc * R * S)).astype(np.float32))
        runs = []
        for _ in range(2):
            gdw = dev.up(np.full((K, Cc, R, S), 0.5, np.float32)); gdb = dev.up(np.ones(K, np.float32)); gdx = dev.zeros(N * Cc * H * W)
            y = dev.zeros(N * K * P * Q)
            dev.lib.lh_conv2d_fwd(x.ptr, w.ptr, 0, y.ptr, *dims)
            dev.lib.lh_conv2d_bwd_data(dy.ptr, w.ptr, gdx.ptr, 0.0, *dims)
            dev.lib.lh_conv2d_bwd_filter(x.ptr, dy.ptr, gdw.ptr, gdb.ptr, 1.0, *dims); dev.check()
            runs.append([dev.down(y, (N, K, P, Q)), dev.down(gdx, (N, Cc, H, W)), dev.down(gdw, (K, Cc, R, S)), dev.down(gdb, (K,))])
        for a, b, what in zip(runs[0], runs[1], ("y", "dx", "dw", "db")):
            np.testing.assert_array_equal(a, b, err_msg=what)
    finally:
        on_hip.setDeterministic(False)
    assert dev.lib.lh_get_deterministic() == 0


@pytest.mark.parametrize("dims", [(5, 256, 7, 7, 64, 1, 1, 1, 1, 0, 0), (4, 16, 7, 7, 24, 3, 3, 1, 1, 1, 1), (2, 4, 21, 37, 32, 5, 3, 2, 1, 0, 1)],
                         ids=lambda d: "x".join(map(str, d)))
def test_filter_gradient_without_the_padded_reduction(on_hip, dims, monkeypatch):
    """Maps whose pixel count is not a multiple of 4: LH_NO_PADDED_REDUCTION=1 keeps the filter gradient on the 4-byte loads over the
    plain numbering of the reduction; both forms (the default one runs in test_conv_fwd_bwd) match the oracle."""
    monkeypatch.setenv("LH_NO_PADDED_REDUCTION", "1")
    check_conv(Dev(on_hip), dims, bias=True)


@pytest.mark.parametrize("dims", [(3, 10, 12, 12, 20, 5, 5, 1, 1, 0, 0), (2, 3, 13, 15, 12, 5, 5, 1, 1, 0, 0), (1, 1, 41, 30, 8, 11, 5, 2, 2, 0, 0)],
                         ids=lambda d: "x".join(map(str, d)))
def test_filter_gradient_of_unpadded_wide_filters_with_the_per_element_gather(on_hip, dims, monkeypatch):
    """LH_NO_SPLIT_GATHER=1 keeps the filter gradient of unpadded filters with rows of 5 taps and more on the loader that decodes every
    element of x per lane; both forms (the default one runs in test_conv_fwd_bwd) match the oracle."""
    monkeypatch.setenv("LH_NO_SPLIT_GATHER", "1")
    check_conv(Dev(on_hip), dims, bias=True)


@pytest.mark.parametrize("dims", [(8, 64, 28, 28, 128, 3, 3, 1, 1, 1, 1), (4, 256, 14, 14, 256, 1, 1, 1, 1, 0, 0), (6, 96, 15, 15, 160, 3, 3, 1, 1, 1, 1),
                                  (16, 32, 28, 28, 32, 3, 3, 1, 1, 1, 1), (8, 128, 28, 28, 256, 1, 1, 2, 2, 0, 0)], ids=lambda d: "x".join(map(str, d)))
def test_plain_tile_plans_give_the_same_bits(on_hip, dims, monkeypatch):
    """The launch plans whose tiles are finished by one block each (128x128, 64x128, 64x64, 32x128) add the same terms in the
    same order: forward output and input gradient are bit-identical whichever of them runs.  Deterministic mode relies on
    that when it keeps the measured choice among them."""
    dev = Dev(on_hip)
    lib = on_hip.lib
    N, Cc, H, W, K, R, S, sH, sW, pH, pW = dims
    P, Q = (H + 2 * pH - R) // sH + 1, (W + 2 * pW - S) // sW + 1
    rng = np.random.RandomState(91)
    xd = dev.up(rng.randn(N, Cc, H, W).astype(np.float32))
    wd = dev.up((rng.randn(K, Cc, R, S) / np.sqrt(Cc * R * S)).astype(np.float32))
    dyd = dev.up(rng.randn(N, K, P, Q).astype(np.float32))
    ny, nx = N * K * P * Q, N * Cc * H * W
    lib.lh_set_deterministic(1)
    try:
        outs = {}
        for plan in (3, 2, 1, 10):
            monkeypatch.setenv("LH_FORCE_PLAN", str(plan))
            y = dev.up(np.full(ny, 7.0, np.float32)); lib.lh_conv2d_fwd(xd.ptr, wd.ptr, 0, y.ptr, *dims)
            dx = dev.up(np.full(nx, 7.0, np.float32)); lib.lh_conv2d_bwd_data(dyd.ptr, wd.ptr, dx.ptr, 0.0, *dims)
            dev.check()
            outs[plan] = (dev.down(y, (ny,)).copy(), dev.down(dx, (nx,)).copy())
        for plan in (2, 1, 10):      # (a plan that does not fit the shape falls back to the rule's tile: equal all the same)
            np.testing.assert_array_equal(outs[plan][0], outs[3][0], err_msg="forward, plan %d against plan 3" % plan)
            np.testing.assert_array_equal(outs[plan][1], outs[3][1], err_msg="input gradient, plan %d against plan 3" % plan)
        assert np.abs(outs[3][0]).max() > 0.1 and np.abs(outs[3][1]).max() > 0.1
    finally:
        monkeypatch.delenv("LH_FORCE_PLAN", raising=False)
        lib.lh_set_deterministic(0)


SHARED_TAIL_SHAPES = [
    (64, 256, 14, 14, 256, 1, 1, 1, 1, 0, 0),     # 784 tiles of 64x64: one round of whole tiles and a tail of 272 (on 256 compute units)
    (16, 512, 7, 7, 512, 3, 3, 1, 1, 1, 1),       # fewer tiles than workers: every tile shared
    (4, 256, 14, 14, 256, 3, 3, 1, 1, 1, 1),      # few tiles over a long reduction
    (6, 96, 15, 15, 160, 3, 3, 1, 1, 1, 1),       # odd map: partial tiles in both directions
    (64, 64, 28, 28, 128, 1, 1, 1, 1, 0, 0),      # short reduction (4 slabs): below the plans' floor, falls back to the rule
    (8, 128, 28, 28, 256, 1, 1, 2, 2, 0, 0),      # stride 2: one class, 2x2 cells
]


@pytest.mark.parametrize("dims", SHARED_TAIL_SHAPES, ids=lambda d: "x".join(map(str, d)))
@pytest.mark.parametrize("plan", [13, 14, 15], ids=["tiles64x64", "tiles64x128", "tiles128x128"])
def test_whole_tiles_and_slices_of_the_last_ones(on_hip, dims, plan, monkeypatch):
    """The launch plans that cut the last tiles (what is left over a multiple of the compute units) into slices along the
    reduction, one block each; the slice that arrives last adds them up and finishes the tile: forward with bias and with the clamp, input gradient overwriting and accumulating,
    against the whole-tile plan; two runs give the same bits (nothing is combined with atomic adds)."""
    dev = Dev(on_hip)
    lib = on_hip.lib
    N, Cc, H, W, K, R, S, sH, sW, pH, pW = dims
    P, Q = (H + 2 * pH - R) // sH + 1, (W + 2 * pW - S) // sW + 1
    rng = np.random.RandomState(97)
    xd = dev.up(rng.randn(N, Cc, H, W).astype(np.float32))
    wd = dev.up((rng.randn(K, Cc, R, S) / np.sqrt(Cc * R * S)).astype(np.float32))
    bd = dev.up(rng.randn(K).astype(np.float32))
    dyd = dev.up(rng.randn(N, K, P, Q).astype(np.float32))
    ny, nx = N * K * P * Q, N * Cc * H * W

    def run(p):
        monkeypatch.setenv("LH_FORCE_PLAN", str(p))
        y = dev.up(np.full(ny, 7.0, np.float32)); lib.lh_conv2d_fwd(xd.ptr, wd.ptr, bd.ptr, y.ptr, *dims)
        dx0 = dev.up(np.full(nx, 7.0, np.float32)); lib.lh_conv2d_bwd_data(dyd.ptr, wd.ptr, dx0.ptr, 0.0, *dims)
        dx1 = dev.up(np.ones(nx, np.float32)); lib.lh_conv2d_bwd_data(dyd.ptr, wd.ptr, dx1.ptr, 1.0, *dims)
        dev.check()
        return [dev.down(y, (ny,)).copy(), dev.down(dx0, (nx,)).copy(), dev.down(dx1, (nx,)).copy() - 1.0]
    try:
        want = run(3)
        got = run(plan)
        again = run(plan)
    finally:
        monkeypatch.delenv("LH_FORCE_PLAN", raising=False)
    for name, g, a, w_ in zip(("forward", "input gradient", "input gradient, accumulating"), got, again, want):
        assert_close(g, w_, rtol=2e-5, what="%s, plan %d" % (name, plan))
        if name != "input gradient, accumulating":
            np.testing.assert_array_equal(g, a, err_msg="%s: two runs of plan %d" % (name, plan))
    assert np.abs(want[0]).max() > 0.1 and np.abs(want[1]).max() > 0.1


@pytest.mark.parametrize("dims", [(64, 256, 14, 14, 256, 1, 1, 1, 1, 0, 0), (16, 512, 7, 7, 512, 3, 3, 1, 1, 1, 1), (6, 96, 15, 15, 160, 3, 3, 1, 1, 1, 1)],
                         ids=lambda d: "x".join(map(str, d)))
@pytest.mark.parametrize("tile", [5, 6, 7], ids=["tiles64x64", "tiles64x128", "tiles128x128"])
def test_sliced_last_tiles_leave_the_same_batchnorm_statistics(on_hip, dims, tile, monkeypatch):
    """The forward launch that leaves batch-norm statistics behind, with its last tiles cut along the reduction: the block that
    finishes a sliced tile has the complete sums, so output and statistics are those of the whole-tile launch (to rounding:
    the slices are added in slice order) and two runs agree bit for bit."""
    dev = Dev(on_hip)
    lib = on_hip.lib
    N, Cc, H, W, K, R, S, sH, sW, pH, pW = dims
    P, Q = (H + 2 * pH - R) // sH + 1, (W + 2 * pW - S) // sW + 1
    rng = np.random.RandomState(101)
    xd = dev.up(rng.randn(N, Cc, H, W).astype(np.float32))
    wd = dev.up((rng.randn(K, Cc, R, S) / np.sqrt(Cc * R * S)).astype(np.float32))
    ny = N * K * P * Q

    def run(f):
        monkeypatch.setenv("LH_FORCE_STATS_TILE", str(f))
        y = dev.up(np.full(ny, 7.0, np.float32)); sm = dev.zeros(K); si = dev.zeros(K); rm = dev.zeros(K); rv = dev.up(np.ones(K, np.float32))
        lib.lh_conv2d_fwd_bnstats(xd.ptr, wd.ptr, 0, y.ptr, *dims, sm.ptr, si.ptr, rm.ptr, rv.ptr, 1e-5, 0.1)
        dev.check()
        return [dev.down(y, (ny,)).copy(), dev.down(sm, (K,)).copy(), dev.down(si, (K,)).copy(), dev.down(rm, (K,)).copy(), dev.down(rv, (K,)).copy()]
    try:
        want = run(3)
        got = run(tile)
        again = run(tile)
    finally:
        monkeypatch.delenv("LH_FORCE_STATS_TILE", raising=False)
    assert_close(got[0], want[0], rtol=2e-5, what="output")
    for i, name in ((1, "mean"), (2, "1/std"), (3, "running mean"), (4, "running variance")):
        np.testing.assert_allclose(got[i], want[i], rtol=2e-5, atol=2e-6, err_msg=name)
    for g, a in zip(got, again):
        np.testing.assert_array_equal(g, a)
