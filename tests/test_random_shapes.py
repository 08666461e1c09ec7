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
