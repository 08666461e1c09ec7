"""Helpers shared by the parity tests."""
import ctypes as C

import numpy as np


def assert_close(got, want, rtol=1e-4, what=""):
    """|got - want| <= rtol * (|want| + rms(want)) element-wise.

    The north-star tolerance is 1e-4 relative with reduction order free to differ; sums of
    products cancel, so the scale of an element's error is the typical magnitude of the output
    (its rms), not the magnitude of that one element.
    """
    got = np.asarray(got, dtype=np.float64); want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, "%s shape %s vs %s" % (what, got.shape, want.shape)
    assert np.isfinite(got).all(), "%s: non-finite values in result" % what
    rms = float(np.sqrt(np.mean(want * want))) if want.size else 0.0
    tol = rtol * (np.abs(want) + rms) + 1e-30
    err = np.abs(got - want)
    bad = err > tol
    if bad.any():
        i = np.unravel_index(np.argmax(err / tol), err.shape)
        raise AssertionError("%s: %d of %d elements off; worst at %s: got %.9g want %.9g (err %.3g, tol %.3g)"
                             % (what, int(bad.sum()), err.size, i, got[i], want[i], err[i], tol[i]))


class Dev:
    """Thin helper over BackendHIP for tests that call the C ABI directly."""

    def __init__(self, be):
        self.be = be
        self.lib = be.lib

    def up(self, arr):
        return self.be.fromHost(np.ascontiguousarray(arr))

    def zeros(self, n):
        return self.be.mallocArray(n)

    def down(self, buf, shape, dtype=np.float32):
        return self.be.toHost(buf, int(np.prod(shape)), dtype).reshape(shape)

    def check(self):
        from lantern_amd import _lib
        _lib.check()


def cptr(arr):
    return C.c_void_p(arr.ctypes.data)
