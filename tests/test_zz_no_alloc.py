"""lh_multi_momentum_static: the multi-tensor momentum update for callers that cannot allocate (a fixed device table written by
launch-argument kernels) against lh_multi_momentum, through the C ABI.  Two calls in a row, the second over fewer and smaller
tensors, so entries the first call left in the shared table must not be read; then the first set again (the table is rewritten).
Results must be bit-identical: both entry points run the same update kernel over the same chunk decomposition."""
import ctypes as C

import numpy as np
import pytest

from lantern_amd import _lib

pytestmark = pytest.mark.gpu


def _tables(bufs):
    k = len(bufs)
    return (k, (C.c_void_p * k)(*[b[0].ptr for b in bufs]), (C.c_void_p * k)(*[b[1].ptr for b in bufs]),
            (C.c_void_p * k)(*[b[2].ptr for b in bufs]), (C.c_int64 * k)(*[b[3] for b in bufs]))


def _run(be, entry, sizes, seed, steps, lr, mu, clip, nesterov):
    """Uploads fresh x, d, v for `sizes`, applies `steps` updates through `entry` (new gradients each step), returns x, d, v."""
    rng = np.random.RandomState(seed)
    host = [(rng.randn(n).astype(np.float32), (rng.randn(n) * 3).astype(np.float32), rng.randn(n).astype(np.float32)) for n in sizes]
    bufs = [(be.fromHost(np.ascontiguousarray(x)), be.fromHost(np.ascontiguousarray(d)), be.fromHost(np.ascontiguousarray(v)), n) for (x, d, v), n in zip(host, sizes)]
    k, xs, ds, vs, ns = _tables(bufs)
    for step in range(steps):
        getattr(be.lib, entry)(k, xs, ds, vs, ns, lr, mu, clip, int(nesterov)); _lib.check()
        if step + 1 < steps:
            for (x, d, v), b in zip(host, bufs):
                be.upload(b[1], d * np.float32(step + 2))
    be.sync()
    return [tuple(be.toHost(b[j], b[3], np.float32) for j in range(3)) for b in bufs]


def test_static_table_update_matches_the_allocating_one_on_two_calls_in_a_row(on_hip):
    be = on_hip
    big = [1, 7, 64, 4096, 4097, 1000, 9 * 64 * 64, 2048 * 1000 + 3] + [257 + 3 * i for i in range(150)]      # 158 tensors: three writer launches
    small = [5, 4096 * 2 + 1, 333]                                                                          # fewer and smaller
    cases = ((big, 1, False), (small, 2, True), (big, 3, True))
    wants = [_run(be, "lh_multi_momentum", sizes, seed, 2, 0.1, 0.9, 2.0, nesterov) for sizes, seed, nesterov in cases]
    gots = [_run(be, "lh_multi_momentum_static", sizes, seed, 2, 0.1, 0.9, 2.0, nesterov) for sizes, seed, nesterov in cases]      # in a row
    for (sizes, _, _), got, want in zip(cases, gots, wants):
        assert len(got) == len(want) == len(sizes)
        for t, (g, w) in enumerate(zip(got, want)):
            for name, a, b in zip(("x", "d", "v"), g, w):
                np.testing.assert_array_equal(a, b, err_msg="tensor %d (%d elements) %s" % (t, sizes[t], name))
            assert not g[1].any()                                   # the gradient is cleared


def test_static_table_rejects_more_tensors_than_it_holds(on_hip):
    be = on_hip
    n = 4097
    buf = be.fromHost(np.ascontiguousarray(np.zeros(4, np.float32)))
    ptrs = (C.c_void_p * n)(*[buf.ptr] * n); ns = (C.c_int64 * n)(*[4] * n)
    be.lib.lh_multi_momentum_static(n, ptrs, ptrs, ptrs, ns, 0.1, 0.9, 1.0, 0)
    with pytest.raises(_lib.LanternHipError, match="at most 4096"):
        _lib.check()
