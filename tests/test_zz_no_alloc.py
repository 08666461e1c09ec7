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


def test_static_table_update_recorded_into_a_graph_carries_its_own_table(on_hip):
    """The table array is shared by every call on the GPU.  A call recorded into a graph records its table writes with it, and
    an eager call never trusts what an earlier call left in the array: eager on set A, recording on set A, eager on set B,
    a replay (set A again), eager on set A: every update lands on the tensors it was given, bit for bit what
    lh_multi_momentum gives for the same sequence."""
    be, lib = on_hip, on_hip.lib
    rng = np.random.RandomState(9)
    size_a, size_b = [300, 4096 * 3 + 5, 17, 70000], [5, 9000]
    host = {k: [(rng.randn(n).astype(np.float32), rng.randn(n).astype(np.float32), rng.randn(n).astype(np.float32)) for n in sizes]
            for k, sizes in (("a", size_a), ("b", size_b))}

    def run(static):
        bufs = {k: [(be.fromHost(x.copy()), be.fromHost(d.copy()), be.fromHost(v.copy()), x.size) for x, d, v in host[k]] for k in host}
        tabs = {k: _tables(bufs[k]) for k in bufs}
        entry = lib.lh_multi_momentum_static if static else lib.lh_multi_momentum
        def call(k):
            entry(*tabs[k], 0.1, 0.9, 2.0, 0); _lib.check()
        def regrad(k, scale):
            for (x, d, v), b in zip(host[k], bufs[k]):
                be.upload(b[1], d * np.float32(scale))
        call("a")                                   # eager, set A
        regrad("a", 2.0)
        graph = None
        if static:
            be.sync()
            be.captureBegin()
            call("a")                               # recorded, not run
            graph = be.captureEnd()
        call("b")                                   # eager, set B: the array now holds B's entries
        if static:
            be.graphLaunch(graph)                   # the replay writes A's entries itself
        else:
            call("a")
        regrad("a", 3.0)
        call("a")                                   # eager, set A again
        be.sync()
        out = {k: [tuple(be.toHost(b[j], b[3]) for j in range(3)) for b in bufs[k]] for k in bufs}
        if graph is not None:
            be.graphDestroy(graph)
        return out
    want, got = run(False), run(True)
    for k in want:
        for t, (w, g) in enumerate(zip(want[k], got[k])):
            for name, a, b in zip(("x", "d", "v"), g, w):
                np.testing.assert_array_equal(a, b, err_msg="set %s tensor %d %s" % (k, t, name))
