"""The library's deferred work, through the C ABI: a program that issues one call per Backend trait method (what
scala/TensorDslHIP.scala emits: lh_malloc for every buffer, lh_conv2d_fwd, lh_bn_train_fwd, lh_unary(LH_RELU) in place,
lh_bcast_op(LH_ADD), their gradients with beta = 1, one lh_momentum per parameter) must give, bit for bit in deterministic
mode, what the hand-fused entry points give (lh_conv2d_fwd_bn_apply, lh_bn_bwd_relu, lh_bn_bwd_add_relu,
lh_multi_momentum on buffers the caller cleared), and lh_fusion_stats must show that the fused kernels did run.
Also the bookkeeping's edge cases: a block read before written reads zero, a slice of an untouched block, results a fused
chain did not store read back later, a rewind in between, fusion switched off."""
import ctypes as C

import numpy as np
import pytest

from lantern_amd import _lib
from lantern_amd import backend as B
from tests.util import Dev, assert_close

pytestmark = pytest.mark.gpu

F = C.c_float
RELU, ADD = B.RELU, B.ADD


def _stats(lib):
    a = (C.c_int64 * 8)()
    lib.lh_fusion_stats(a, 8)
    return np.array(list(a), dtype=np.int64)


def _ints(*v):
    return (C.c_int * len(v))(*v)


class Prog:
    """A few helpers over the raw library for programs written the way generated code is."""

    def __init__(self, be):
        self.be, self.lib, self.dev = be, be.lib, Dev(be)

    def malloc(self, n):                      # what mallocArray emits: zero-filled arena memory
        p = self.lib.lh_malloc(4 * int(n)); _lib.check()
        return p

    def up(self, arr):
        arr = np.ascontiguousarray(arr, np.float32)
        p = self.lib.lh_malloc_uninit(arr.nbytes); _lib.check()
        self.lib.lh_h2d(p, arr.ctypes.data, arr.nbytes); _lib.check()
        return p

    def down(self, p, shape):
        out = np.empty(int(np.prod(shape)), np.float32)
        self.lib.lh_d2h(out.ctypes.data, p, out.nbytes); _lib.check()
        return out.reshape(shape)


@pytest.fixture
def prog(on_hip):
    on_hip.setDeterministic(True)
    on_hip.lib.lh_set_side_stream(0)
    yield Prog(on_hip)
    on_hip.lib.lh_set_fusion(1)
    on_hip.lib.lh_set_side_stream(1)
    on_hip.setDeterministic(False)


# geometry large enough that every activation is more than 1 MiB (the blocks whose clearing is put off)
N, CI, H, K = 8, 64, 28, 64
NX, NY = N * CI * H * H, N * K * H * H


def _inputs(seed):
    rng = np.random.RandomState(seed)
    return dict(x=rng.randn(N, CI, H, H).astype(np.float32), w=(rng.randn(K, CI, 3, 3) * 0.05).astype(np.float32),
                gamma=(1.0 + 0.1 * rng.randn(K)).astype(np.float32), beta=(0.1 * rng.randn(K)).astype(np.float32),
                sc=rng.randn(N, K, H, H).astype(np.float32), dout=rng.randn(N, K, H, H).astype(np.float32))


def _conv_args():
    return (N, CI, H, H, K, 3, 3, 1, 1, 1, 1)


def _trait_conv_bn_relu(pg, inp, join):
    """conv -> batchNorm -> [+ shortcut] -> relu(inPlace) and its backward, one call per trait method."""
    lib = pg.lib
    x, w, gamma, beta = pg.up(inp["x"]), pg.up(inp["w"]), pg.up(inp["gamma"]), pg.up(inp["beta"])
    sc = pg.up(inp["sc"])
    rm, rv = pg.malloc(K), pg.malloc(K)
    dgamma, dbeta, dw, dx, dsc = pg.malloc(K), pg.malloc(K), pg.malloc(K * CI * 9), pg.malloc(NX), pg.malloc(NY)
    y = pg.malloc(NY); lib.lh_conv2d_fwd(x, w, 0, y, *_conv_args())
    dy = pg.malloc(NY)                                                         # TensorR(y).d
    t = pg.malloc(NY); sm, si = pg.malloc(K), pg.malloc(K)
    lib.lh_bn_train_fwd(y, gamma, beta, rm, rv, t, sm, si, N, K, H * H, 1e-5, 0.1)
    dt = pg.malloc(NY)
    if join:
        dims = _ints(N, K, H, H)
        out = pg.malloc(NY); lib.lh_bcast_op(ADD, t, dims, sc, dims, out, dims, 4)
        dout = pg.malloc(NY)
    else:
        out, dout = t, dt
    lib.lh_unary(RELU, out, out, NY, 0.0, 0.0)
    _lib.check()
    # the loss's gradient arrives in dout; then the tape in reverse
    g = np.ascontiguousarray(inp["dout"]); lib.lh_h2d(dout, g.ctypes.data, g.nbytes)
    lib.lh_unary_grad(RELU, out, out, dout, dout, NY, 1, 0.0, 0.0)
    if join:
        lib.lh_bcast_op_grad(ADD, t, dt, dims, 0, sc, dsc, dims, 0, dout, dims, 4)
    lib.lh_bn_bwd(y, dt, gamma, sm, si, dy, 1.0, dgamma, dbeta, N, K, H * H)
    lib.lh_conv2d_bwd_data(dy, w, dx, 1.0, *_conv_args())
    lib.lh_conv2d_bwd_filter(x, dy, dw, 0, 1.0, *_conv_args())
    _lib.check()
    res = dict(out=pg.down(out, (NY,)), dx=pg.down(dx, (NX,)), dw=pg.down(dw, (K * CI * 9,)), dgamma=pg.down(dgamma, (K,)), dbeta=pg.down(dbeta, (K,)),
               rm=pg.down(rm, (K,)), rv=pg.down(rv, (K,)))
    if join:
        res["dsc"] = pg.down(dsc, (NY,))
    # read last: what a fused chain does not store
    res["late_t"] = pg.down(t, (NY,)) if join else None
    res["late_dt"] = pg.down(dt, (NY,))
    res["late_dout"] = pg.down(dout, (NY,))
    return res


def _fused_conv_bn_relu(pg, inp, join):
    """The same through the hand-fused entry points, on buffers this program clears itself."""
    lib = pg.lib
    x, w, gamma, beta = pg.up(inp["x"]), pg.up(inp["w"]), pg.up(inp["gamma"]), pg.up(inp["beta"])
    sc = pg.up(inp["sc"])
    z = lambda n: pg.up(np.zeros(n, np.float32))
    rm, rv, dgamma, dbeta = z(K), z(K), z(K), z(K)
    dw, dx, dsc, dy = z(K * CI * 9), z(NX), z(NY), z(NY)
    y, out, sm, si = z(NY), z(NY), z(K), z(K)
    lib.lh_conv2d_fwd_bn_apply(x, w, 0, y, *_conv_args(), gamma, beta, sm, si, rm, rv, 1e-5, 0.1, sc if join else 0, out, 1)
    dout = pg.up(inp["dout"])
    if join:
        lib.lh_bn_bwd_add_relu(y, out, dout, gamma, sm, si, dy, 0.0, dsc, 0.0, dgamma, dbeta, N, K, H * H)
    else:
        lib.lh_bn_bwd_relu(y, out, dout, gamma, beta, sm, si, dy, 0.0, dgamma, dbeta, N, K, H * H)
    lib.lh_conv2d_bwd_data(dy, w, dx, 0.0, *_conv_args())
    lib.lh_conv2d_bwd_filter(x, dy, dw, 0, 0.0, *_conv_args())
    _lib.check()
    res = dict(out=pg.down(out, (NY,)), dx=pg.down(dx, (NX,)), dw=pg.down(dw, (K * CI * 9,)), dgamma=pg.down(dgamma, (K,)), dbeta=pg.down(dbeta, (K,)),
               rm=pg.down(rm, (K,)), rv=pg.down(rv, (K,)))
    if join:
        res["dsc"] = pg.down(dsc, (NY,))
    return res


@pytest.mark.parametrize("join", [False, True], ids=["conv_bn_relu", "residual_join"])
def test_trait_call_sequence_gives_the_bits_of_the_fused_entry_points(prog, join):
    inp = _inputs(11 + join)
    s0 = _stats(prog.lib)
    got = _trait_conv_bn_relu(prog, inp, join)
    s1 = _stats(prog.lib)
    assert s1[0] - s0[0] == 1 and s1[1] - s0[1] == 1, "one forward and one backward chain were to be fused: %s" % (s1 - s0)
    assert s1[3] - s0[3] >= 4, "gradient buffers nobody had touched were to be written, not cleared and added into: %s" % (s1 - s0)
    want = _fused_conv_bn_relu(prog, inp, join)
    for k, v in want.items():
        np.testing.assert_array_equal(got[k], v, err_msg=k)
    # what the chain left out is there when somebody asks: relu_grad in place masks the gradient buffer, add_grad hands the
    # masked gradient to the batch norm's output gradient, and the batch norm's own output under a join
    g = inp["dout"].ravel() * (want["out"] > 0)
    np.testing.assert_array_equal(got["late_dout"], g)
    np.testing.assert_array_equal(got["late_dt"], g)
    if join:
        lib = prog.lib
        prog.lib.lh_set_fusion(0)
        plain = _trait_conv_bn_relu(prog, inp, join)
        # (to rounding: with fusion off the statistics come from a pass over the convolution's output, not from its epilogue)
        np.testing.assert_allclose(got["late_t"], plain["late_t"], rtol=1e-5, atol=1e-5)
        assert s1[5] - s0[5] >= 2, "reading them was to run their recipes: %s" % (s1 - s0)


@pytest.mark.parametrize("join", [False, True], ids=["conv_bn_relu", "residual_join"])
def test_trait_call_sequence_with_fusion_off_agrees(prog, join):
    inp = _inputs(21 + join)
    got = _trait_conv_bn_relu(prog, inp, join)
    prog.lib.lh_set_fusion(0)
    s0 = _stats(prog.lib)
    plain = _trait_conv_bn_relu(prog, inp, join)
    assert (_stats(prog.lib) == s0).all(), "with fusion off nothing is put off"
    for k, v in plain.items():
        if v is not None:
            assert_close(got[k], v, rtol=1e-5, what=k)


def test_gathered_momentum_calls_give_the_bits_of_the_multi_tensor_call(prog):
    lib = prog.lib
    rng = np.random.RandomState(5)
    sizes = [7, 4096, 300000, 64, 1 << 20, 33]
    host = [(rng.randn(n).astype(np.float32), rng.randn(n).astype(np.float32), rng.randn(n).astype(np.float32)) for n in sizes]

    def run(gathered):
        bufs = [(prog.up(x), prog.up(d), prog.up(v)) for x, d, v in host]
        if gathered:
            s0 = _stats(lib)
            for (x, d, v), n in zip(bufs, sizes):
                lib.lh_momentum(x, d, v, 0.1, 0.9, 0.5, 0, n)
            lib.lh_flush_deferred()
            assert _stats(lib)[2] - s0[2] == len(sizes)
        else:
            k = len(sizes)
            arr = lambda i: (C.c_void_p * k)(*[b[i] for b in bufs])
            lib.lh_multi_momentum(k, arr(0), arr(1), arr(2), (C.c_int64 * k)(*sizes), 0.1, 0.9, 0.5, 0)
        _lib.check()
        return [(prog.down(x, (n,)), prog.down(d, (n,)), prog.down(v, (n,))) for (x, d, v), n in zip(bufs, sizes)]
    for a, b in zip(run(True), run(False)):
        for u, v in zip(a, b):
            np.testing.assert_array_equal(u, v)
    # different hyper-parameters do not share a launch, and the plain kernel agrees with the gathered one
    bufs = [(prog.up(x), prog.up(d), prog.up(v)) for x, d, v in host[:2]]
    lib.lh_momentum(*bufs[0], 0.1, 0.9, 0.5, 0, sizes[0])
    lib.lh_momentum(*bufs[1], 0.2, 0.9, 0.5, 1, sizes[1])
    got = [prog.down(bufs[i][0], (sizes[i],)) for i in range(2)]
    lib.lh_set_fusion(0)
    bufs = [(prog.up(x), prog.up(d), prog.up(v)) for x, d, v in host[:2]]
    lib.lh_momentum(*bufs[0], 0.1, 0.9, 0.5, 0, sizes[0])
    lib.lh_momentum(*bufs[1], 0.2, 0.9, 0.5, 1, sizes[1])
    for i in range(2):
        np.testing.assert_array_equal(got[i], prog.down(bufs[i][0], (sizes[i],)))


def test_untouched_blocks_read_zero_whoever_asks(prog):
    """lh_malloc's promise (Tensor.zeros relies on it) with the clearing put off: a read-back, an operator that reads, an
    operator that adds into a slice, a rewind and a second allocation of the same memory."""
    lib = prog.lib
    n = 1 << 20                                   # 4 MiB
    mark = lib.lh_mark()
    dirty = lib.lh_malloc_uninit(4 * n); lib.lh_fill(dirty, F(7.0), n); _lib.check()
    lib.lh_rewind(mark)
    a = prog.malloc(n)                             # the same memory, now promised zero
    assert a == dirty
    assert not prog.down(a, (n,)).any()            # read-back
    lib.lh_rewind(mark)
    lib.lh_fill(dirty, F(7.0), n)
    a = prog.malloc(n); b = prog.malloc(n)
    lib.lh_geam(a, F(1.0), a, F(1.0), b, n)        # an operator that reads a and overwrites b
    assert not prog.down(b, (n,)).any()
    # adding into a slice of an untouched block: the rest of the block still reads zero
    c = prog.malloc(n)
    ones = prog.up(np.ones(1000, np.float32))
    lib.lh_geam(c + 4 * 5000, F(1.0), ones, F(2.0), c + 4 * 5000, 1000)
    got = prog.down(c, (n,))
    assert (got[5000:6000] == 2.0).all() and not got[:5000].any() and not got[6000:].any()
    # a gradient entry point with beta = 1 on an untouched block behaves as on a cleared one
    d = prog.malloc(n)
    lib.lh_unary_grad(RELU, ones, ones, ones, d + 4 * 100, 1000, 0, 0.0, 0.0)      # a slice: cleared, then accumulated
    got = prog.down(d, (n,))
    assert (got[100:1100] == 1.0).all() and not got[:100].any() and not got[1100:].any()
    # popped and rewound blocks are forgotten, not cleared later by accident
    lib.lh_rewind(mark)
    e = lib.lh_malloc_uninit(4 * n); lib.lh_fill(e, F(3.0), n)
    assert (prog.down(e, (n,)) == 3.0).all()
    lib.lh_rewind(mark)
    _lib.check()


def test_parked_calls_run_in_program_order_around_other_calls(prog):
    """Whatever is parked is launched before any call that does not continue its chain: a read-back, a copy, an allocation
    in between, lh_sync, a rewind."""
    lib = prog.lib
    inp = _inputs(31)
    x, w, gamma, beta = prog.up(inp["x"]), prog.up(inp["w"]), prog.up(inp["gamma"]), prog.up(inp["beta"])
    # conv parked, then read: the convolution has run
    y = prog.malloc(NY); lib.lh_conv2d_fwd(x, w, 0, y, *_conv_args())
    y_host = prog.down(y, (NY,))
    assert np.abs(y_host).max() > 0.1
    # conv + bn parked, then a copy of the batch norm's output: both have run (the statistics taken from the convolution)
    rm, rv, sm, si = prog.malloc(K), prog.malloc(K), prog.malloc(K), prog.malloc(K)
    y2 = prog.malloc(NY); lib.lh_conv2d_fwd(x, w, 0, y2, *_conv_args())
    spare = prog.malloc(NY)                         # allocations in between do not end a chain
    t = prog.malloc(NY); lib.lh_bn_train_fwd(y2, gamma, beta, rm, rv, t, sm, si, N, K, H * H, 1e-5, 0.1)
    cp = prog.malloc(NY); lib.lh_d2d(cp, t, 4 * NY)
    t_host = prog.down(cp, (NY,)).reshape(N, K, H * H)
    yh = y_host.reshape(N, K, H * H).astype(np.float64)
    mu = yh.mean((0, 2), keepdims=True); var = yh.var((0, 2), keepdims=True)
    want = inp["gamma"].reshape(1, K, 1) * (yh - mu) / np.sqrt(var + 1e-5) + inp["beta"].reshape(1, K, 1)
    np.testing.assert_allclose(t_host, want, rtol=1e-4, atol=1e-4)
    assert not prog.down(spare, (NY,)).any()
    # relu in place on something that is NOT the parked chain's output: the chain runs unfused, then the relu
    t2 = prog.malloc(NY); lib.lh_bn_train_fwd(y2, gamma, beta, rm, rv, t2, sm, si, N, K, H * H, 1e-5, 0.1)
    lib.lh_unary(RELU, cp, cp, NY, 0.0, 0.0)
    np.testing.assert_array_equal(prog.down(cp, (NY,)), np.maximum(t_host.ravel(), 0))
    np.testing.assert_allclose(prog.down(t2, (NY,)), t_host.ravel(), rtol=1e-5, atol=1e-5)      # statistics from a pass of their own here
    _lib.check()


def _trait_conv_bias_relu(pg, inp, geom, side=False):
    """conv(+ bias) -> relu(inPlace) and its backward, one call per trait method: what a network without batch norms
    (SqueezeNet's fire modules) issues.  The filter gradient goes first, as the backends issue it when there is a bias."""
    lib = pg.lib
    n, c, h, k, r, pad = geom
    args = (n, c, h, h, k, r, r, 1, 1, pad, pad)
    p = h + 2 * pad - r + 1
    nx, ny = n * c * h * h, n * k * p * p
    x, w, b = pg.up(inp["x"]), pg.up(inp["w"]), pg.up(inp["b"])
    dw, db, dx = pg.malloc(k * c * r * r), pg.malloc(k), pg.malloc(nx)
    y = pg.malloc(ny); lib.lh_conv2d_fwd(x, w, b, y, *args)
    dy = pg.malloc(ny)
    lib.lh_unary(RELU, y, y, ny, 0.0, 0.0)
    _lib.check()
    g = np.ascontiguousarray(inp["dout"]); lib.lh_h2d(dy, g.ctypes.data, g.nbytes)
    lib.lh_unary_grad(RELU, y, y, dy, dy, ny, 1, 0.0, 0.0)
    if side: lib.lh_side_begin()
    lib.lh_conv2d_bwd_filter(x, dy, dw, db, 1.0, *args)
    if side: lib.lh_side_end()
    lib.lh_conv2d_bwd_data(dy, w, dx, 1.0, *args)
    _lib.check()
    return dict(y=pg.down(y, (ny,)), dy=pg.down(dy, (ny,)), dw=pg.down(dw, (k * c * r * r,)), db=pg.down(db, (k,)), dx=pg.down(dx, (nx,)))


def _bias_inputs(seed, geom):
    n, c, h, k, r, pad = geom
    p = h + 2 * pad - r + 1
    rng = np.random.RandomState(seed)
    return dict(x=rng.randn(n, c, h, h).astype(np.float32), w=(rng.randn(k, c, r, r) / np.sqrt(c * r * r)).astype(np.float32),
                b=(0.3 * rng.randn(k)).astype(np.float32), dout=rng.randn(n, k, p, p).astype(np.float32))


@pytest.mark.parametrize("geom", [(8, 64, 28, 64, 3, 1), (64, 16, 16, 64, 1, 0), (4, 48, 9, 24, 3, 0)], ids=["3x3_28", "1x1_16", "ragged"])
def test_conv_bias_relu_and_its_gradient_run_as_two_fewer_kernels_with_the_same_bits(prog, geom):
    inp = _bias_inputs(41, geom)
    s0 = _stats(prog.lib)
    got = _trait_conv_bias_relu(prog, inp, geom)
    s1 = _stats(prog.lib)
    assert s1[0] - s0[0] == 1 and s1[1] - s0[1] == 1, "the clamp was to ride in the convolution's epilogue and the mask in the bias sums: %s" % (s1 - s0)
    prog.lib.lh_set_fusion(0)
    plain = _trait_conv_bias_relu(prog, inp, geom)
    for k, v in plain.items():
        np.testing.assert_array_equal(got[k], v, err_msg=k)
    assert (got["y"] >= 0).all() and (got["y"] == 0).any()
    np.testing.assert_array_equal(got["dy"], inp["dout"].ravel() * (got["y"] > 0))


def test_conv_bias_relu_where_partial_sums_are_added_and_on_the_side_stream(on_hip):
    """Default mode: a long reduction over few tiles runs with several blocks per tile adding their partial sums, so the
    clamp cannot ride in the epilogue everywhere (it is applied by a pass behind the launch), and the filter gradient, bias
    sums included, is issued on the side stream with the relu_grad still parked."""
    pg = Prog(on_hip)
    geom = (16, 1024, 16, 256, 3, 1)
    inp = _bias_inputs(43, geom)
    got = _trait_conv_bias_relu(pg, inp, geom, side=True)
    on_hip.lib.lh_set_fusion(0)
    try:
        plain = _trait_conv_bias_relu(pg, inp, geom, side=True)
    finally:
        on_hip.lib.lh_set_fusion(1)
    assert (got["y"] >= 0).all() and (got["y"] == 0).any()
    for k, v in plain.items():
        assert_close(got[k], v, rtol=2e-5, what=k)
    # the mask is a function of y's sign, and a sum that lands within rounding of zero may fall on either side
    agree = (got["y"] > 0) == (plain["y"] > 0)
    assert agree.mean() > 0.9999


def test_concat_of_more_tensors_than_one_launch_takes(prog):
    lib = prog.lib
    rng = np.random.RandomState(47)
    outer, inner = 6, 35
    sizes = [3, 1, 0, 7, 2, 5, 4]
    parts = [rng.randn(outer, s, inner).astype(np.float32) for s in sizes]
    ptrs = [prog.up(p) if p.size else 0 for p in parts]
    row = sum(sizes)
    out = prog.malloc(outer * row * inner)
    lib.lh_concat(len(sizes), (C.c_void_p * len(sizes))(*ptrs), _ints(*sizes), out, outer, inner); _lib.check()
    want = np.concatenate(parts, axis=1)
    np.testing.assert_array_equal(prog.down(out, want.shape), want)
    # gradient: accumulated into some, overwriting others, skipped for one
    dout = rng.randn(*want.shape).astype(np.float32)
    d_out = prog.up(dout)
    init = [rng.randn(*p.shape).astype(np.float32) for p in parts]
    dptrs = [prog.up(a) if a.size else 0 for a in init]
    dptrs[3] = 0
    betas = [1.0, 0.0, 1.0, 1.0, 0.0, 1.0, 1.0]
    lib.lh_concat_grad_beta(len(sizes), (C.c_void_p * len(sizes))(*dptrs), (F * len(sizes))(*betas), _ints(*sizes), d_out, outer, inner); _lib.check()
    off = 0
    for t, s in enumerate(sizes):
        if s and dptrs[t]:
            np.testing.assert_array_equal(prog.down(dptrs[t], init[t].shape), betas[t] * init[t] + dout[:, off:off + s, :], err_msg="tensor %d" % t)
        off += s


def test_kept_filter_copies_end_with_every_write_of_the_filter(prog):
    """The convolution kernels read copies of the filter in layouts of their own; the library keeps a copy while nothing
    writes the filter.  Every way of writing it (an upload, an operator in place, a fill, the gathered optimizer launch, a
    rewind that hands its memory to another tensor) must end the copy: each time the convolution and its input gradient,
    stride 1 and stride 2, are compared with what the library computes with nothing kept (lh_set_fusion(0))."""
    lib = prog.lib
    rng = np.random.RandomState(53)
    n, c, h, k = 4, 32, 14, 48
    x = prog.up(rng.randn(n, c, h, h).astype(np.float32))
    w_host = (rng.randn(k, c, 3, 3) * 0.1).astype(np.float32)
    mark0 = lib.lh_mark()
    w = prog.up(w_host)
    nw = w_host.size

    def run(stride):
        p = (h + 2 - 3) // stride + 1
        args = (n, c, h, h, k, 3, 3, stride, stride, 1, 1)
        y = prog.malloc(n * k * p * p); lib.lh_conv2d_fwd(x, w, 0, y, *args)
        yh = prog.down(y, (n * k * p * p,))
        dy = prog.up(np.cos(np.arange(n * k * p * p, dtype=np.float32)))
        dx = prog.malloc(n * c * h * h); lib.lh_conv2d_bwd_data(dy, w, dx, 1.0, *args)
        _lib.check()
        return yh, prog.down(dx, (n * c * h * h,))

    def check(what):
        mark = lib.lh_mark()
        got = [run(1), run(2)]
        s0 = _stats(lib)[7]
        again = [run(1), run(2)]                   # nothing written in between: served from the kept copies
        assert _stats(lib)[7] - s0 >= 6, "forward (1 copy), stride-1 input gradient (1) and stride-2 input gradient (4 classes) were to find their copies: %s" % what
        lib.lh_set_fusion(0)
        want = [run(1), run(2)]
        lib.lh_set_fusion(1)
        for g, a, t in zip(got, again, want):
            for u, v, z in zip(g, a, t):
                np.testing.assert_array_equal(u, z, err_msg=what)
                np.testing.assert_array_equal(v, z, err_msg=what + " (second time)")
        lib.lh_rewind(mark)
        return got[0][0]

    y0 = check("first use")
    w2 = (w_host * 1.5 + 0.01).astype(np.float32)
    lib.lh_h2d(w, w2.ctypes.data, w2.nbytes)
    y1 = check("after an upload")
    assert np.abs(y1 - y0).max() > 1e-3
    lib.lh_geam(w, F(0.5), w, F(0.0), w, nw)                     # in place
    y2 = check("after an operator in place")
    assert np.abs(y2 - y1).max() > 1e-3
    lib.lh_fill(w + 4 * 100, F(0.25), 50)                        # part of it
    y3 = check("after a fill over part of the filter")
    assert np.abs(y3 - y2).max() > 1e-4
    d = prog.up(rng.randn(nw).astype(np.float32)); v = prog.up(np.zeros(nw, np.float32))
    lib.lh_momentum(w, d, v, 0.1, 0.9, 400.0, 0, nw)             # gathered, launched by the next call; copies made again behind it
    y4 = check("after the optimizer")
    assert np.abs(y4 - y3).max() > 1e-3
    # the filter's memory handed to another tensor
    lib.lh_rewind(mark0)
    w_other = prog.up((rng.randn(k, c, 3, 3) * 0.1).astype(np.float32))
    assert w_other == w
    y5 = check("after a rewind that released the filter")
    assert np.abs(y5 - y4).max() > 1e-3


def test_kept_filter_copies_end_with_a_graph_replay(on_hip):
    """A recorded optimizer step replayed with lh_graph_launch changes the filter without any call that names it: the
    convolution issued after the replay must read the new weights."""
    pg = Prog(on_hip)
    lib = on_hip.lib
    rng = np.random.RandomState(59)
    n, c, h, k = 4, 32, 14, 32
    args = (n, c, h, h, k, 3, 3, 1, 1, 1, 1)
    x = pg.up(rng.randn(n, c, h, h).astype(np.float32))
    w = pg.up((rng.randn(k, c, 3, 3) * 0.1).astype(np.float32))
    nw = k * c * 9
    d = pg.up(rng.randn(nw).astype(np.float32)); v = pg.up(np.zeros(nw, np.float32))

    def conv():
        mark = lib.lh_mark()
        y = pg.malloc(n * k * h * h); lib.lh_conv2d_fwd(x, w, 0, y, *args)
        out = pg.down(y, (n * k * h * h,)); _lib.check()
        lib.lh_rewind(mark)
        return out
    on_hip.setDeterministic(True)                           # (one launch plan, no atomics: the comparison below is bit for bit; the side stream stays on)
    try:
        _graph_replay_body(lib, conv, w, d, v, nw)
    finally:
        on_hip.setDeterministic(False)


def _graph_replay_body(lib, conv, w, d, v, nw):
    y0 = conv(); conv()                                     # the second call finds the kept copy
    lib.lh_capture_begin()
    lib.lh_momentum(w, d, v, 0.1, 0.9, 400.0, 0, nw)
    gid = lib.lh_capture_end(); _lib.check()
    for _ in range(2):
        lib.lh_graph_launch(gid); _lib.check()
        y1 = conv()
        lib.lh_set_fusion(0)
        try:
            want = conv()
        finally:
            lib.lh_set_fusion(1)
        np.testing.assert_array_equal(y1, want)
        assert np.abs(y1 - y0).max() > 1e-3
        y0 = y1
    lib.lh_graph_destroy(gid); _lib.check()
