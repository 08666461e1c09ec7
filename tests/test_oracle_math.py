"""Pins the parts of the CPU oracle that the reference's own unit-test vectors leave open
(tests/test_reference_vectors.py covers the rest): closed forms, brute force on tiny inputs,
central-difference gradient checks in double, and library routines (torch on the CPU) used as
an independent textbook implementation at real layer shapes.  A dropped term, a wrong sign, a
transposed operand or an off-by-one in the oracle fails one of these."""
import ctypes as C

import numpy as np
import pytest

from oracle.backend_cpu import load
from tests.util import cptr

lc = load()
I, F, L = C.c_int, C.c_float, C.c_long


def conv_ref(x, w, b, sH, sW, pH, pW):
    """7-loop definition in float64."""
    N, Cc, H, W = x.shape; K, _, R, S = w.shape
    P, Q = (H + 2 * pH - R) // sH + 1, (W + 2 * pW - S) // sW + 1
    y = np.zeros((N, K, P, Q))
    for n in range(N):
        for k in range(K):
            for p in range(P):
                for q in range(Q):
                    acc = 0.0 if b is None else float(b[k])
                    for c in range(Cc):
                        for r in range(R):
                            for s in range(S):
                                h, ww = p * sH - pH + r, q * sW - pW + s
                                if 0 <= h < H and 0 <= ww < W:
                                    acc += float(x[n, c, h, ww]) * float(w[k, c, r, s])
                    y[n, k, p, q] = acc
    return y


def oracle_conv(x, w, b, dims, dy=None):
    N, Cc, H, W, K, R, S, sH, sW, pH, pW = dims
    P, Q = (H + 2 * pH - R) // sH + 1, (W + 2 * pW - S) // sW + 1
    y = np.zeros((N, K, P, Q), np.float32); fin = np.zeros((N, Cc * R * S, P * Q), np.float32)
    ints = [I(v) for v in dims]
    lc.lc_conv2d_fwd(cptr(x), cptr(w), cptr(b) if b is not None else None, cptr(y), cptr(fin), *ints)
    if dy is None:
        return y
    dx = np.zeros_like(x); dw = np.zeros_like(w); db = np.zeros(K, np.float32); sc = np.zeros_like(fin)
    lc.lc_conv2d_bwd(cptr(fin), cptr(w), cptr(dy), cptr(dx), cptr(dw), cptr(db), cptr(sc), *ints)
    return y, dx, dw, db


@pytest.mark.parametrize("dims", [(2, 3, 5, 7, 4, 3, 3, 1, 1, 1, 1), (1, 2, 7, 6, 3, 3, 2, 2, 1, 1, 0), (2, 1, 6, 6, 2, 1, 1, 2, 2, 0, 0),
                                  (1, 2, 9, 5, 2, 5, 3, 2, 1, 2, 1)])
def test_conv_forward_against_definition_nonsquare(dims):
    """Non-square outputs included: the reference's im2col mis-addresses them (CPU:491, outputWidth
    squared); the oracle follows the mathematical definition."""
    rng = np.random.RandomState(1)
    N, Cc, H, W, K, R, S, sH, sW, pH, pW = dims
    x = rng.randn(N, Cc, H, W).astype(np.float32); w = rng.randn(K, Cc, R, S).astype(np.float32); b = rng.randn(K).astype(np.float32)
    np.testing.assert_allclose(oracle_conv(x, w, b, dims), conv_ref(x, w, b, sH, sW, pH, pW), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(oracle_conv(x, w, None, dims), conv_ref(x, w, None, sH, sW, pH, pW), rtol=1e-5, atol=1e-5)


def test_conv_gradients_by_central_differences():
    rng = np.random.RandomState(2)
    dims = (2, 2, 5, 6, 3, 3, 2, 2, 1, 1, 0)
    N, Cc, H, W, K, R, S, sH, sW, pH, pW = dims
    x = rng.randn(N, Cc, H, W).astype(np.float32); w = rng.randn(K, Cc, R, S).astype(np.float32); b = rng.randn(K).astype(np.float32)
    y0 = conv_ref(x, w, b, sH, sW, pH, pW)
    dy = rng.randn(*y0.shape).astype(np.float32)
    _, dx, dw, db = oracle_conv(x, w, b, dims, dy)
    loss = lambda xx, ww, bb: float((conv_ref(xx, ww, bb, sH, sW, pH, pW) * dy).sum())
    eps = 1e-3
    for arr, grad in ((x, dx), (w, dw), (b, db)):
        flat = arr.reshape(-1); g = grad.reshape(-1)
        for i in rng.choice(flat.size, size=min(12, flat.size), replace=False):
            old = flat[i]
            flat[i] = old + eps; lp = loss(x, w, b)
            flat[i] = old - eps; lm = loss(x, w, b)
            flat[i] = old
            assert abs((lp - lm) / (2 * eps) - g[i]) < 2e-2 * max(1.0, abs(g[i])), (i, (lp - lm) / (2 * eps), g[i])


def test_conv_pool_bn_against_torch_at_layer_shapes():
    torch = pytest.importorskip("torch")
    import torch.nn.functional as Fn
    rng = np.random.RandomState(3)
    for dims in [(2, 64, 14, 14, 64, 3, 3, 1, 1, 1, 1), (2, 32, 15, 15, 48, 3, 3, 2, 2, 1, 1), (2, 3, 32, 32, 16, 7, 7, 2, 2, 3, 3), (2, 64, 8, 8, 128, 1, 1, 2, 2, 0, 0)]:
        N, Cc, H, W, K, R, S, sH, sW, pH, pW = dims
        x = rng.randn(N, Cc, H, W).astype(np.float32); w = (rng.randn(K, Cc, R, S) / 8).astype(np.float32)
        tx = torch.tensor(x, requires_grad=True); tw = torch.tensor(w, requires_grad=True)
        ty = Fn.conv2d(tx, tw, None, (sH, sW), (pH, pW))
        dy = rng.randn(*ty.shape).astype(np.float32)
        ty.backward(torch.tensor(dy))
        y, dx, dw, _ = oracle_conv(x, w, None, dims, dy)
        np.testing.assert_allclose(y, ty.detach().numpy(), rtol=1e-4, atol=1e-4)
        np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=1e-4, atol=1e-4)
        np.testing.assert_allclose(dw, tw.grad.numpy(), rtol=1e-3, atol=1e-3)
    # max pool with padding: values and the argmax as a global flat index, first maximum wins
    x = rng.randn(3, 4, 9, 9).astype(np.float32)
    y = np.zeros((3, 4, 5, 5), np.float32); idx = np.zeros((3, 4, 5, 5), np.int32)
    lc.lc_maxpool_fwd(cptr(x), cptr(y), cptr(idx), I(3), I(4), I(9), I(9), I(3), I(3), I(2), I(2), I(1))
    ty, tidx = Fn.max_pool2d(torch.tensor(x), 3, 2, 1, return_indices=True)
    np.testing.assert_array_equal(y, ty.numpy())
    base = (np.arange(12) * 81).reshape(3, 4, 1, 1)
    np.testing.assert_array_equal(idx, tidx.numpy() + base)
    # batch norm (training) forward/backward, running statistics with the unbiased variance
    x = (rng.randn(4, 6, 5, 5) * 2 + 1).astype(np.float32); g = rng.rand(6).astype(np.float32) + 0.5; b = rng.randn(6).astype(np.float32)
    rm = np.zeros(6, np.float32); rv = np.ones(6, np.float32)
    y = np.zeros_like(x); sm = np.zeros(6, np.float32); si = np.zeros(6, np.float32)
    lc.lc_bn_train_fwd(cptr(x), cptr(g), cptr(b), cptr(rm), cptr(rv), cptr(y), cptr(sm), cptr(si), I(4), I(6), I(25), F(1e-5), F(0.1))
    tx = torch.tensor(x, requires_grad=True); tg = torch.tensor(g, requires_grad=True); tb = torch.tensor(b, requires_grad=True)
    trm = torch.zeros(6); trv = torch.ones(6)
    ty = Fn.batch_norm(tx, trm, trv, tg, tb, True, 0.1, 1e-5)
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(rm, trm.numpy(), rtol=1e-5, atol=1e-6); np.testing.assert_allclose(rv, trv.numpy(), rtol=1e-5, atol=1e-6)
    dy = rng.randn(*x.shape).astype(np.float32)
    ty.backward(torch.tensor(dy))
    dx = np.zeros_like(x); dg = np.zeros(6, np.float32); db = np.zeros(6, np.float32)
    lc.lc_bn_bwd(cptr(x), cptr(dy), cptr(g), cptr(sm), cptr(si), cptr(dx), cptr(dg), cptr(db), I(4), I(6), I(25))
    np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=1e-3, atol=1e-5)
    np.testing.assert_allclose(dg, tg.grad.numpy(), rtol=1e-4, atol=1e-4); np.testing.assert_allclose(db, tb.grad.numpy(), rtol=1e-4, atol=1e-4)


def test_softmax_invariants_and_gradient():
    rng = np.random.RandomState(4)
    x = (rng.randn(5, 7) * 3).astype(np.float32)
    y = np.zeros_like(x); ly = np.zeros_like(x)
    lc.lc_softmax(I(0), cptr(x), cptr(y), I(5), I(7)); lc.lc_softmax(I(1), cptr(x), cptr(ly), I(5), I(7))
    np.testing.assert_allclose(y.sum(1), 1.0, rtol=1e-6)
    np.testing.assert_allclose(np.exp(ly), y, rtol=1e-5)
    x64 = x.astype(np.float64); e = np.exp(x64 - x64.max(1, keepdims=True)); ref = e / e.sum(1, keepdims=True)
    np.testing.assert_allclose(y, ref, rtol=1e-5)
    dy = rng.randn(5, 7).astype(np.float32)
    dx = np.zeros_like(x)
    lc.lc_softmax_grad(I(0), cptr(y), cptr(dy), cptr(dx), I(5), I(7))
    jac = ref * (dy - (dy * ref).sum(1, keepdims=True))     # J^T dy for softmax
    np.testing.assert_allclose(dx, jac, rtol=1e-4, atol=1e-6)
    # [outer, c, inner] view equals the transposed 2-D problem
    x3 = rng.randn(2, 4, 3).astype(np.float32); y3 = np.zeros_like(x3)
    lc.lc_softmax3(I(0), cptr(x3), cptr(y3), I(2), I(4), I(3))
    e3 = np.exp(x3 - x3.max(1, keepdims=True)); np.testing.assert_allclose(y3, e3 / e3.sum(1, keepdims=True), rtol=1e-5)


def test_optimizer_recurrences():
    """SGD (NN:265-287), momentum (CPU:1232-1246) and Adagrad (CPU:1217-1230) against the recurrences in double."""
    rng = np.random.RandomState(5)
    n = 33
    x0 = rng.randn(n).astype(np.float32)
    for nesterov in (0, 1):
        x = x0.copy(); v = np.zeros(n, np.float32); xr = x0.astype(np.float64); vr = np.zeros(n)
        for step in range(4):
            g = (rng.randn(n) * 300).astype(np.float32)          # some beyond the clip of 400
            d = g.copy()
            lc.lc_momentum(cptr(x), cptr(d), cptr(v), F(0.1), F(0.9), F(400.0), I(nesterov), L(n))
            assert (d == 0).all()
            gc = np.clip(g.astype(np.float64), -400, 400)
            vr = 0.9 * vr + gc
            xr -= 0.1 * ((gc + 0.9 * vr) if nesterov else vr)
            np.testing.assert_allclose(x, xr, rtol=1e-5, atol=1e-4)
    x = x0.copy(); m = np.zeros(n, np.float32); xr = x0.astype(np.float64); mr = np.zeros(n)
    for step in range(4):
        g = (rng.randn(n) * 2).astype(np.float32); d = g.copy()
        lc.lc_adagrad(cptr(x), cptr(d), cptr(m), F(0.05), F(1.0), L(n))
        gc = np.clip(g.astype(np.float64), -1, 1); mr += gc * gc; xr -= 0.05 * gc / np.sqrt(mr + 1e-8)
        np.testing.assert_allclose(x, xr, rtol=1e-5, atol=1e-6); assert (d == 0).all()
    x = x0.copy(); d = np.ones(n, np.float32)
    lc.lc_sgd(cptr(x), cptr(d), F(0.5), L(n))
    np.testing.assert_allclose(x, x0 - 0.5, rtol=1e-6); assert (d == 0).all()


def test_sgemm_all_cases_and_ragged_sizes():
    rng = np.random.RandomState(6)
    for (ta, tb, m, n, k) in [(0, 0, 7, 5, 3), (0, 1, 13, 17, 300), (1, 0, 6, 16, 257), (1, 1, 97, 33, 65), (0, 0, 1, 1, 1), (0, 0, 100, 2100, 40)]:
        A = rng.randn(*((k, m) if ta else (m, k))).astype(np.float32); B = rng.randn(*((n, k) if tb else (k, n))).astype(np.float32)
        Cm = rng.randn(m, n).astype(np.float32); ref = 0.5 * ((A.T if ta else A).astype(np.float64) @ (B.T if tb else B)) + 2.0 * Cm
        lc.lc_sgemm(I(ta), I(tb), I(m), I(n), I(k), F(0.5), cptr(A), I(A.shape[1]), cptr(B), I(B.shape[1]), F(2.0), cptr(Cm), I(n))
        np.testing.assert_allclose(Cm, ref, rtol=1e-4, atol=1e-4)


def test_dropout_counter_generator_and_glibc_order():
    n = 20000
    x = np.ones(n, np.float32); y = np.zeros(n, np.float32); m = np.zeros(n, np.float32)
    lc.lc_dropout_ctr(cptr(x), cptr(y), cptr(m), L(n), F(0.5), C.c_uint64(42), C.c_uint64(0))
    keep = (m > 0).mean()
    assert abs(keep - 0.5) < 0.02 and set(np.unique(m)) == {0.0, 2.0} and (y == m).all()
    y2 = np.zeros(n, np.float32); m2 = np.zeros(n, np.float32)
    lc.lc_dropout_ctr(cptr(x), cptr(y2), cptr(m2), L(n // 2), F(0.5), C.c_uint64(42), C.c_uint64(n // 2))
    np.testing.assert_array_equal(m2[:n // 2], m[n // 2:])           # keyed by (seed, offset + index)
    lc.lc_srand(C.c_uint(42))
    r = np.zeros(8, np.float32); lc.lc_rand_uniform(cptr(r), L(8))
    lc.lc_srand(C.c_uint(42))
    lc.lc_dropout_rand(cptr(x), cptr(y), cptr(m), L(8), F(0.5))
    np.testing.assert_array_equal(m[:8] > 0, (r + 0.5) > 0.5)        # same glibc sequence, keep iff rand > p (CPU:1075)


def test_ctc_against_torch():
    """lc_ctc_loss has no asserted vector in the reference ("parity unpinned" there); the maths is
    checked against torch's CTC: cost, and gradient w.r.t. the pre-softmax activations / batch."""
    torch = pytest.importorskip("torch")
    rng = np.random.RandomState(7)
    Tn, B, A = 12, 3, 6
    act = rng.randn(Tn, B, A).astype(np.float32)
    lens = np.array([3, 2, 4], np.int32); labels = np.array([1, 2, 1, 3, 3, 5, 4, 2, 1], np.int32); ilen = np.array([12, 10, 12], np.int32)
    ta = torch.tensor(act, requires_grad=True)
    lp = torch.log_softmax(ta, 2)
    loss = torch.nn.functional.ctc_loss(lp, torch.tensor(labels.astype(np.int64)), torch.tensor(ilen.astype(np.int64)), torch.tensor(lens.astype(np.int64)),
                                        blank=0, reduction="none")
    loss.sum().backward()          # the gradient of the SUM of costs (what cuDNN writes), not of their mean
    probs = torch.softmax(torch.tensor(act), 2).numpy().astype(np.float32)
    costs = np.zeros(B, np.float32); d = np.zeros_like(probs)
    lc.lc_ctc_loss(cptr(probs), cptr(d), cptr(labels), cptr(lens), cptr(ilen), cptr(costs), I(Tn), I(B), I(A))
    np.testing.assert_allclose(costs, loss.detach().numpy(), rtol=1e-4, atol=1e-4)
    g = ta.grad.numpy().copy()
    for b in range(B):
        g[ilen[b]:, b, :] = 0; 
    np.testing.assert_allclose(d, g, rtol=1e-3, atol=1e-5)


@pytest.mark.parametrize("mode", [0, 1], ids=["relu", "tanh"])
@pytest.mark.parametrize("bidir", [False, True], ids=["uni", "bi"])
def test_rnn_against_torch(mode, bidir):
    """lc_rnn_fwd / lc_rnn_bwd (no counterpart on the reference's CPU side) against torch.nn.RNN: outputs, input
    gradient and every weight gradient, with the packed weight order W_ih, W_hh, b_ih, b_hh per direction."""
    torch = pytest.importorskip("torch")
    rng = np.random.RandomState(8 + mode)
    T, B, In, H = 7, 3, 5, 6
    D = 2 if bidir else 1
    per = H * In + H * H + 2 * H
    w = (rng.randn(D * per) * 0.4).astype(np.float32)
    x = rng.randn(T, B, In).astype(np.float32); dy = rng.randn(T, B, D * H).astype(np.float32)
    rnn = torch.nn.RNN(In, H, 1, nonlinearity="tanh" if mode == 1 else "relu", bidirectional=bidir)
    names = ["weight_ih_l0", "weight_hh_l0", "bias_ih_l0", "bias_hh_l0"]
    with torch.no_grad():
        for d in range(D):
            o = d * per
            for nm, size, shape in zip(names, (H * In, H * H, H, H), ((H, In), (H, H), (H,), (H,))):
                getattr(rnn, nm + ("_reverse" if d else "")).copy_(torch.tensor(w[o:o + size].reshape(shape))); o += size
    tx = torch.tensor(x, requires_grad=True)
    ty, _ = rnn(tx)
    ty.backward(torch.tensor(dy))
    y = np.zeros((T, B, D * H), np.float32)
    lc.lc_rnn_fwd(I(mode), cptr(x), cptr(w), cptr(y), I(T), I(B), I(In), I(H), I(int(bidir)))
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=1e-5, atol=1e-6)
    dx = np.ones_like(x); dw = np.ones_like(w)                    # both accumulate
    lc.lc_rnn_bwd(I(mode), cptr(x), cptr(y), cptr(dy), cptr(w), cptr(dx), cptr(dw), I(T), I(B), I(In), I(H), I(int(bidir)))
    np.testing.assert_allclose(dx - 1, tx.grad.numpy(), rtol=1e-4, atol=1e-5)
    for d in range(D):
        o = d * per
        for nm, size in zip(names, (H * In, H * H, H, H)):
            g = getattr(rnn, nm + ("_reverse" if d else "")).grad.numpy().ravel()
            np.testing.assert_allclose(dw[o:o + size] - 1, g, rtol=1e-4, atol=1e-5, err_msg=nm + str(d)); o += size


@pytest.mark.parametrize("mode", [2, 3], ids=["lstm", "gru"])
@pytest.mark.parametrize("bidir", [False, True], ids=["uni", "bi"])
def test_gated_rnn_against_torch(mode, bidir):
    """lc_rnn_gated_fwd / lc_rnn_gated_bwd (cuDNN's LSTM / GRU formulas; nothing on the reference's CPU side) against
    torch.nn.LSTM / torch.nn.GRU, which use the same gate order (i f g o; r z n) and the same reset-after-product GRU:
    outputs, input gradient and every weight gradient, packed W_ih, W_hh, b_ih, b_hh per direction.  A swapped gate, a
    reset gate applied before the product or a bias on the wrong side of it changes the output or one of the bias gradients."""
    torch = pytest.importorskip("torch")
    rng = np.random.RandomState(20 + mode)
    T, B, In, H = 6, 3, 5, 4
    D, G = (2 if bidir else 1), (4 if mode == 2 else 3) * H
    per = G * In + G * H + 2 * G
    w = (rng.randn(D * per) * 0.5).astype(np.float32)
    x = rng.randn(T, B, In).astype(np.float32); dy = rng.randn(T, B, D * H).astype(np.float32)
    net = (torch.nn.LSTM if mode == 2 else torch.nn.GRU)(In, H, 1, bidirectional=bidir)
    names = ["weight_ih_l0", "weight_hh_l0", "bias_ih_l0", "bias_hh_l0"]
    sizes, shapes = (G * In, G * H, G, G), ((G, In), (G, H), (G,), (G,))
    with torch.no_grad():
        for d in range(D):
            o = d * per
            for nm, size, shape in zip(names, sizes, shapes):
                getattr(net, nm + ("_reverse" if d else "")).copy_(torch.tensor(w[o:o + size].reshape(shape))); o += size
    tx = torch.tensor(x, requires_grad=True)
    ty, _ = net(tx)
    ty.backward(torch.tensor(dy))
    y = np.zeros((T, B, D * H), np.float32)
    lc.lc_rnn_gated_fwd(I(mode), cptr(x), cptr(w), cptr(y), I(T), I(B), I(In), I(H), I(int(bidir)))
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=1e-5, atol=1e-6)
    dx = np.ones_like(x); dw = np.ones_like(w)                    # both accumulate
    lc.lc_rnn_gated_bwd(I(mode), cptr(x), cptr(dy), cptr(w), cptr(dx), cptr(dw), I(T), I(B), I(In), I(H), I(int(bidir)))
    np.testing.assert_allclose(dx - 1, tx.grad.numpy(), rtol=1e-4, atol=1e-5)
    for d in range(D):
        o = d * per
        for nm, size in zip(names, sizes):
            g = getattr(net, nm + ("_reverse" if d else "")).grad.numpy().ravel()
            np.testing.assert_allclose(dw[o:o + size] - 1, g, rtol=1e-4, atol=1e-5, err_msg=nm + str(d)); o += size


@pytest.mark.parametrize("mode", [0, 1, 2, 3], ids=["relu", "tanh", "lstm", "gru"])
@pytest.mark.parametrize("bidir", [False, True], ids=["uni", "bi"])
def test_rnn_initial_states_against_torch(mode, bidir):
    """The *_init forms (initial hidden state, and cell state for the LSTM, as values without a gradient) against torch's
    h_0 / c_0: outputs, input gradient and weight gradients.  A state handed to the wrong direction, used as a zero in the
    backward pass (the W_hh gradient of the first step would miss its term) or a cell state read as hidden state fails."""
    torch = pytest.importorskip("torch")
    rng = np.random.RandomState(50 + mode)
    T, B, In, H = 5, 3, 4, 6
    ng = {0: 1, 1: 1, 2: 4, 3: 3}[mode]
    D, G = (2 if bidir else 1), ng * H
    per = G * In + G * H + 2 * G
    w = (rng.randn(D * per) * 0.5).astype(np.float32)
    x = rng.randn(T, B, In).astype(np.float32); dy = rng.randn(T, B, D * H).astype(np.float32)
    hx = rng.randn(D, B, H).astype(np.float32); cx = rng.randn(D, B, H).astype(np.float32)
    if mode < 2:
        net = torch.nn.RNN(In, H, 1, nonlinearity="tanh" if mode == 1 else "relu", bidirectional=bidir)
    else:
        net = (torch.nn.LSTM if mode == 2 else torch.nn.GRU)(In, H, 1, bidirectional=bidir)
    names = ["weight_ih_l0", "weight_hh_l0", "bias_ih_l0", "bias_hh_l0"]
    sizes, shapes = (G * In, G * H, G, G), ((G, In), (G, H), (G,), (G,))
    with torch.no_grad():
        for d in range(D):
            o = d * per
            for nm, size, shape in zip(names, sizes, shapes):
                getattr(net, nm + ("_reverse" if d else "")).copy_(torch.tensor(w[o:o + size].reshape(shape))); o += size
    tx = torch.tensor(x, requires_grad=True)
    state = (torch.tensor(hx), torch.tensor(cx)) if mode == 2 else torch.tensor(hx)
    ty, _ = net(tx, state)
    ty.backward(torch.tensor(dy))
    y = np.zeros((T, B, D * H), np.float32)
    dx = np.ones_like(x); dw = np.ones_like(w)
    if mode < 2:
        lc.lc_rnn_fwd_init(I(mode), cptr(x), cptr(hx), cptr(w), cptr(y), I(T), I(B), I(In), I(H), I(int(bidir)))
        lc.lc_rnn_bwd_init(I(mode), cptr(x), cptr(hx), cptr(y), cptr(dy), cptr(w), cptr(dx), cptr(dw), I(T), I(B), I(In), I(H), I(int(bidir)))
    else:
        c0 = cptr(cx) if mode == 2 else None
        lc.lc_rnn_gated_fwd_init(I(mode), cptr(x), cptr(hx), c0, cptr(w), cptr(y), I(T), I(B), I(In), I(H), I(int(bidir)))
        lc.lc_rnn_gated_bwd_init(I(mode), cptr(x), cptr(hx), c0, cptr(dy), cptr(w), cptr(dx), cptr(dw), I(T), I(B), I(In), I(H), I(int(bidir)))
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(dx - 1, tx.grad.numpy(), rtol=1e-4, atol=1e-5)
    for d in range(D):
        o = d * per
        for nm, size in zip(names, sizes):
            g = getattr(net, nm + ("_reverse" if d else "")).grad.numpy().ravel()
            np.testing.assert_allclose(dw[o:o + size] - 1, g, rtol=1e-4, atol=1e-5, err_msg=nm + str(d)); o += size


@pytest.mark.parametrize("p", [(2, 3, 8, 8, 3, 3, 1, 1, 1, 1), (1, 2, 5, 9, 2, 4, 2, 3, 1, 2), (2, 2, 13, 13, 3, 3, 2, 2, 0, 1), (1, 1, 4, 4, 4, 4, 3, 3, 3, 3)],
                         ids=lambda s: "x".join(map(str, s)))
def test_padded_avgpool_against_torch(p):
    """lc_avgpool_pad_fwd / _bwd (the reference's CPU backend has nothing here) against torch's avg_pool2d with
    count_include_pad=False, values and autograd; a divisor that counts the padding fails on every border output."""
    torch = pytest.importorskip("torch")
    N, C, H, W, kH, kW, sH, sW, pH, pW = p
    if pH > kH // 2 or pW > kW // 2:
        pytest.skip("torch limits the pad to half the kernel")
    rng = np.random.RandomState(33)
    x = rng.randn(N, C, H, W).astype(np.float32)
    tx = torch.tensor(x, requires_grad=True)
    ty = torch.nn.functional.avg_pool2d(tx, (kH, kW), (sH, sW), (pH, pW), count_include_pad=False)
    dy = rng.randn(*ty.shape).astype(np.float32)
    ty.backward(torch.tensor(dy))
    y = np.zeros(ty.shape, np.float32)
    args = [I(v) for v in (N, C, H, W, kH, kW, sH, sW, pH, pW)]
    lc.lc_avgpool_pad_fwd(cptr(x), cptr(y), *args)
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=1e-5, atol=1e-6)
    dx = np.ones_like(x)
    lc.lc_avgpool_pad_bwd(cptr(dy), cptr(dx), *args)
    np.testing.assert_allclose(dx - 1, tx.grad.numpy(), rtol=1e-5, atol=1e-6)


def test_mean_clip_bias_fill_and_sgemv_literals():
    """Literal answers for the one-liners that no reference vector reaches: mean (CPU:1115-1124: sum, then one division by the
    count), clipAt (CPU:112-119: symmetric clamp, values inside untouched), fillWithBias (CPU:39-62: the bias runs along the middle
    of outer x c x inner) and the matrix-vector kernel behind the dot family (both orientations, alpha and beta)."""
    x = np.array([1, 2, 3, 6], np.float32); out = np.full(1, -7, np.float32)
    lc.lc_mean_all(cptr(x), cptr(out), L(4))
    assert out[0] == 3.0
    x = np.array([0.5, -1.5, 4.0], np.float32); lc.lc_mean_all(cptr(x), cptr(out), L(3))
    assert out[0] == 1.0                                   # not the sum (3), not divided by n-1 (1.5)

    v = np.array([-2.0, 0.3, 2.0, -0.5, 0.5, -0.25], np.float32)
    lc.lc_clip(cptr(v), F(0.5), L(6))
    np.testing.assert_array_equal(v, np.array([-0.5, 0.3, 0.5, -0.5, 0.5, -0.25], np.float32))
    v = np.array([3.0, -3.0, 9.0], np.float32); lc.lc_clip(cptr(v), F(1.0), L(2))          # the count bounds it
    np.testing.assert_array_equal(v, np.array([1.0, -1.0, 9.0], np.float32))

    y = np.full((2, 3, 2), -1, np.float32); bias = np.array([10, 20, 30], np.float32)
    lc.lc_fill_with_bias(cptr(y), cptr(bias), L(2), L(3), L(2))
    np.testing.assert_array_equal(y, np.array([[[10, 10], [20, 20], [30, 30]]] * 2, np.float32))
    y = np.zeros((4, 3), np.float32); lc.lc_fill_with_bias(cptr(y), cptr(bias), L(4), L(3), L(1))   # the linear layers' [batch, out] case
    np.testing.assert_array_equal(y, np.tile(bias, (4, 1)))

    A = np.array([[1, 2, 3], [4, 5, 6]], np.float32); xv = np.array([1, -1, 2], np.float32); yv = np.array([100, 200], np.float32)
    lc.lc_sgemv(I(0), I(2), I(3), F(2.0), cptr(A), I(3), cptr(xv), F(0.5), cptr(yv))      # y = 2*A x + 0.5*y
    np.testing.assert_array_equal(yv, np.array([2 * 5 + 50, 2 * 11 + 100], np.float32))
    tv = np.array([1, -1], np.float32); zv = np.array([1, 1, 1], np.float32)
    lc.lc_sgemv(I(1), I(2), I(3), F(1.0), cptr(A), I(3), cptr(tv), F(1.0), cptr(zv))      # z += A^T t
    np.testing.assert_array_equal(zv, np.array([1 - 3, 1 - 3, 1 - 3], np.float32))


@pytest.mark.parametrize("shape,context", [((7, 3, 5), 2), ((5, 4), 4), ((9,), 1), ((30, 2, 16), 20), ((4, 1, 1), 0)], ids=str)
def test_repeat0_and_its_gradient_against_numpy(shape, context):
    """repeat0 (TD:1446-1451; CDN:378-399): out[i0, i1] = in[i0 + i1] against numpy's sliding windows, bit for bit; the gradient
    against the scatter the definition fixes (every window's slice added back onto the rows it was cut from, on top of what the
    gradient buffer held), a literal case included."""
    rng = np.random.RandomState(51)
    x = rng.randn(*shape).astype(np.float32)
    rows, inner = shape[0], int(np.prod(shape[1:]))
    oshape = (rows - context, context + 1) + tuple(shape[1:])
    y = np.full(oshape, -9, np.float32)
    lc.lc_repeat0(cptr(x), cptr(y), I(rows), I(context), L(inner))
    np.testing.assert_array_equal(y, np.stack([x[i:i + context + 1] for i in range(rows - context)]))
    dy = rng.randn(*oshape).astype(np.float32)
    dx = np.ones_like(x)
    want = np.ones_like(x)
    for i0 in range(rows - context):
        for i1 in range(context + 1):
            want[i0 + i1] += dy[i0, i1]
    lc.lc_repeat0_grad(cptr(dx), cptr(dy), I(rows), I(context), L(inner))
    np.testing.assert_allclose(dx, want, rtol=1e-6, atol=1e-6)
    # by hand: rows 0..3, context 1 -> windows (0,1), (1,2), (2,3); ones as the windows' gradient: rows get 1, 2, 2, 1
    d = np.zeros(4, np.float32); g = np.ones((3, 2), np.float32)
    lc.lc_repeat0_grad(cptr(d), cptr(g), I(4), I(1), L(1))
    np.testing.assert_array_equal(d, np.array([1, 2, 2, 1], np.float32))
