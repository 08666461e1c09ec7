#!/usr/bin/env python3
"""Operator-level measurements on one MI355X through the C ABI (HIP events on the library's stream).

  python -m lantern_amd.microbench conv   [fwd|bwd_data|bwd_filter|all]   every distinct convolution of ResNet-50 (batch 64, 224x224), TFLOP/s
  python -m lantern_amd.microbench stream                                  batch norm, relu, add, fill, copy at ResNet-50 tensor sizes, TB/s
  python -m lantern_amd.microbench gemm                                    sgemm at a few sizes, TFLOP/s
  python -m lantern_amd.microbench rnn_gated                               LSTM / GRU layer forward + backward at T 185, B 32, I = H = 800
  python -m lantern_amd.microbench copy   [MiB]                            one out-of-place element-wise pass over MiB of input: the
                                                                           known-size kernel the HBM byte counters are calibrated with

Algorithmic work: conv 2*N*K*C*R*S*P*Q flop; streaming ops in bytes per element as listed beside each op
(reads and writes that the operation cannot avoid, 4-byte elements).
"""
import sys

import numpy as np

import lantern_amd as la

# (count in the network, C, H, K, kernel, stride, pad)
RESNET50_CONVS = [(1, 3, 224, 64, 7, 2, 3), (1, 64, 56, 64, 1, 1, 0), (3, 64, 56, 64, 3, 1, 1), (4, 64, 56, 256, 1, 1, 0), (2, 256, 56, 64, 1, 1, 0),
                  (1, 256, 56, 128, 1, 1, 0), (1, 128, 56, 128, 3, 2, 1), (4, 128, 28, 512, 1, 1, 0), (1, 256, 56, 512, 1, 2, 0), (3, 512, 28, 128, 1, 1, 0),
                  (3, 128, 28, 128, 3, 1, 1), (1, 512, 28, 256, 1, 1, 0), (1, 256, 28, 256, 3, 2, 1), (6, 256, 14, 1024, 1, 1, 0), (1, 512, 28, 1024, 1, 2, 0),
                  (5, 1024, 14, 256, 1, 1, 0), (5, 256, 14, 256, 3, 1, 1), (1, 1024, 14, 512, 1, 1, 0), (1, 512, 14, 512, 3, 2, 1), (3, 512, 7, 2048, 1, 1, 0),
                  (1, 1024, 14, 2048, 1, 2, 0), (2, 2048, 7, 512, 1, 1, 0), (2, 512, 7, 512, 3, 1, 1)]
# (count, C, H) of the batch-normalised tensors
RESNET50_BN = [(1, 64, 112), (3, 64, 56), (4, 256, 56), (2, 64, 56), (1, 128, 56), (4, 128, 28), (4, 512, 28), (1, 128, 28), (1, 256, 28), (6, 256, 14),
               (7, 1024, 14), (1, 512, 14), (3, 512, 7), (4, 2048, 7)]


def timer(lib):
    def t(f, reps=5):
        f(); f()
        e0 = lib.lh_event_create(); e1 = lib.lh_event_create()
        lib.lh_event_record(e0)
        for _ in range(reps):
            f()
        lib.lh_event_record(e1)
        ms = lib.lh_event_elapsed_ms(e0, e1) / reps
        la._lib.check()
        return ms
    return t


def conv(be, which="all", N=64):
    lib, t = be.lib, timer(be.lib)
    rng = np.random.RandomState(0)
    tot = {}; totf = {}
    for (cnt, Cc, H, K, k, s, p) in RESNET50_CONVS:
        P = (H + 2 * p - k) // s + 1
        mark = be.getMallocAddr()
        x = be.fromHost(rng.randn(N * Cc * H * H).astype(np.float32)); w = be.fromHost((rng.randn(K * Cc * k * k) * 0.05).astype(np.float32))
        y = be.fromHost(rng.randn(N * K * P * P).astype(np.float32))      # also the dy of the gradient passes: real data (with an all-zero dy the input gradient measured 6 % faster)
        dx = be.mallocArray(N * Cc * H * H); dw = be.mallocArray(K * Cc * k * k)
        dims = (N, Cc, H, H, K, k, k, s, s, p, p)
        fl = 2.0 * N * K * Cc * k * k * P * P
        res = {}
        for name, fn in (("fwd", lambda: lib.lh_conv2d_fwd(x.ptr, w.ptr, 0, y.ptr, *dims)),
                         ("bwd_data", lambda: lib.lh_conv2d_bwd_data(y.ptr, w.ptr, dx.ptr, 0.0, *dims)),
                         ("bwd_filter", lambda: lib.lh_conv2d_bwd_filter(x.ptr, y.ptr, dw.ptr, 0, 1.0, *dims))):
            if which not in ("all", name) or (name == "bwd_data" and Cc == 3):
                continue
            ms = t(fn)
            res[name] = fl / ms / 1e9
            tot[name] = tot.get(name, 0.0) + cnt * ms; totf[name] = totf.get(name, 0.0) + cnt * fl
        print("%dx C%-4d H%-3d K%-4d k%d s%d  GEMM %5dx%6dx%5d  " % (cnt, Cc, H, K, k, s, K, N * P * P, Cc * k * k)
              + "  ".join("%s %6.1f TF" % (n, v) for n, v in res.items()), flush=True)
        be.resetMallocAddr(mark)
    for n in tot:
        print("%s total %.2f ms  %.1f TFLOP/s" % (n, tot[n], totf[n] / tot[n] / 1e9))


def stream(be, N=64):
    lib, t = be.lib, timer(be.lib)
    tot = {}; totb = {}
    for (cnt, Cc, H) in RESNET50_BN:
        HW = H * H; n = N * Cc * HW
        mark = be.getMallocAddr()
        x = be.mallocArray(n, zero=False); y = be.mallocArray(n, zero=False); dy = be.mallocArray(n, zero=False); dx = be.mallocArray(n); d2 = be.mallocArray(n)
        lib.lh_fill(x.ptr, 1.0, n); lib.lh_fill(dy.ptr, 0.5, n)
        g = be.mallocArray(Cc); b = be.mallocArray(Cc); sm = be.mallocArray(Cc); si = be.mallocArray(Cc); dg = be.mallocArray(Cc); db = be.mallocArray(Cc)
        lib.lh_fill(g.ptr, 1.0, Cc)
        lib.lh_bn_train_fwd_relu(x.ptr, g.ptr, b.ptr, 0, 0, y.ptr, sm.ptr, si.ptr, N, Cc, HW, 1e-5, 0.1)
        one = be._bn_one_pass(N, Cc, HW)      # a channel fits one block: the tensor is read once (forward 8, backward 12 bytes per element)
        ops = {      # name: (callable, algorithmic bytes per element)
            "bn_fwd+relu": (lambda: lib.lh_bn_train_fwd_relu(x.ptr, g.ptr, b.ptr, 0, 0, y.ptr, sm.ptr, si.ptr, N, Cc, HW, 1e-5, 0.1), 8 if one else 12),
            "bn_bwd+relu": (lambda: lib.lh_bn_bwd_relu(x.ptr, y.ptr, dy.ptr, g.ptr, b.ptr, sm.ptr, si.ptr, dx.ptr, 0.0, dg.ptr, db.ptr, N, Cc, HW), 12 if one else 20),
            "bn_bwd": (lambda: lib.lh_bn_bwd(x.ptr, dy.ptr, g.ptr, sm.ptr, si.ptr, dx.ptr, 0.0, dg.ptr, db.ptr, N, Cc, HW), 12 if one else 20),
            "add+relu": (lambda: lib.lh_add_relu(x.ptr, dy.ptr, y.ptr, n), 12),
            "add+relu grad": (lambda: lib.lh_add_relu_grad(y.ptr, dy.ptr, dx.ptr, 0.0, d2.ptr, 0.0, n), 16),
            "relu": (lambda: lib.lh_unary(0, x.ptr, x.ptr, n, 0.0, 0.0), 8),
            "fill": (lambda: lib.lh_fill(dx.ptr, 0.0, n), 4),
            "copy": (lambda: lib.lh_scalar_op(2, x.ptr, dx.ptr, 1.0, n), 8),
        }
        line = []
        for name, (fn, bpe) in ops.items():
            ms = t(fn)
            line.append("%s %.3f ms %.2f TB/s" % (name, ms, n * bpe / ms / 1e9))
            tot[name] = tot.get(name, 0.0) + cnt * ms; totb[name] = totb.get(name, 0.0) + cnt * n * bpe
        print("%dx [64,%d,%d,%d] %6.1f MB: " % (cnt, Cc, H, H, n * 4 / 1e6) + "  ".join(line), flush=True)
        be.resetMallocAddr(mark)
    print("whole network (sum over its batch-normalised tensors):")
    for n in tot:
        print("  %-14s %.3f ms  %.2f TB/s (algorithmic bytes)" % (n, tot[n], totb[n] / tot[n] / 1e9))


def gemm(be):
    lib, t = be.lib, timer(be.lib)
    rng = np.random.RandomState(0)
    for (ta, tb, m, n, k) in [(0, 1, 4096, 4096, 4096), (0, 0, 4096, 4096, 4096), (1, 0, 4096, 4096, 4096), (0, 1, 6144, 6144, 4096), (0, 1, 64, 1000, 2048),
                              (0, 0, 5920, 800, 672), (1, 0, 800, 800, 5920)]:
        mark = be.getMallocAddr()
        A = be.fromHost(rng.randn(m * k).astype(np.float32)); Bm = be.fromHost(rng.randn(k * n).astype(np.float32)); Cm = be.mallocArray(m * n)
        lda = m if ta else k; ldb = k if tb else n
        ms = t(lambda: lib.lh_sgemm(ta, tb, m, n, k, 1.0, A.ptr, lda, Bm.ptr, ldb, 0.0, Cm.ptr, n))
        print("sgemm ta%d tb%d %dx%dx%d: %.3f ms %.1f TFLOP/s" % (ta, tb, m, n, k, ms, 2.0 * m * n * k / ms / 1e9), flush=True)
        be.resetMallocAddr(mark)


def rnn_gated(be, T=185, B=32, I=800, H=800):
    """LSTM / GRU layer, forward + backward, at the DeepSpeech2 layer shape (HIP events around three calls)."""
    lib, t = be.lib, timer(be.lib)
    rng = np.random.RandomState(0)
    for mode, name in ((2, "lstm"), (3, "gru")):
        for bidir in (False, True):
            D, G = (2 if bidir else 1), (4 if mode == 2 else 3) * H
            mark = be.getMallocAddr()
            w = be.fromHost((rng.randn(D * (G * I + G * H + 2 * G)) * 0.03).astype(np.float32))
            x = be.fromHost(rng.randn(T * B * I).astype(np.float32)); dy = be.fromHost(rng.randn(T * B * D * H).astype(np.float32))
            dx = be.mallocArray(T * B * I); dw = be.mallocArray(D * (G * I + G * H + 2 * G))
            inner = be.getMallocAddr()

            def step():
                y, r = be.rnn_gated_forward(mode, x, w, T, B, I, H, bidir)
                be.rnn_gated_backward(mode, x, y, dy, w, r, dx, dw, T, B, I, H, bidir, 0.0)
                be.resetMallocAddr(inner)

            ms = t(step, reps=3)
            flop = 3 * 2.0 * T * B * G * (I + H) * D
            print("%s %s T%d B%d I%d H%d: forward + backward %.2f ms, %.1f TFLOP/s" % (name, "bidirectional" if bidir else "one direction", T, B, I, H, ms, flop / ms / 1e9), flush=True)
            be.resetMallocAddr(mark)


def copy(be, mib=256):
    n = int(mib) * (1 << 20) // 4
    x = be.mallocArray(n, zero=False); y = be.mallocArray(n, zero=False)
    be.lib.lh_fill(x.ptr, 1.0, n)
    for _ in range(3):
        be.lib.lh_scalar_op(2, x.ptr, y.ptr, 1.0, n)          # k_ew_vec<1, ...>: reads n*4 bytes, writes n*4 bytes
    be.sync()
    print("copy: %d elements, %d bytes read and %d bytes written per launch (3 launches)" % (n, 4 * n, 4 * n))


def main():
    what = sys.argv[1] if len(sys.argv) > 1 else "conv"
    be = la.BackendHIP(heap_bytes=8 << 30)
    be.setup()
    la.set_backend(be)
    if what == "conv": conv(be, sys.argv[2] if len(sys.argv) > 2 else "all")
    elif what == "stream": stream(be)
    elif what == "gemm": gemm(be)
    elif what == "rnn_gated": rnn_gated(be)
    elif what == "copy": copy(be, sys.argv[2] if len(sys.argv) > 2 else 256)
    else: sys.exit(__doc__)
    be.cleanup()


if __name__ == "__main__":
    main()
