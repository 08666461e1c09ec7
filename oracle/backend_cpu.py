"""TEST INFRASTRUCTURE, NOT PRODUCT: the CPU oracle behind the same Backend interface.

`BackendCPU` plays the role of the reference's BackendCPU (src/main/scala/lantern/
TensorDslCPU.scala:15-1248): it implements lantern_amd.backend.Backend on host memory by calling
oracle/liblantern_cpu.so (the C restatement in lantern_cpu.c).  Tests run the same Tensor/TensorR
programs on it and on BackendHIP and compare; the benchmark times it as the CPU baseline.
Nothing in lantern_amd/ imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

from lantern_amd.backend import Backend, Buf, conv_size

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liblantern_cpu.so")
_lib = None


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE])


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = C.CDLL(LIB_PATH)
        _lib.lc_ctr_uniform.restype = C.c_float
        _lib.lc_get_threads.restype = C.c_int
    return _lib


P, I, F, L, U64 = C.c_void_p, C.c_int, C.c_float, C.c_long, C.c_uint64


def _ints(seq):
    return (C.c_int * len(seq))(*[int(v) for v in seq])


class BackendCPU(Backend):
    name = "cpu-oracle"

    def __init__(self, threads=1):
        self.lib = load()
        self.threads = threads
        self.dropout_seed = 42
        self.dropout_offset = 0
        self.dropout_mode = "ctr"       # "ctr": counter-based (matches the device); "rand": glibc order (CPU:1066-1084)

    def setup(self):
        self.lib.lc_set_threads(I(self.threads))

    def cleanup(self): pass
    def sync(self): pass

    # -- memory -------------------------------------------------------------------------------
    def mallocArray(self, length, zero=True):
        arr = np.zeros(max(int(length), 1), dtype=np.float32)
        return Buf(arr.ctypes.data, arr.size, arr)

    def getMallocAddr(self): return 0
    def resetMallocAddr(self, addr): pass

    def copyFloatArray(self, dest, src, length):
        C.memmove(dest.ptr, src.ptr, 4 * int(length))

    def fromHost(self, arr):
        a = np.array(arr, copy=True, order="C")
        assert a.dtype.itemsize == 4
        if a.size == 0:
            a = np.zeros(1, dtype=a.dtype)
        return Buf(a.ctypes.data, a.size, a)

    def upload(self, buf, arr):
        arr = np.ascontiguousarray(arr)
        C.memmove(buf.ptr, arr.ctypes.data, arr.nbytes)

    def toHost(self, buf, n, dtype=np.float32):
        out = np.empty(int(n), dtype=dtype)
        C.memmove(out.ctypes.data, buf.ptr, out.nbytes)
        return out

    def _c(self, name, *args):
        getattr(self.lib, name)(*args)

    # -- fills ----------------------------------------------------------------------------------
    def fillInPlace(self, data, n, value): self._c("lc_fill", P(data.ptr), F(value), L(n))

    def fillWithBias(self, dims, bias, dim):
        outer = int(np.prod(dims[:dim], dtype=np.int64)); c = dims[dim]; inner = int(np.prod(dims[dim + 1:], dtype=np.int64))
        res = self.mallocArray(outer * c * inner)
        self._c("lc_fill_with_bias", P(res.ptr), P(bias.ptr), L(outer), L(c), L(inner))
        return res

    def clipAt(self, data, n, bound): self._c("lc_clip", P(data.ptr), F(bound), L(n))

    # -- dot family ---------------------------------------------------------------------------------
    def vectorVectorDot(self, x, y, n):
        res = self.mallocArray(1); self._c("lc_dot_vv", P(x.ptr), P(y.ptr), P(res.ptr), I(n)); return res

    def matrixVectorDot(self, x, y, m, n):
        res = self.mallocArray(m); self._c("lc_dot_mv", P(x.ptr), P(y.ptr), P(res.ptr), I(m), I(n)); return res

    def matrixMatrixDot(self, x, y, m, k, n):
        res = self.mallocArray(m * n); self._c("lc_dot_mm", P(x.ptr), P(y.ptr), P(res.ptr), I(m), I(k), I(n)); return res

    def addMul_scalar(self, xd, s, y, n): self._c("lc_addmul_scalar", P(xd.ptr), P(s.ptr), P(y.ptr), L(n))
    def add_cartesian(self, xd, y, outd, m, n): self._c("lc_add_cartesian", P(xd.ptr), P(y.ptr), P(outd.ptr), I(m), I(n))
    def add_composition(self, xd, y, outd, m, n): self._c("lc_add_composition", P(xd.ptr), P(y.ptr), P(outd.ptr), I(m), I(n))
    def add_dotTrans1(self, xd, y, outd, d1, d2, d3): self._c("lc_add_dottrans1", P(xd.ptr), P(y.ptr), P(outd.ptr), I(d1), I(d2), I(d3))
    def add_dotTrans2(self, xd, y, outd, d1, d2, d3): self._c("lc_add_dottrans2", P(xd.ptr), P(y.ptr), P(outd.ptr), I(d1), I(d2), I(d3))

    def gemm(self, x, tx, y, ty, alpha, d1, d2, d3):
        res = self.mallocArray(d1 * d3)
        self._c("lc_gemm", I(int(tx)), I(int(ty)), I(d1), I(d2), I(d3), F(alpha), P(x.ptr), P(y.ptr), P(res.ptr))
        return res

    def gemm_grad(self, x, xd, x_in, tx, y, yd, y_in, ty, alpha, od, d1, d2, d3, xbeta=1.0, ybeta=1.0):
        # host memory from mallocArray is always zero, so overwrite (beta 0) and accumulate coincide
        self._c("lc_gemm_grad", I(int(tx)), I(int(ty)), I(d1), I(d2), I(d3), F(alpha), P(x.ptr), P(xd.ptr if xd is not None else 0), I(int(x_in)),
                P(y.ptr), P(yd.ptr if yd is not None else 0), I(int(y_in)), P(od.ptr))

    # -- broadcast -----------------------------------------------------------------------------------
    def bcast_op(self, op, a, ashape, b, bshape, oshape):
        res = self.mallocArray(int(np.prod(oshape, dtype=np.int64)))
        self._c("lc_bcast_op", I(op), P(a.ptr), _ints(ashape), P(b.ptr), _ints(bshape), P(res.ptr), _ints(oshape), I(len(oshape)))
        return res

    def bcast_op_grad(self, op, a, ad, ashape, a_in, b, bd, bshape, b_in, od, oshape):
        self._c("lc_bcast_op_grad", I(op), P(a.ptr), P(ad.ptr), _ints(ashape), I(int(a_in)), P(b.ptr), P(bd.ptr), _ints(bshape), I(int(b_in)),
                P(od.ptr), _ints(oshape), I(len(oshape)))

    def bcast_update(self, op, a, ashape, b, bshape):
        self._c("lc_bcast_update", I(op), P(a.ptr), _ints(ashape), P(b.ptr), _ints(bshape), I(len(ashape)))

    def scalar_op(self, op, x, s, n, out=None):
        res = out if out is not None else self.mallocArray(n)
        self._c("lc_scalar_op", I(op), P(x.ptr), P(res.ptr), F(s), L(n))
        return res

    def geam(self, x, alpha, y, beta, out, n): self._c("lc_geam", P(x.ptr), F(alpha), P(y.ptr), F(beta), P(out.ptr), L(n))

    def trans(self, x, rows, cols):
        res = self.mallocArray(rows * cols); self._c("lc_trans", P(x.ptr), P(res.ptr), I(rows), I(cols)); return res

    def trans_grad(self, xd, yd, rows, cols): self._c("lc_trans_grad", P(xd.ptr), P(yd.ptr), I(rows), I(cols))

    def permute(self, x, dims, perm):
        res = self.mallocArray(int(np.prod(dims, dtype=np.int64)))
        self._c("lc_permute", P(x.ptr), P(res.ptr), _ints(dims), _ints(perm), I(len(dims)))
        return res

    def permute_grad(self, xd, yd, dims, perm): self._c("lc_permute_grad", P(xd.ptr), P(yd.ptr), _ints(dims), _ints(perm), I(len(dims)))

    # -- conv / pool / bn ---------------------------------------------------------------------------------
    def conv2D_batch(self, x, w, bias, N, C_, H, W, K, R, S, sH, sW, pH, pW):
        Pp, Q = conv_size(H, R, sH, pH), conv_size(W, S, sW, pW)
        y = self.mallocArray(N * K * Pp * Q)
        finput = self.mallocArray(N * C_ * R * S * Pp * Q)
        self._c("lc_conv2d_fwd", P(x.ptr), P(w.ptr), P(bias.ptr if bias is not None else 0), P(y.ptr), P(finput.ptr),
                *[I(v) for v in (N, C_, H, W, K, R, S, sH, sW, pH, pW)])
        return y, finput

    def conv2D_batch_grad(self, x, xd, x_in, finput, w, wd, dy, bd, N, C_, H, W, K, R, S, sH, sW, pH, pW, beta_dx=1.0):
        Pp, Q = conv_size(H, R, sH, pH), conv_size(W, S, sW, pW)
        scratch = None if x_in else self.mallocArray(N * C_ * R * S * Pp * Q)
        if finput is None:      # the caller kept no unfolded input (the forward wrote into its own buffer): unfold again
            _, finput = self.conv2D_batch(x, w, None, N, C_, H, W, K, R, S, sH, sW, pH, pW)
        self._c("lc_conv2d_bwd", P(finput.ptr), P(w.ptr), P(dy.ptr), P(0 if x_in else xd.ptr), P(wd.ptr), P(bd.ptr if bd is not None else 0),
                P(0 if x_in else scratch.ptr), *[I(v) for v in (N, C_, H, W, K, R, S, sH, sW, pH, pW)])

    def maxPool2D_batch(self, x, N, C_, H, W, kH, kW, sH, sW, pad):
        Pp, Q = conv_size(H, kH, sH, pad), conv_size(W, kW, sW, pad)
        y = self.mallocArray(N * C_ * Pp * Q); idx = self.mallocArray(N * C_ * Pp * Q)
        self._c("lc_maxpool_fwd", P(x.ptr), P(y.ptr), P(idx.ptr), *[I(v) for v in (N, C_, H, W, kH, kW, sH, sW, pad)])
        return y, idx

    def maxPool2D_batch_grad(self, xd, dy, idx, n_out, geom=None, beta=1.0): self._c("lc_maxpool_bwd", P(dy.ptr), P(idx.ptr), P(xd.ptr), L(n_out))

    def averagePool2D_batch(self, x, N, C_, H, W, kH, kW, sH, sW, pH=0, pW=0):
        y = self.mallocArray(N * C_ * conv_size(H, kH, sH, pH) * conv_size(W, kW, sW, pW))
        if pH or pW: self._c("lc_avgpool_pad_fwd", P(x.ptr), P(y.ptr), *[I(v) for v in (N, C_, H, W, kH, kW, sH, sW, pH, pW)])
        else: self._c("lc_avgpool_fwd", P(x.ptr), P(y.ptr), *[I(v) for v in (N, C_, H, W, kH, kW, sH, sW)])
        return y

    def averagePool2D_batch_grad(self, xd, dy, N, C_, H, W, kH, kW, sH, sW, pH=0, pW=0):
        if pH or pW: self._c("lc_avgpool_pad_bwd", P(dy.ptr), P(xd.ptr), *[I(v) for v in (N, C_, H, W, kH, kW, sH, sW, pH, pW)])
        else: self._c("lc_avgpool_bwd", P(dy.ptr), P(xd.ptr), *[I(v) for v in (N, C_, H, W, kH, kW, sH, sW)])

    def batchNormInference(self, x, scale, bias, rmean, rvar, N, C_, HW, eps=1e-5):
        y = self.mallocArray(N * C_ * HW)
        self._c("lc_bn_infer", P(x.ptr), P(scale.ptr), P(bias.ptr), P(rmean.ptr), P(rvar.ptr), P(y.ptr), I(N), I(C_), I(HW), F(eps))
        return y

    def batchNormTraining(self, x, scale, bias, rmean, rvar, N, C_, HW, eps=1e-5, factor=0.1):
        y = self.mallocArray(N * C_ * HW); sm = self.mallocArray(C_); si = self.mallocArray(C_)
        self._c("lc_bn_train_fwd", P(x.ptr), P(scale.ptr), P(bias.ptr), P(rmean.ptr), P(rvar.ptr), P(y.ptr), P(sm.ptr), P(si.ptr),
                I(N), I(C_), I(HW), F(eps), F(factor))
        return y, sm, si

    def batchNorm_grad(self, x, xd, dy, scale, scaled, biasd, sm, si, N, C_, HW, beta_dx=1.0, y_relu=None, bias=None):
        if y_relu is not None:      # the unfused sequence: relu_grad(inPlace) on dy, then batchNorm_grad
            self.unary_grad(0, y_relu, y_relu, dy, dy, N * C_ * HW, inPlace=True)
        self._c("lc_bn_bwd", P(x.ptr), P(dy.ptr), P(scale.ptr), P(sm.ptr), P(si.ptr), P(xd.ptr if xd is not None else 0),
                P(scaled.ptr), P(biasd.ptr), I(N), I(C_), I(HW))

    def dropout(self, x, n, prob):
        if not (0.0 <= prob < 1.0):
            raise ValueError("dropout rate should be [0.0, 1), got %s" % prob)
        y = self.mallocArray(n); mask = self.mallocArray(n)
        if self.dropout_mode == "rand":
            self._c("lc_dropout_rand", P(x.ptr), P(y.ptr), P(mask.ptr), L(n), F(prob))
        else:
            self._c("lc_dropout_ctr", P(x.ptr), P(y.ptr), P(mask.ptr), L(n), F(prob), U64(self.dropout_seed), U64(self.dropout_offset))
            self.dropout_offset += n
        return y, mask

    def dropout_grad(self, xd, dy, mask, n): self._c("lc_dropout_bwd", P(dy.ptr), P(mask.ptr), P(xd.ptr), L(n))
    def mask4D(self, x, lengths, n, c, d, t): self._c("lc_mask4d", P(x.ptr), P(lengths.ptr), I(n), I(c), I(d), I(t))

    def unary(self, op, x, n, inPlace=False, lo=-1.0, hi=1.0):
        y = x if inPlace else self.mallocArray(n)
        self._c("lc_unary", I(op), P(x.ptr), P(y.ptr), L(n), F(lo), F(hi))
        return y

    def unary_grad(self, op, x, y, dy, dx, n, inPlace=False, lo=-1.0, hi=1.0):
        self._c("lc_unary_grad", I(op), P(x.ptr), P(y.ptr), P(dy.ptr), P(dx.ptr), L(n), I(int(inPlace)), F(lo), F(hi))

    def softmax(self, is_log, x, outer, c, inner):
        y = self.mallocArray(outer * c * inner)
        self._c("lc_softmax3", I(int(is_log)), P(x.ptr), P(y.ptr), I(outer), I(c), I(inner))
        return y

    def softmax_grad(self, is_log, y, dy, dx, outer, c, inner):
        self._c("lc_softmax3_grad", I(int(is_log)), P(y.ptr), P(dy.ptr), P(dx.ptr), I(outer), I(c), I(inner))

    def nllLoss(self, x, target, batch, stride):
        y = self.mallocArray(batch); self._c("lc_nll", P(x.ptr), P(target.ptr), P(y.ptr), I(batch), I(stride)); return y

    def nllLoss_grad(self, dx, target, dy, batch, stride): self._c("lc_nll_grad", P(dx.ptr), P(target.ptr), P(dy.ptr), I(batch), I(stride))

    def sum(self, x, n):
        y = self.mallocArray(1); self._c("lc_sum_all", P(x.ptr), P(y.ptr), L(n)); return y

    def mean(self, x, n):
        y = self.mallocArray(1); self._c("lc_mean_all", P(x.ptr), P(y.ptr), L(n)); return y

    def add_scalar_from(self, dx, dy1, scale, n): self._c("lc_add_scalar_from", P(dx.ptr), P(dy1.ptr), F(scale), L(n))

    def sum_dim(self, x, outer, dim, inner):
        y = self.mallocArray(outer * inner); self._c("lc_sum_dim", P(x.ptr), P(y.ptr), I(outer), I(dim), I(inner)); return y

    def sum_dim_grad(self, dx, dy, outer, dim, inner): self._c("lc_sum_dim_grad", P(dx.ptr), P(dy.ptr), I(outer), I(dim), I(inner))

    def concat(self, bufs, sizes, outer, inner):
        res = self.mallocArray(outer * inner * sum(sizes))
        ptrs = (C.c_void_p * len(bufs))(*[b.ptr for b in bufs])
        self._c("lc_concat", I(len(bufs)), ptrs, _ints(sizes), P(res.ptr), I(outer), I(inner))
        return res

    def concat_grad(self, dbufs, sizes, outd, outer, inner, betas=None):      # host memory starts at zero: overwrite = accumulate
        # the oracle has no isInput skip: give inputs a throw-away gradient
        keep = [b if b is not None else self.mallocArray(outer * inner * s) for b, s in zip(dbufs, sizes)]
        ptrs = (C.c_void_p * len(keep))(*[b.ptr for b in keep])
        self._c("lc_concat_grad", I(len(keep)), ptrs, _ints(sizes), P(outd.ptr), I(outer), I(inner))

    def ctcLoss(self, probs, probs_d, input_lengths, labels, label_lengths, T, B, A):
        """probs [T,B,A] after softmax; lengths and labels are host int arrays; returns per-sample costs [B]."""
        costs = self.mallocArray(B)
        il = np.ascontiguousarray(input_lengths, np.int32); lb = np.ascontiguousarray(labels, np.int32); ll = np.ascontiguousarray(label_lengths, np.int32)
        self._c("lc_ctc_loss", P(probs.ptr), P(probs_d.ptr if probs_d is not None else 0), P(lb.ctypes.data), P(ll.ctypes.data), P(il.ctypes.data),
                P(costs.ptr), I(T), I(B), I(A))
        return costs

    def rnn_forward(self, mode, x, w, T, B, I_, H, bidir, hx=None):
        y = self.mallocArray(T * B * H * (2 if bidir else 1))
        self._c("lc_rnn_fwd_init", I(mode), P(x.ptr), P(hx.ptr if hx is not None else 0), P(w.ptr), P(y.ptr), I(T), I(B), I(I_), I(H), I(int(bidir)))
        return y

    def rnn_backward(self, mode, x, y, dy, w, dx, dw, T, B, I_, H, bidir, beta_dx=1.0, hx=None):
        self._c("lc_rnn_bwd_init", I(mode), P(x.ptr), P(hx.ptr if hx is not None else 0), P(y.ptr), P(dy.ptr), P(w.ptr), P(dx.ptr if dx is not None else 0),
                P(dw.ptr), I(T), I(B), I(I_), I(H), I(int(bidir)))

    def repeat0(self, x, rows, context, inner):
        y = self.mallocArray((rows - context) * (context + 1) * inner)
        self._c("lc_repeat0", P(x.ptr), P(y.ptr), I(rows), I(context), L(inner))
        return y

    def repeat0_grad(self, xd, yd, rows, context, inner):
        self._c("lc_repeat0_grad", P(xd.ptr), P(yd.ptr), I(rows), I(context), L(inner))

    def rnn_gated_forward(self, mode, x, w, T, B, I_, H, bidir, hx=None, cx=None):
        y = self.mallocArray(T * B * H * (2 if bidir else 1))
        self._c("lc_rnn_gated_fwd_init", I(mode), P(x.ptr), P(hx.ptr if hx is not None else 0), P(cx.ptr if cx is not None else 0), P(w.ptr), P(y.ptr),
                I(T), I(B), I(I_), I(H), I(int(bidir)))
        return y, None

    def rnn_gated_backward(self, mode, x, y, dy, w, reserve, dx, dw, T, B, I_, H, bidir, beta_dx=1.0, hx=None, cx=None):
        self._c("lc_rnn_gated_bwd_init", I(mode), P(x.ptr), P(hx.ptr if hx is not None else 0), P(cx.ptr if cx is not None else 0), P(dy.ptr), P(w.ptr),
                P(dx.ptr if dx is not None else 0), P(dw.ptr), I(T), I(B), I(I_), I(H), I(int(bidir)))

    def sgd_update(self, x, d, lr, n): self._c("lc_sgd", P(x.ptr), P(d.ptr), F(lr), L(n))
    def adagrad_update(self, x, d, m, lr, clip, n): self._c("lc_adagrad", P(x.ptr), P(d.ptr), P(m.ptr), F(lr), F(clip), L(n))
    def momentum_update(self, x, d, v, lr, mu, clip, nesterov, n):
        self._c("lc_momentum", P(x.ptr), P(d.ptr), P(v.ptr), F(lr), F(mu), F(clip), I(int(nesterov)), L(n))

    def multi_momentum_update(self, params, lr, mu, clip, nesterov):
        for x, d, v, n in params: self.momentum_update(x, d, v, lr, mu, clip, nesterov, n)

    def multi_sgd_update(self, params, lr):
        for x, d, n in params: self.sgd_update(x, d, lr, n)
