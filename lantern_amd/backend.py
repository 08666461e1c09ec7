"""Host-side mirror of Lantern's `Backend` trait and its MI355X implementation, BackendHIP.

Reference: src/main/scala/lantern/TensorDifferentiation.scala:137-379 (the trait) and the slot
BackendCudnn occupies (src/main/scala/lantern/TensorDslCudnn.scala:142-1939).  Method names and
argument meaning follow the trait; Scala's symbolic methods are spelled out
(`+` -> add, `-` -> sub, `*` -> mul, `/` -> div, `+=` -> add_inplace, ...).

In the reference these methods run on the JVM at staging time and emit C++ text; here the same
calls are issued directly, one C-ABI call (include/lantern_hip.h) per emitted call.
"""
import ctypes as C
import os

import numpy as np

from . import _lib

ADD, SUB, MUL, DIV = 0, 1, 2, 3
RELU, TANH, SIGMOID, EXP, LOG, SQRT, SQUARE, HARDTANH = range(8)


class Buf:
    """A span of backend memory: address, element count (4-byte elements) and an owner to keep alive."""
    __slots__ = ("ptr", "n", "keep")

    def __init__(self, ptr, n, keep=None):
        self.ptr = int(ptr)
        self.n = int(n)
        self.keep = keep

    def offset(self, k, n=None):
        """`slice(arr, off)` of the reference (TD:55): same memory, starting k elements in."""
        return Buf(self.ptr + 4 * int(k), self.n - int(k) if n is None else n, self.keep)


_INTS_CACHE = {}


def _ints(seq):
    """A C int array of the values (shape and permutation arguments); the arrays are read-only, so equal tuples share one."""
    key = tuple(seq)
    arr = _INTS_CACHE.get(key)
    if arr is None:
        arr = (C.c_int * len(key))(*[int(v) for v in key])
        if len(_INTS_CACHE) < 4096:
            _INTS_CACHE[key] = arr
    return arr


def dim_broadcast(a, b):
    """Tensor.dimBroadcast (TD:997-1016): right-aligned numpy rules -> (aShape, bShape, resShape)."""
    a, b = list(a), list(b)
    r = max(len(a), len(b))
    a = [1] * (r - len(a)) + a
    b = [1] * (r - len(b)) + b
    res = []
    for x, y in zip(a, b):
        if not (x == 1 or y == 1 or x == y):
            raise ValueError("dimensions not compatible for broadcasting %s with %s" % (a, b))
        res.append(max(x, y))
    return tuple(a), tuple(b), tuple(res)


def conv_size(size, kernel, stride, pad=0):
    """convSize (TD:34)."""
    return (size + 2 * pad - kernel) // stride + 1


class Backend:
    """Operator API (TD:137-379).  Tensors are passed as objects with `.data` (Buf) and `.shape`."""

    name = "abstract"
    convs_open = 0    # kept by the tape: forward convolutions whose gradient call is still to come

    # -- memory ---------------------------------------------------------------------------
    def setup(self): raise NotImplementedError
    def cleanup(self): raise NotImplementedError
    def mallocArray(self, length, zero=True): raise NotImplementedError     # TD:145
    def copyFloatArray(self, dest, src, length): raise NotImplementedError  # TD:150
    def fromHost(self, arr): raise NotImplementedError                      # toGPU (CUB:37-66)
    def toHost(self, buf, n, dtype=np.float32): raise NotImplementedError   # toCPU (CUB:68-107)
    def getMallocAddr(self): raise NotImplementedError                      # TD:1782-1784 / CUB:18-20
    def resetMallocAddr(self, addr): raise NotImplementedError              # TD:1786-1789 / CUB:22-25

    # -- the library's fused entry points, callable directly (tests, hand-fused front ends); the defaults are the sequences
    #    of trait calls they stand for.  The TensorR front end does not use them: it issues one trait call per operator. ----
    def batchNormTraining_into(self, x, scale, bias, rmean, rvar, y, sm, si, N, C, HW, relu, eps=1e-5, factor=0.1):
        """batchNormTraining writing into caller-provided y / saveMean / saveInvStd, optionally followed by relu(inPlace)."""
        yy, m, v = self.batchNormTraining(x, scale, bias, rmean, rvar, N, C, HW, eps, factor)
        self.copyFloatArray(y, yy, N * C * HW); self.copyFloatArray(sm, m, C); self.copyFloatArray(si, v, C)
        if relu:
            self.unary(RELU, y, N * C * HW, inPlace=True)

    def add_into(self, a, b, out, n, relu):
        self.geam(a, 1.0, b, 1.0, out, n)
        if relu:
            self.unary(RELU, out, n, inPlace=True)

    # out = relu(batchNorm(x) + shortcut): the unfused sequence batchNorm -> + -> relu(inPlace)
    def batchNormTraining_add_relu_into(self, x, scale, bias, rmean, rvar, shortcut, out, sm, si, N, C, HW, eps=1e-5, factor=0.1):
        self.batchNormTraining_into(x, scale, bias, rmean, rvar, out, sm, si, N, C, HW, False, eps, factor)
        self.add_into(out, shortcut, out, N * C * HW, True)

    def conv2D_batch_bn_add_relu_into(self, x, w, bias, yconv, dims, scale, bbias, rmean, rvar, shortcut, out, sm, si, eps=1e-5, factor=0.1):
        N, C, H, W, K, R, S, sH, sW, pH, pW = dims
        finput = self.conv2D_batch_into(x, w, bias, yconv, *dims)
        HW = conv_size(H, R, sH, pH) * conv_size(W, S, sW, pW)
        self.batchNormTraining_add_relu_into(yconv, scale, bbias, rmean, rvar, shortcut, out, sm, si, N, K, HW, eps, factor)
        return finput

    def batchNorm_add_relu_grad(self, x, xd, beta_dx, out, dout, scale, scaled, biasd, sm, si, sd, beta_sd, N, C, HW):
        """Backward of out = relu(batchNorm(x) + shortcut): relu_grad(inPlace) masks dout, the shortcut's gradient takes it,
        batchNorm_grad does the rest.  dout is overwritten."""
        n = N * C * HW
        self.unary_grad(RELU, out, out, dout, dout, n, inPlace=True)
        if sd is not None:
            if beta_sd == 0.0: self.copyFloatArray(sd, dout, n)
            else: self.geam(sd, 1.0, dout, 1.0, sd, n)
        self.batchNorm_grad(x, xd, dout, scale, scaled, biasd, sm, si, N, C, HW, beta_dx)

    def conv2D_batch_into(self, x, w, bias, y, N, C, H, W, K, R, S, sH, sW, pH, pW):
        """conv2D_batch writing into a caller-provided y; returns the unfolded input if the backend keeps one (CPU:532-571)."""
        yy, finput = self.conv2D_batch(x, w, bias, N, C, H, W, K, R, S, sH, sW, pH, pW)
        self.copyFloatArray(y, yy, N * K * conv_size(H, R, sH, pH) * conv_size(W, S, sW, pW))
        return finput

    def conv2D_batch_bn_into(self, x, w, bias, yconv, dims, scale, bbias, rmean, rvar, ybn, sm, si, relu, eps=1e-5, factor=0.1):
        """conv2D_batch followed by batchNormTraining of its output (and relu): the unfused sequence."""
        N, C, H, W, K, R, S, sH, sW, pH, pW = dims
        finput = self.conv2D_batch_into(x, w, bias, yconv, *dims)
        HW = conv_size(H, R, sH, pH) * conv_size(W, S, sW, pW)
        self.batchNormTraining_into(yconv, scale, bbias, rmean, rvar, ybn, sm, si, N, K, HW, relu, eps, factor)
        return finput

    def add_relu_grad(self, y, dy, ad, abeta, bd, bbeta, n):
        self.unary_grad(RELU, y, y, dy, dy, n, inPlace=True)            # masks dy in place (CPU:725-726 with the y > 0 mask)
        for d in (ad, bd):
            if d is not None:
                self.geam(d, 1.0, dy, 1.0, d, n)                        # buffers from mallocArray start at zero


class BackendHIP(Backend):
    """The MI355X backend: every method is one or a few calls into liblantern_hip.so.

    Errors raise LanternHipError (the library runs in "record and return" mode under Python;
    generated C++ hosts keep the reference's print-and-exit behaviour).
    """

    name = "hip"

    def __init__(self, heap_bytes=8 << 30):
        self.heap_bytes = int(heap_bytes)
        self.lib = None
        self.dropout_seed = 42
        self.side_order = int(os.environ.get("LH_SIDE_ORDER", "1"))
        self.side_min_convs = int(os.environ.get("LH_SIDE_MIN_CONVS", "2"))
        self.dropout_offset = 0
        self.work = {}            # algorithmic flop / bytes issued, by kind, while count_work is on (the benchmark's profiled pass)
        self.count_work = False

    def _count(self, kind, amount):
        self.work[kind] = self.work.get(kind, 0.0) + amount

    # -- lifetime / arena -------------------------------------------------------------------
    def setup(self):
        self.lib = _lib.load()
        self.lib.lh_set_error_mode(1)
        self.lib.lh_setup(self.heap_bytes)
        _lib.check()
        self._chunk_ptr, self._chunk_left = 0, 0

    def cleanup(self):
        if self.lib is not None:
            self.lib.lh_cleanup()
            for p in getattr(self, "_pinned", []):
                self.lib.lh_host_free(p)
            self._pinned = []
            self.lib = None

    def sync(self):
        self.lib.lh_sync(); _lib.check()

    def setDeterministic(self, on=True):
        """Fixed-order reductions and rule-chosen launch plans: two runs of the same program give the same bits."""
        self.lib.lh_set_deterministic(1 if on else 0); _lib.check()

    def captureBegin(self):
        """Record everything issued until captureEnd() into a HIP graph instead of running it."""
        self.lib.lh_capture_begin(); _lib.check()

    def captureEnd(self):
        g = self.lib.lh_capture_end(); _lib.check()
        return g

    def graphLaunch(self, g):
        self.lib.lh_graph_launch(g); _lib.check()

    def graphDestroy(self, g):
        self.lib.lh_graph_destroy(g); _lib.check()

    def batchSmallOps(self, on=True):
        """Record small operations into the library's command list instead of launching each (launch-bound programs)."""
        (self.lib.lh_cmdlist_begin if on else self.lib.lh_cmdlist_end)(); _lib.check()

    def cmdlistStats(self):
        rec, launches = C.c_int64(0), C.c_int64(0)
        self.lib.lh_cmdlist_stats(C.byref(rec), C.byref(launches))
        return rec.value, launches.value

    def mallocArray(self, length, zero=True):
        n = int(length) if length > 0 else 1
        nb = (4 * n + 255) & -256
        if nb <= self.SMALL_BLOCK:
            # Small blocks are cut from a zero-filled 1 MiB block of the arena on this side of the boundary: a TreeLSTM
            # tree asks for ~1900 blocks of a few hundred bytes, and a foreign call costs more than everything else
            # this method does.  Generated C++ calls lh_malloc directly.
            if nb > self._chunk_left:
                self._chunk_ptr = self.lib.lh_malloc(self.CHUNK)
                _lib.check()
                self._chunk_left = self.CHUNK
            p = self._chunk_ptr
            self._chunk_ptr = p + nb
            self._chunk_left -= nb
            return Buf(p, n)
        p = (self.lib.lh_malloc if zero else self.lib.lh_malloc_uninit)(4 * n)
        _lib.check()
        return Buf(p, n)

    SMALL_BLOCK = 1 << 16
    CHUNK = 1 << 20

    def getMallocAddr(self):
        self._chunk_left = 0        # what is handed out from here on lies above the mark
        return self.lib.lh_mark()

    def resetMallocAddr(self, addr):
        self._chunk_left = 0
        self.lib.lh_rewind(addr); _lib.check()

    def copyFloatArray(self, dest, src, length):
        self.lib.lh_d2d(dest.ptr, src.ptr, 4 * int(length)); _lib.check()

    def fromHost(self, arr):
        arr = np.ascontiguousarray(arr)
        assert arr.dtype.itemsize == 4, "only 4-byte element types cross the boundary"
        buf = self.mallocArray(arr.size)
        if arr.size:
            self.lib.lh_h2d(buf.ptr, arr.ctypes.data, arr.nbytes); _lib.check()
        return buf

    def toHost(self, buf, n, dtype=np.float32):
        out = np.empty(int(n), dtype=dtype)
        if n:
            self.lib.lh_d2h(out.ctypes.data, buf.ptr, out.nbytes); _lib.check()
        return out

    def upload(self, buf, arr):
        arr = np.ascontiguousarray(arr)
        self.lib.lh_h2d(buf.ptr, arr.ctypes.data, arr.nbytes); _lib.check()

    # -- transfers that do not stall the step (pinned host memory, copy stream, deferred read-back) ----------
    def hostArray(self, shape, dtype=np.float32):
        """A numpy array over pinned host memory (freed by cleanup())."""
        n = int(np.prod(shape, dtype=np.int64)) * np.dtype(dtype).itemsize
        p = self.lib.lh_host_alloc(n); _lib.check()
        self._pinned = getattr(self, "_pinned", [])
        self._pinned.append(p)
        return np.ctypeslib.as_array((C.c_byte * n).from_address(p)).view(dtype).reshape(shape)

    def uploadAsync(self, buf, pinned_arr):
        """Upload on the copy stream: after everything issued so far, beside everything issued from now on (copyJoin before use)."""
        self.lib.lh_h2d_async(buf.ptr, pinned_arr.ctypes.data, pinned_arr.nbytes); _lib.check()

    def copyJoin(self):
        self.lib.lh_copy_join(); _lib.check()

    def downloadAsync(self, pinned_arr, buf):
        """Read-back that returns at once; the values are there after the next sync()."""
        self.lib.lh_d2h_async(pinned_arr.ctypes.data, buf.ptr, pinned_arr.nbytes); _lib.check()

    # -- fills ------------------------------------------------------------------------------
    def fillInPlace(self, data, n, value):
        self.lib.lh_fill(data.ptr, value, n); _lib.check()

    def fillWithBias(self, dims, bias, dim):
        outer = int(np.prod(dims[:dim], dtype=np.int64)); c = dims[dim]; inner = int(np.prod(dims[dim + 1:], dtype=np.int64))
        res = self.mallocArray(outer * c * inner)
        self.lib.lh_fill_with_bias(res.ptr, bias.ptr, outer, c, inner); _lib.check()
        return res

    def clipAt(self, data, n, bound):
        self.lib.lh_clip(data.ptr, bound, n); _lib.check()

    # -- dot family (TD:186-219; CUB:173-282) -----------------------------------------------
    def vectorVectorDot(self, x, y, n):
        res = self.mallocArray(1)
        self.lib.lh_dot_vv(x.ptr, y.ptr, res.ptr, n); _lib.check()
        return res

    def matrixVectorDot(self, x, y, m, n):
        res = self.mallocArray(m)
        self.lib.lh_sgemv(0, m, n, 1.0, x.ptr, n, y.ptr, 0.0, res.ptr); _lib.check()
        if self.count_work: self._count("gemv_flop", 2.0 * m * n); self._count("gemv_bytes", 4.0 * m * n)
        return res

    def matrixMatrixDot(self, x, y, m, k, n):
        res = self.mallocArray(m * n)
        self.lib.lh_sgemm(0, 0, m, n, k, 1.0, x.ptr, k, y.ptr, n, 0.0, res.ptr, n); _lib.check()
        if self.count_work: self._count("gemm_flop", 2.0 * m * n * k)
        return res

    def addMul_scalar(self, xd, s, y, n):           # x.d.addMul(output.d.data(0), y.x)  (CPU:174-175)
        self.lib.lh_axpy_dev(xd.ptr, s.ptr, y.ptr, n); _lib.check()

    def add_cartesian(self, xd, y, outd, m, n):     # xd[m,n] += outd[m] (x) y[n]
        self.lib.lh_ger(m, n, outd.ptr, y.ptr, xd.ptr); _lib.check()
        if self.count_work: self._count("gemv_flop", 2.0 * m * n); self._count("gemv_bytes", 8.0 * m * n)

    def add_composition(self, xd, y, outd, m, n):   # xd[n] += y[m,n]^T outd[m]
        self.lib.lh_sgemv(1, m, n, 1.0, y.ptr, n, outd.ptr, 1.0, xd.ptr); _lib.check()
        if self.count_work: self._count("gemv_flop", 2.0 * m * n); self._count("gemv_bytes", 4.0 * m * n)

    def add_dotTrans1(self, xd, y, outd, d1, d2, d3):  # xd[d2,d3] += y[d1,d2]^T outd[d1,d3]
        self.lib.lh_sgemm(1, 0, d2, d3, d1, 1.0, y.ptr, d2, outd.ptr, d3, 1.0, xd.ptr, d3); _lib.check()
        if self.count_work: self._count("gemm_flop", 2.0 * d1 * d2 * d3)

    def add_dotTrans2(self, xd, y, outd, d1, d2, d3):  # xd[d1,d2] += y[d1,d3] outd[d2,d3]^T
        self.lib.lh_sgemm(0, 1, d1, d2, d3, 1.0, y.ptr, d3, outd.ptr, d3, 1.0, xd.ptr, d2); _lib.check()
        if self.count_work: self._count("gemm_flop", 2.0 * d1 * d2 * d3)

    # -- gemm (TD:279-280; CUB:589-688): result [d1,d3], contraction d2 --------------------------
    def gemm(self, x, tx, y, ty, alpha, d1, d2, d3):
        res = self.mallocArray(d1 * d3)
        self.lib.lh_sgemm(int(tx), int(ty), d1, d3, d2, alpha, x.ptr, d1 if tx else d2, y.ptr, d2 if ty else d3, 0.0, res.ptr, d3)
        _lib.check()
        if self.count_work: self._count("gemm_flop", 2.0 * d1 * d2 * d3)
        return res

    def gemm_grad(self, x, xd, x_in, tx, y, yd, y_in, ty, alpha, od, d1, d2, d3, xbeta=1.0, ybeta=1.0):
        """CUB:630-688; beta = 0 overwrites a gradient buffer that has no content yet."""
        g = self.lib.lh_sgemm
        if not tx and not ty:
            if not x_in: g(0, 1, d1, d2, d3, alpha, od.ptr, d3, y.ptr, d3, xbeta, xd.ptr, d2)
            if not y_in: g(1, 0, d2, d3, d1, alpha, x.ptr, d2, od.ptr, d3, ybeta, yd.ptr, d3)
        elif not tx and ty:
            if not x_in: g(0, 0, d1, d2, d3, alpha, od.ptr, d3, y.ptr, d2, xbeta, xd.ptr, d2)
            if not y_in: g(1, 0, d3, d2, d1, alpha, od.ptr, d3, x.ptr, d2, ybeta, yd.ptr, d2)
        elif tx and not ty:
            if not x_in: g(0, 1, d2, d1, d3, alpha, y.ptr, d3, od.ptr, d3, xbeta, xd.ptr, d1)
            if not y_in: g(0, 0, d2, d3, d1, alpha, x.ptr, d1, od.ptr, d3, ybeta, yd.ptr, d3)
        else:
            if not x_in: g(1, 1, d2, d1, d3, alpha, y.ptr, d2, od.ptr, d3, xbeta, xd.ptr, d1)
            if not y_in: g(1, 1, d3, d2, d1, alpha, od.ptr, d3, x.ptr, d1, ybeta, yd.ptr, d2)
        _lib.check()
        if self.count_work: self._count("gemm_flop", 2.0 * d1 * d2 * d3 * ((not x_in) + (not y_in)))

    # -- broadcast arithmetic (TD:222-270) ---------------------------------------------------------
    def bcast_op(self, op, a, ashape, b, bshape, oshape):
        n = int(np.prod(oshape, dtype=np.int64))
        res = self.mallocArray(n)
        self.lib.lh_bcast_op(op, a.ptr, _ints(ashape), b.ptr, _ints(bshape), res.ptr, _ints(oshape), len(oshape)); _lib.check()
        return res

    def bcast_op_grad(self, op, a, ad, ashape, a_in, b, bd, bshape, b_in, od, oshape):
        self.lib.lh_bcast_op_grad(op, a.ptr, 0 if a_in else ad.ptr, _ints(ashape), int(a_in), b.ptr, 0 if b_in else bd.ptr, _ints(bshape), int(b_in),
                                  od.ptr, _ints(oshape), len(oshape)); _lib.check()

    def bcast_update(self, op, a, ashape, b, bshape):
        self.lib.lh_bcast_update(op, a.ptr, _ints(ashape), b.ptr, _ints(bshape), len(ashape)); _lib.check()

    def scalar_op(self, op, x, s, n, out=None):
        res = out if out is not None else self.mallocArray(n)
        self.lib.lh_scalar_op(op, x.ptr, res.ptr, s, n); _lib.check()
        return res

    def geam(self, x, alpha, y, beta, out, n):
        self.lib.lh_geam(x.ptr, alpha, y.ptr, beta, out.ptr, n); _lib.check()

    def trans(self, x, rows, cols):
        res = self.mallocArray(rows * cols)
        self.lib.lh_trans(x.ptr, res.ptr, rows, cols); _lib.check()
        return res

    def trans_grad(self, xd, yd, rows, cols):
        self.lib.lh_trans_grad(xd.ptr, yd.ptr, rows, cols); _lib.check()

    def permute(self, x, dims, perm):
        res = self.mallocArray(int(np.prod(dims, dtype=np.int64)))
        self.lib.lh_permute(x.ptr, res.ptr, _ints(dims), _ints(perm), len(dims)); _lib.check()
        return res

    def permute_grad(self, xd, yd, dims, perm):
        self.lib.lh_permute_grad(xd.ptr, yd.ptr, _ints(dims), _ints(perm), len(dims)); _lib.check()

    # -- conv / pool / bn ---------------------------------------------------------------------------
    def conv2D_batch(self, x, w, bias, N, C, H, W, K, R, S, sH, sW, pH, pW):
        P, Q = conv_size(H, R, sH, pH), conv_size(W, S, sW, pW)
        y = self.mallocArray(N * K * P * Q)
        self.lib.lh_conv2d_fwd(x.ptr, w.ptr, bias.ptr if bias is not None else 0, y.ptr, N, C, H, W, K, R, S, sH, sW, pH, pW); _lib.check()
        if self.count_work: self._count("conv_flop", 2.0 * N * K * C * R * S * P * Q)
        return y, None      # no im2col buffer is kept (BackendCudnn returns None too, CDN:859-866)

    def conv2D_batch_into(self, x, w, bias, y, N, C, H, W, K, R, S, sH, sW, pH, pW):
        self.lib.lh_conv2d_fwd(x.ptr, w.ptr, bias.ptr if bias is not None else 0, y.ptr, N, C, H, W, K, R, S, sH, sW, pH, pW); _lib.check()
        if self.count_work: self._count("conv_flop", 2.0 * N * K * C * R * S * conv_size(H, R, sH, pH) * conv_size(W, S, sW, pW))

    def conv2D_batch_bn_into(self, x, w, bias, yconv, dims, scale, bbias, rmean, rvar, ybn, sm, si, relu, eps=1e-5, factor=0.1):
        N, C, H, W, K, R, S, sH, sW, pH, pW = dims
        HW = conv_size(H, R, sH, pH) * conv_size(W, S, sW, pW)
        self.lib.lh_conv2d_fwd_bn_apply(x.ptr, w.ptr, bias.ptr if bias is not None else 0, yconv.ptr, *dims, scale.ptr, bbias.ptr, sm.ptr, si.ptr,
                                        rmean.ptr, rvar.ptr, eps, factor, 0, ybn.ptr, int(relu)); _lib.check()
        if self.count_work: self._count("conv_flop", 2.0 * N * K * C * R * S * HW)

    def conv2D_batch_grad(self, x, xd, x_in, finput, w, wd, dy, bd, N, C, H, W, K, R, S, sH, sW, pH, pW, beta_dx=1.0):
        # The filter gradient is read by the optimizer only: it goes to the side stream, where it runs beside the
        # rest of the backward pass (x and dy stay untouched until the optimizer joins).  The input gradient, which
        # the next backward operator waits for, is issued first and stays on the main stream.
        so = self.side_order
        if x_in or self.convs_open < self.side_min_convs:
            so = 0      # (almost) nothing left to run beside it (fewer than two convolution gradients follow): the optimizer's join would only add the cross-stream hand-over
        # With a bias the filter gradient goes first in any case: its bias sums are the first reader of dy, and a relu_grad(in place)
        # issued just before is applied in that pass.
        first = so == 2 or bd is not None
        if first:
            if so: self.lib.lh_side_begin()
            self.lib.lh_conv2d_bwd_filter(x.ptr, dy.ptr, wd.ptr, bd.ptr if bd is not None else 0, 1.0, N, C, H, W, K, R, S, sH, sW, pH, pW)
            if so: self.lib.lh_side_end()
        if not x_in:
            self.lib.lh_conv2d_bwd_data(dy.ptr, w.ptr, xd.ptr, beta_dx, N, C, H, W, K, R, S, sH, sW, pH, pW)
        if not first:
            if so: self.lib.lh_side_begin()
            self.lib.lh_conv2d_bwd_filter(x.ptr, dy.ptr, wd.ptr, bd.ptr if bd is not None else 0, 1.0, N, C, H, W, K, R, S, sH, sW, pH, pW)
            if so: self.lib.lh_side_end()
        _lib.check()
        P, Q = conv_size(H, R, sH, pH), conv_size(W, S, sW, pW)
        if self.count_work: self._count("conv_flop", 2.0 * N * K * C * R * S * P * Q * (1 if x_in else 2))

    def maxPool2D_batch(self, x, N, C, H, W, kH, kW, sH, sW, pad):
        P, Q = conv_size(H, kH, sH, pad), conv_size(W, kW, sW, pad)
        y = self.mallocArray(N * C * P * Q); idx = self.mallocArray(N * C * P * Q)
        self.lib.lh_maxpool_fwd(x.ptr, y.ptr, idx.ptr, N, C, H, W, kH, kW, sH, sW, pad); _lib.check()
        return y, idx

    def maxPool2D_batch_grad(self, xd, dy, idx, n_out, geom=None, beta=1.0):
        """geom = (N, C, H, W, kH, kW, sH, sW, pad) selects the gather form, which can also overwrite (beta 0)."""
        if geom is not None:
            self.lib.lh_maxpool_bwd_dense(dy.ptr, idx.ptr, xd.ptr, beta, *geom)
        else:
            assert beta == 1.0
            self.lib.lh_maxpool_bwd(dy.ptr, idx.ptr, xd.ptr, n_out)
        _lib.check()

    def averagePool2D_batch(self, x, N, C, H, W, kH, kW, sH, sW, pH=0, pW=0):
        P, Q = conv_size(H, kH, sH, pH), conv_size(W, kW, sW, pW)
        y = self.mallocArray(N * C * P * Q)
        if pH or pW: self.lib.lh_avgpool_pad_fwd(x.ptr, y.ptr, N, C, H, W, kH, kW, sH, sW, pH, pW)
        else: self.lib.lh_avgpool_fwd(x.ptr, y.ptr, N, C, H, W, kH, kW, sH, sW)
        _lib.check()
        return y

    def averagePool2D_batch_grad(self, xd, dy, N, C, H, W, kH, kW, sH, sW, pH=0, pW=0):
        if pH or pW: self.lib.lh_avgpool_pad_bwd(dy.ptr, xd.ptr, N, C, H, W, kH, kW, sH, sW, pH, pW)
        else: self.lib.lh_avgpool_bwd(dy.ptr, xd.ptr, N, C, H, W, kH, kW, sH, sW)
        _lib.check()

    def batchNormInference(self, x, scale, bias, rmean, rvar, N, C, HW, eps=1e-5):
        y = self.mallocArray(N * C * HW)
        self.lib.lh_bn_infer(x.ptr, scale.ptr, bias.ptr, rmean.ptr, rvar.ptr, y.ptr, N, C, HW, eps); _lib.check()
        return y

    def batchNormTraining(self, x, scale, bias, rmean, rvar, N, C, HW, eps=1e-5, factor=0.1):
        y = self.mallocArray(N * C * HW)
        sm = self.mallocArray(C); si = self.mallocArray(C)
        self.lib.lh_bn_train_fwd(x.ptr, scale.ptr, bias.ptr, rmean.ptr, rvar.ptr, y.ptr, sm.ptr, si.ptr, N, C, HW, eps, factor); _lib.check()
        return y, sm, si

    def batchNormTraining_into(self, x, scale, bias, rmean, rvar, y, sm, si, N, C, HW, relu, eps=1e-5, factor=0.1):
        f = self.lib.lh_bn_train_fwd_relu if relu else self.lib.lh_bn_train_fwd
        f(x.ptr, scale.ptr, bias.ptr, rmean.ptr, rvar.ptr, y.ptr, sm.ptr, si.ptr, N, C, HW, eps, factor); _lib.check()

    def batchNorm_grad(self, x, xd, dy, scale, scaled, biasd, sm, si, N, C, HW, beta_dx=1.0, y_relu=None, bias=None):
        """y_relu: the layer's output went through a fused in-place relu; `bias` (the layer's beta) lets the
        kernel rebuild the relu mask from x instead of reading y."""
        xdp = xd.ptr if xd is not None else 0
        if y_relu is not None:
            self.lib.lh_bn_bwd_relu(x.ptr, y_relu.ptr, dy.ptr, scale.ptr, bias.ptr if bias is not None else 0, sm.ptr, si.ptr, xdp, beta_dx,
                                    scaled.ptr, biasd.ptr, N, C, HW)
        else:
            self.lib.lh_bn_bwd(x.ptr, dy.ptr, scale.ptr, sm.ptr, si.ptr, xdp, beta_dx, scaled.ptr, biasd.ptr, N, C, HW)
        _lib.check()

    def batchNormTraining_add_relu_into(self, x, scale, bias, rmean, rvar, shortcut, out, sm, si, N, C, HW, eps=1e-5, factor=0.1):
        self.lib.lh_bn_stats(x.ptr, sm.ptr, si.ptr, rmean.ptr, rvar.ptr, N, C, HW, eps, factor)
        self.lib.lh_bn_apply_add_relu(x.ptr, scale.ptr, bias.ptr, sm.ptr, si.ptr, shortcut.ptr, out.ptr, N, C, HW); _lib.check()

    def conv2D_batch_bn_add_relu_into(self, x, w, bias, yconv, dims, scale, bbias, rmean, rvar, shortcut, out, sm, si, eps=1e-5, factor=0.1):
        N, C, H, W, K, R, S, sH, sW, pH, pW = dims
        HW = conv_size(H, R, sH, pH) * conv_size(W, S, sW, pW)
        self.lib.lh_conv2d_fwd_bn_apply(x.ptr, w.ptr, bias.ptr if bias is not None else 0, yconv.ptr, *dims, scale.ptr, bbias.ptr, sm.ptr, si.ptr,
                                        rmean.ptr, rvar.ptr, eps, factor, shortcut.ptr, out.ptr, 1); _lib.check()
        if self.count_work: self._count("conv_flop", 2.0 * N * K * C * R * S * HW)

    def batchNorm_add_relu_grad(self, x, xd, beta_dx, out, dout, scale, scaled, biasd, sm, si, sd, beta_sd, N, C, HW):
        self.lib.lh_bn_bwd_add_relu(x.ptr, out.ptr, dout.ptr, scale.ptr, sm.ptr, si.ptr, xd.ptr if xd is not None else 0, beta_dx,
                                    sd.ptr if sd is not None else 0, beta_sd, scaled.ptr, biasd.ptr, N, C, HW); _lib.check()

    def add_into(self, a, b, out, n, relu):
        if relu: self.lib.lh_add_relu(a.ptr, b.ptr, out.ptr, n)
        else: self.lib.lh_geam(a.ptr, 1.0, b.ptr, 1.0, out.ptr, n)
        _lib.check()

    def add_relu_grad(self, y, dy, ad, abeta, bd, bbeta, n):
        self.lib.lh_add_relu_grad(y.ptr, dy.ptr, ad.ptr if ad is not None else 0, abeta, bd.ptr if bd is not None else 0, bbeta, n); _lib.check()

    # -- dropout ------------------------------------------------------------------------------------
    def dropout(self, x, n, prob):
        if not (0.0 <= prob < 1.0):
            raise ValueError("dropout rate should be [0.0, 1), got %s" % prob)
        y = self.mallocArray(n); mask = self.mallocArray(n)
        self.lib.lh_dropout_fwd(x.ptr, y.ptr, mask.ptr, n, prob, self.dropout_seed, self.dropout_offset); _lib.check()
        self.dropout_offset += n
        return y, mask

    def dropout_grad(self, xd, dy, mask, n):
        self.lib.lh_dropout_bwd(dy.ptr, mask.ptr, xd.ptr, n); _lib.check()

    def mask4D(self, x, lengths, n, c, d, t):
        self.lib.lh_mask4d(x.ptr, lengths.ptr, n, c, d, t); _lib.check()

    def repeat0(self, x, rows, context, inner):
        y = self.mallocArray((rows - context) * (context + 1) * inner)
        self.lib.lh_repeat0(x.ptr, y.ptr, rows, context, inner); _lib.check()
        return y

    def repeat0_grad(self, xd, yd, rows, context, inner):
        self.lib.lh_repeat0_grad(xd.ptr, yd.ptr, rows, context, inner); _lib.check()

    def cifar_decode(self, records, count):
        """records: uint8 host array [n, count + 1] (label byte, then pixels).  Uploads the bytes and decodes them on the
        device; returns (x float32 [n, count], y int32 [n]) in arena memory (TensorDataLoader.scala:109-127)."""
        records = np.ascontiguousarray(records, dtype=np.uint8)
        n = int(records.shape[0])
        assert records.ndim == 2 and records.shape[1] == count + 1, "records must be [n, count + 1] bytes"
        raw = self.mallocArray((records.nbytes + 3) // 4)
        x = self.mallocArray(n * count)
        y = self.mallocArray(n)
        if n:
            self.lib.lh_h2d(raw.ptr, records.ctypes.data, records.nbytes); _lib.check()
            self.lib.lh_cifar_decode(raw.ptr, x.ptr, y.ptr, n, count); _lib.check()
        return x, y

    # -- activations ---------------------------------------------------------------------------------
    def unary(self, op, x, n, inPlace=False, lo=-1.0, hi=1.0):
        y = x if inPlace else self.mallocArray(n)
        self.lib.lh_unary(op, x.ptr, y.ptr, n, lo, hi); _lib.check()
        return y

    def unary_grad(self, op, x, y, dy, dx, n, inPlace=False, lo=-1.0, hi=1.0):
        self.lib.lh_unary_grad(op, x.ptr, y.ptr, dy.ptr, dx.ptr, n, int(inPlace), lo, hi); _lib.check()

    # -- softmax / loss --------------------------------------------------------------------------------
    def softmax(self, is_log, x, outer, c, inner):
        y = self.mallocArray(outer * c * inner)
        self.lib.lh_softmax(int(is_log), x.ptr, y.ptr, outer, c, inner); _lib.check()
        return y

    def softmax_grad(self, is_log, y, dy, dx, outer, c, inner):
        self.lib.lh_softmax_grad(int(is_log), y.ptr, dy.ptr, dx.ptr, outer, c, inner); _lib.check()

    def nllLoss(self, x, target, batch, stride):
        y = self.mallocArray(batch)
        self.lib.lh_nll(x.ptr, target.ptr, y.ptr, batch, stride); _lib.check()
        return y

    def nllLoss_grad(self, dx, target, dy, batch, stride):
        self.lib.lh_nll_grad(dx.ptr, target.ptr, dy.ptr, batch, stride); _lib.check()

    # -- reductions -------------------------------------------------------------------------------------
    def sum(self, x, n):
        y = self.mallocArray(1)
        self.lib.lh_sum_all(x.ptr, y.ptr, n); _lib.check()
        return y

    def mean(self, x, n):
        y = self.mallocArray(1)
        self.lib.lh_mean_all(x.ptr, y.ptr, n); _lib.check()
        return y

    def add_scalar_from(self, dx, dy1, scale, n):       # sum_grad / mean_grad
        self.lib.lh_add_scalar_from(dx.ptr, dy1.ptr, scale, n); _lib.check()

    def sum_dim(self, x, outer, dim, inner):
        y = self.mallocArray(outer * inner)
        self.lib.lh_sum_dim(x.ptr, y.ptr, outer, dim, inner); _lib.check()
        return y

    def sum_dim_grad(self, dx, dy, outer, dim, inner):
        self.lib.lh_sum_dim_grad(dx.ptr, dy.ptr, outer, dim, inner); _lib.check()

    def concat(self, bufs, sizes, outer, inner):
        total = outer * inner * sum(sizes)
        res = self.mallocArray(total)
        ptrs = (C.c_void_p * len(bufs))(*[b.ptr for b in bufs])
        self.lib.lh_concat(len(bufs), ptrs, _ints(sizes), res.ptr, outer, inner); _lib.check()
        return res

    def concat_grad(self, dbufs, sizes, outd, outer, inner, betas=None):
        ptrs = (C.c_void_p * len(dbufs))(*[(b.ptr if b is not None else 0) for b in dbufs])
        if betas is None:
            self.lib.lh_concat_grad(len(dbufs), ptrs, _ints(sizes), outd.ptr, outer, inner)
        else:
            self.lib.lh_concat_grad_beta(len(dbufs), ptrs, (C.c_float * len(betas))(*betas), _ints(sizes), outd.ptr, outer, inner)
        _lib.check()

    # -- recurrent layer, CTC (CDN:1638-1938) ------------------------------------------------------------
    def ctcLoss(self, probs, probs_d, input_lengths, labels, label_lengths, T, B, A):
        """probs [T,B,A] after softmax; lengths and labels are host int arrays; returns per-sample costs [B]."""
        costs = self.mallocArray(B)
        il = np.ascontiguousarray(input_lengths, np.int32); lb = np.ascontiguousarray(labels, np.int32); ll = np.ascontiguousarray(label_lengths, np.int32)
        self.lib.lh_ctc_loss(probs.ptr, probs_d.ptr if probs_d is not None else 0, lb.ctypes.data, ll.ctypes.data, il.ctypes.data, costs.ptr, T, B, A)
        _lib.check()
        return costs

    def rnn_forward(self, mode, x, w, T, B, I, H, bidir, hx=None):
        y = self.mallocArray(T * B * H * (2 if bidir else 1))
        self.lib.lh_rnn_fwd_init(mode, x.ptr, hx.ptr if hx is not None else 0, w.ptr, y.ptr, T, B, I, H, int(bidir)); _lib.check()
        if self.count_work: self._count("gemm_flop", 2.0 * T * B * H * I * (2 if bidir else 1)); self._count("rnn_flop", 2.0 * T * B * H * H * (2 if bidir else 1))
        return y

    def rnn_backward(self, mode, x, y, dy, w, dx, dw, T, B, I, H, bidir, beta_dx=1.0, hx=None):
        self.lib.lh_rnn_bwd_init(mode, x.ptr, hx.ptr if hx is not None else 0, y.ptr, dy.ptr, w.ptr, dx.ptr if dx is not None else 0, beta_dx, dw.ptr,
                                 T, B, I, H, int(bidir)); _lib.check()
        D = 2 if bidir else 1
        if self.count_work: self._count("gemm_flop", 2.0 * T * B * H * D * (I * (2 if dx is not None else 1) + H)); self._count("rnn_flop", 2.0 * T * B * H * H * D)

    def rnn_gated_forward(self, mode, x, w, T, B, I, H, bidir, hx=None, cx=None):
        """LSTM (mode 2) / GRU (mode 3): returns (y, reserve); the reserve goes to rnn_gated_backward, once."""
        D = 2 if bidir else 1
        y = self.mallocArray(T * B * H * D)
        reserve = self.mallocArray(self.lib.lh_rnn_gated_reserve_floats(mode, T, B, H, int(bidir)))
        self.lib.lh_rnn_gated_fwd_init(mode, x.ptr, hx.ptr if hx is not None else 0, cx.ptr if cx is not None else 0, w.ptr, y.ptr, reserve.ptr,
                                       T, B, I, H, int(bidir)); _lib.check()
        G = (4 if mode == 2 else 3) * H
        if self.count_work: self._count("gemm_flop", 2.0 * T * B * G * (I + H) * D)
        return y, reserve

    def rnn_gated_backward(self, mode, x, y, dy, w, reserve, dx, dw, T, B, I, H, bidir, beta_dx=1.0, hx=None, cx=None):
        self.lib.lh_rnn_gated_bwd_init(mode, x.ptr, hx.ptr if hx is not None else 0, cx.ptr if cx is not None else 0, y.ptr, dy.ptr, w.ptr, reserve.ptr,
                                       dx.ptr if dx is not None else 0, beta_dx, dw.ptr, T, B, I, H, int(bidir)); _lib.check()
        G = (4 if mode == 2 else 3) * H
        if self.count_work: self._count("gemm_flop", 2.0 * T * B * G * (I * (2 if dx is not None else 1) + 2 * H) * (2 if bidir else 1))

    # -- optimizers ----------------------------------------------------------------------------------------
    def sgd_update(self, x, d, lr, n):
        self.lib.lh_sgd(x.ptr, d.ptr, lr, n); _lib.check()

    def adagrad_update(self, x, d, m, lr, clip, n):
        self.lib.lh_adagrad(x.ptr, d.ptr, m.ptr, lr, clip, n); _lib.check()

    def momentum_update(self, x, d, v, lr, mu, clip, nesterov, n):
        self.lib.lh_momentum(x.ptr, d.ptr, v.ptr, lr, mu, clip, int(nesterov), n); _lib.check()

    def multi_momentum_update(self, params, lr, mu, clip, nesterov):
        """params: list of (x Buf, d Buf, v Buf, n).  One launch for the whole model."""
        k = len(params)
        key = tuple((p[0].ptr, p[1].ptr, p[2].ptr, p[3]) for p in params)
        if getattr(self, "_mt_key", None) != key:
            self._mt_key = key
            self._mt = ((C.c_void_p * k)(*[p[0].ptr for p in params]), (C.c_void_p * k)(*[p[1].ptr for p in params]),
                        (C.c_void_p * k)(*[p[2].ptr for p in params]), (C.c_int64 * k)(*[p[3] for p in params]))
        xs, ds, vs, ns = self._mt
        self.lib.lh_multi_momentum(k, xs, ds, vs, ns, lr, mu, clip, int(nesterov)); _lib.check()

    def multi_sgd_update(self, params, lr):
        k = len(params)
        key = tuple((p[0].ptr, p[1].ptr, p[2]) for p in params)
        if getattr(self, "_ms_key", None) != key:
            self._ms_key = key
            self._ms = ((C.c_void_p * k)(*[p[0].ptr for p in params]), (C.c_void_p * k)(*[p[1].ptr for p in params]),
                        (C.c_int64 * k)(*[p[2] for p in params]))
        xs, ds, ns = self._ms
        self.lib.lh_multi_sgd(k, xs, ds, ns, lr); _lib.check()
