// conv2D_batch forward, input gradient and filter gradient (NCHW fp32 cross-correlation) as
// implicit GEMM on fp32 MFMA.  Reference behaviour being replaced: CPU:532-692 (im2col +
// SGEMM per sample) and CDN:515-880 (cuDNN forward / backward-data / backward-filter / bias).
//
//   forward         Y[k, (n,p,q)]   = sum_{(c,r,s)} W[k, (c,r,s)]   * X[(c,r,s), (n,p,q)]
//   input gradient  dX[c, (n,h,w)] += sum_{(k,r,s)} Wt[c, (k,r,s)]  * dY[(k,r,s), (n,h,w)]
//   filter gradient dW[k, (c,r,s)] += sum_{(n,p,q)} dY[k, (n,p,q)]  * X[(n,p,q), (c,r,s)]
//
// Algorithmic work of each: 2*N*K*C*R*S*P*Q flop.
#include "lh_igemm.h"
using namespace lh;

namespace {
constexpr int TPB = 256;

struct ConvDims { int N, C, H, W, K, R, S, sH, sW, pH, pW, P, Q; };

static bool make_dims(ConvDims& d, int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW) {
  if (N < 1 || C < 1 || H < 1 || W < 1 || K < 1 || R < 1 || S < 1 || sH < 1 || sW < 1 || pH < 0 || pW < 0) return false;
  if (H + 2 * pH < R || W + 2 * pW < S) return false;
  d = {N, C, H, W, K, R, S, sH, sW, pH, pW, (H + 2 * pH - R) / sH + 1, (W + 2 * pW - S) / sW + 1};
  const int64_t lim = 0x7fffffffLL;
  if ((int64_t)N * C * H * W >= lim || (int64_t)N * K * d.P * d.Q >= lim || (int64_t)K * C * R * S >= lim) return false;
  return true;
}

// ---- B operand of the forward pass: im2col gather of x --------------------------------------
// column j = (n, p, q) fixed per thread; k = (c, r, s) is uniform across a wavefront.
struct LoadConvFwdB {
  static constexpr bool ALONG_K = false;
  const float* x; int C, H, W, sH, sW, pH, pW, HW;
  FastDiv dPQ, dQ, dRS, dS;
  struct State { int base, h0, w0; bool valid; };
  __device__ __forceinline__ void init(State& s, int j, int ncols) const {
    s.valid = j < ncols;
    uint32_t n, pq, p, q;
    dPQ.divmod(s.valid ? j : 0, n, pq); dQ.divmod(pq, p, q);
    s.base = (int)n * C * HW; s.h0 = (int)p * sH - pH; s.w0 = (int)q * sW - pW;
  }
  __device__ __forceinline__ float one(const State& s, int k, int kend) const {
    if (!s.valid || k >= kend) return 0.f;
    uint32_t c, rs, r, ss;
    dRS.divmod(k, c, rs); dS.divmod(rs, r, ss);
    int h = s.h0 + (int)r, w = s.w0 + (int)ss;
    if ((unsigned)h >= (unsigned)H || (unsigned)w >= (unsigned)W) return 0.f;
    return x[s.base + ((int)c * H + h) * W + w];
  }
  __device__ __forceinline__ float4 load4(const State& s, int k, int kend) const {
    return make_float4(one(s, k, kend), one(s, k + 1, kend), one(s, k + 2, kend), one(s, k + 3, kend));
  }
};

// ---- B operand of the input gradient: gather of dy ------------------------------------------------
// column j = (n, h, w) of dx fixed per thread; k = (ko, r, s) uniform across a wavefront.
struct LoadConvBwdDataB {
  static constexpr bool ALONG_K = false;
  const float* dy; int K, P, Q, PQ;
  FastDiv dHW, dW, dRS, dS, dsH, dsW;
  int pH, pW;
  struct State { int base, hh, ww; bool valid; };
  __device__ __forceinline__ void init(State& s, int j, int ncols) const {
    s.valid = j < ncols;
    uint32_t n, hw, h, w;
    dHW.divmod(s.valid ? j : 0, n, hw); dW.divmod(hw, h, w);
    s.base = (int)n * K * PQ; s.hh = (int)h + pH; s.ww = (int)w + pW;
  }
  __device__ __forceinline__ float one(const State& s, int k, int kend) const {
    if (!s.valid || k >= kend) return 0.f;
    uint32_t ko, rs, r, ss;
    dRS.divmod(k, ko, rs); dS.divmod(rs, r, ss);
    int th = s.hh - (int)r, tw = s.ww - (int)ss;
    if (th < 0 || tw < 0) return 0.f;
    uint32_t p, ph, q, qw;
    dsH.divmod(th, p, ph); dsW.divmod(tw, q, qw);
    if (ph != 0 || qw != 0 || (int)p >= P || (int)q >= Q) return 0.f;
    return dy[s.base + ((int)ko * P + (int)p) * Q + (int)q];
  }
  __device__ __forceinline__ float4 load4(const State& s, int k, int kend) const {
    return make_float4(one(s, k, kend), one(s, k + 1, kend), one(s, k + 2, kend), one(s, k + 3, kend));
  }
};

// ---- A operand of the filter gradient: dy rows, reduction index (n, p, q) ------------------------------
struct LoadConvBwdFilterA {
  static constexpr bool ALONG_K = true;
  const float* dy; int K, PQ, vec;      // vec: PQ % 4 == 0 and dy 16-byte aligned
  FastDiv dPQ;
  struct State { int rowoff; bool valid; };
  __device__ __forceinline__ void init(State& s, int i, int nrows) const { s.valid = i < nrows; s.rowoff = (s.valid ? i : 0) * PQ; }
  __device__ __forceinline__ float one(const State& s, int kk, int kend) const {
    if (kk >= kend) return 0.f;
    uint32_t n, pq; dPQ.divmod(kk, n, pq);
    return dy[(int64_t)n * K * PQ + s.rowoff + pq];
  }
  __device__ __forceinline__ float4 load4(const State& s, int kk, int kend) const {
    if (!s.valid) return make_float4(0.f, 0.f, 0.f, 0.f);
    if (vec && kk + 3 < kend) {
      uint32_t n, pq; dPQ.divmod(kk, n, pq);
      return *reinterpret_cast<const float4*>(dy + (int64_t)n * K * PQ + s.rowoff + pq);
    }
    return make_float4(one(s, kk, kend), one(s, kk + 1, kend), one(s, kk + 2, kend), one(s, kk + 3, kend));
  }
};

// ---- B operand of the filter gradient: gather of x, reduction index (n, p, q) ------------------------------
// column j = (c, r, s) fixed per thread.
struct LoadConvBwdFilterB {
  static constexpr bool ALONG_K = true;
  const float* x; int C, H, W, sH, sW, pH, pW, CHW;
  FastDiv dPQ, dQ, dRS, dS;
  int rowvec;   // Q % 4 == 0: four consecutive reduction indices share (n, p)
  struct State { int coff, dh, dw; bool valid; };
  __device__ __forceinline__ void init(State& s, int j, int ncols) const {
    s.valid = j < ncols;
    uint32_t c, rs, r, ss;
    dRS.divmod(s.valid ? j : 0, c, rs); dS.divmod(rs, r, ss);
    s.coff = (int)c * H * W; s.dh = (int)r - pH; s.dw = (int)ss - pW;
  }
  __device__ __forceinline__ float one(const State& s, int kk, int kend) const {
    if (kk >= kend) return 0.f;
    uint32_t n, pq, p, q;
    dPQ.divmod(kk, n, pq); dQ.divmod(pq, p, q);
    int h = (int)p * sH + s.dh, w = (int)q * sW + s.dw;
    if ((unsigned)h >= (unsigned)H || (unsigned)w >= (unsigned)W) return 0.f;
    return x[(int64_t)n * CHW + s.coff + h * W + w];
  }
  __device__ __forceinline__ float4 load4(const State& s, int kk, int kend) const {
    if (!s.valid) return make_float4(0.f, 0.f, 0.f, 0.f);
    if (rowvec && kk + 3 < kend) {
      uint32_t n, pq, p, q;
      dPQ.divmod(kk, n, pq); dQ.divmod(pq, p, q);
      int h = (int)p * sH + s.dh, w = (int)q * sW + s.dw;
      if ((unsigned)h >= (unsigned)H) return make_float4(0.f, 0.f, 0.f, 0.f);
      const float* row = x + (int64_t)n * CHW + s.coff + h * W;
      float4 r;
      r.x = (unsigned)w < (unsigned)W ? row[w] : 0.f;
      r.y = (unsigned)(w + sW) < (unsigned)W ? row[w + sW] : 0.f;
      r.z = (unsigned)(w + 2 * sW) < (unsigned)W ? row[w + 2 * sW] : 0.f;
      r.w = (unsigned)(w + 3 * sW) < (unsigned)W ? row[w + 3 * sW] : 0.f;
      return r;
    }
    return make_float4(one(s, kk, kend), one(s, kk + 1, kend), one(s, kk + 2, kend), one(s, kk + 3, kend));
  }
};

// ---- epilogue writing an NCHW activation: row i = channel, column j = (n, pixel) --------------------------
struct EpiConvOut {
  float* out; const float* bias; int chan, PIX; float beta;
  FastDiv dPIX;
  struct Col { int off; bool valid; };
  __device__ __forceinline__ Col col(int j, int N) const {
    Col c; c.valid = j < N;
    uint32_t n, pix; dPIX.divmod(c.valid ? j : 0, n, pix);
    c.off = (int)n * chan * PIX + (int)pix;
    return c;
  }
  __device__ __forceinline__ void store(const Col& c, int i, int M, float v) const {
    if (!c.valid || i >= M) return;
    float* p = out + c.off + i * PIX;
    if (bias) v += bias[i];
    *p = beta == 0.f ? v : v + beta * *p;
  }
};

// w[K][C][RS] -> wt[C][K][RS]
__global__ void __launch_bounds__(TPB) k_filter_transpose(const float* __restrict__ w, float* __restrict__ wt, int K, int C, int RS, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n; i += st) {
    int rs = (int)(i % RS); int64_t t = i / RS; int k = (int)(t % K); int c = (int)(t / K);
    wt[i] = w[((int64_t)k * C + c) * RS + rs];
  }
}
// db[k] += sum over n, p, q of dy: one block per k
__global__ void __launch_bounds__(TPB) k_conv_bwd_bias(const float* __restrict__ dy, float* db, int N, int K, int PQ) {
  __shared__ float sm[17];
  int k = blockIdx.x;
  float acc = 0.f;
  int64_t tot = (int64_t)N * PQ;
  for (int64_t j = threadIdx.x; j < tot; j += TPB) { int n = (int)(j / PQ); int l = (int)(j - (int64_t)n * PQ); acc += dy[((int64_t)n * K + k) * PQ + l]; }
  acc = lh_block_sum(acc, sm);
  if (threadIdx.x == 0) db[k] += acc;
}

template <class AL, class BL, class EP>
static bool launch_tiles(const AL& al, const BL& bl, const EP& ep, int M, int N, int K) {
  TilePick tp = pick_tile(M, N);
  if (tp.bm == 128) return igemm_launch<128, 128, 16>(al, bl, ep, M, N, K, 1);
  if (tp.bn == 128) return igemm_launch<64, 128, 16>(al, bl, ep, M, N, K, 1);
  return igemm_launch<64, 64, 16>(al, bl, ep, M, N, K, 1);
}
}  // namespace

extern "C" {

void lh_conv2d_fwd(const float* x, const float* w, const float* bias, float* y,
                   int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW) {
  ProfScope prof_(CAT_CONV_FWD);
  ConvDims d;
  LH_REQUIRE(make_dims(d, N, C, H, W, K, R, S, sH, sW, pH, pW), "lh_conv2d_fwd: bad shape N%d C%d H%d W%d K%d R%d S%d s(%d,%d) p(%d,%d)", N, C, H, W, K, R, S, sH, sW, pH, pW);
  const int CRS = C * R * S, PQ = d.P * d.Q;
  LoadPlainK al; al.base = w; al.ld = CRS; al.vec = (CRS % 4 == 0) && (((uintptr_t)w & 15) == 0);
  LoadConvFwdB bl; bl.x = x; bl.C = C; bl.H = H; bl.W = W; bl.sH = sH; bl.sW = sW; bl.pH = pH; bl.pW = pW; bl.HW = H * W;
  bl.dPQ.init(PQ); bl.dQ.init(d.Q); bl.dRS.init(R * S); bl.dS.init(S);
  EpiConvOut ep; ep.out = y; ep.bias = bias; ep.chan = K; ep.PIX = PQ; ep.beta = 0.f; ep.dPIX.init(PQ);
  if (!launch_tiles(al, bl, ep, K, N * PQ, CRS)) return;
  LH_CHECK_LAUNCH();
}

void lh_conv2d_bwd_data(const float* dy, const float* w, float* dx, float beta,
                        int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW) {
  ProfScope prof_(CAT_CONV_BWD_DATA);
  ConvDims d;
  LH_REQUIRE(make_dims(d, N, C, H, W, K, R, S, sH, sW, pH, pW), "lh_conv2d_bwd_data: bad shape");
  LH_REQUIRE(beta == 0.f || beta == 1.f, "lh_conv2d_bwd_data: beta must be 0 or 1");
  const int RS = R * S, KRS = K * RS, HW = H * W, PQ = d.P * d.Q;
  LoadConvBwdDataB bl; bl.dy = dy; bl.K = K; bl.P = d.P; bl.Q = d.Q; bl.PQ = PQ; bl.pH = pH; bl.pW = pW;
  bl.dHW.init(HW); bl.dW.init(W); bl.dRS.init(RS); bl.dS.init(S); bl.dsH.init(sH); bl.dsW.init(sW);
  EpiConvOut ep; ep.out = dx; ep.bias = nullptr; ep.chan = C; ep.PIX = HW; ep.beta = beta; ep.dPIX.init(HW);
  bool ok;
  if (RS == 1) {
    LoadPlainT al; al.base = w; al.ld = C;          // A[c][k] = w[k][c]
    ok = launch_tiles(al, bl, ep, C, N * HW, KRS);
  } else {
    // transposed filter in scratch taken from the arena top and released again: later
    // allocations may reuse it, but only by work enqueued after this call on the same stream.
    size_t bytes = (size_t)KRS * C * sizeof(float);
    float* wt = (float*)lh_malloc_uninit(bytes);
    if (wt == nullptr) return;
    int64_t n = (int64_t)KRS * C;
    hipLaunchKernelGGL(k_filter_transpose, dim3(stream_grid(n, TPB * 4)), dim3(TPB), 0, g_stream, w, wt, K, C, RS, n);
    LoadPlainK al; al.base = wt; al.ld = KRS; al.vec = (KRS % 4 == 0);
    ok = launch_tiles(al, bl, ep, C, N * HW, KRS);
    lh_free_top(bytes);
  }
  if (!ok) return;
  LH_CHECK_LAUNCH();
}

void lh_conv2d_bwd_filter(const float* x, const float* dy, float* dw, float* db, float beta,
                          int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW) {
  ProfScope prof_(CAT_CONV_BWD_FILTER);
  ConvDims d;
  LH_REQUIRE(make_dims(d, N, C, H, W, K, R, S, sH, sW, pH, pW), "lh_conv2d_bwd_filter: bad shape");
  LH_REQUIRE(beta == 0.f || beta == 1.f, "lh_conv2d_bwd_filter: beta must be 0 or 1");
  const int CRS = C * R * S, PQ = d.P * d.Q;
  const int64_t red = (int64_t)N * PQ;
  LH_REQUIRE(red < 0x7fffffffLL, "lh_conv2d_bwd_filter: reduction length too large");
  LoadConvBwdFilterA al; al.dy = dy; al.K = K; al.PQ = PQ; al.vec = (PQ % 4 == 0) && (((uintptr_t)dy & 15) == 0); al.dPQ.init(PQ);
  LoadConvBwdFilterB bl; bl.x = x; bl.C = C; bl.H = H; bl.W = W; bl.sH = sH; bl.sW = sW; bl.pH = pH; bl.pW = pW; bl.CHW = C * H * W;
  bl.dPQ.init(PQ); bl.dQ.init(d.Q); bl.dRS.init(R * S); bl.dS.init(S); bl.rowvec = (d.Q % 4 == 0);
  // The output is small (K x CRS) and the reduction long (N*P*Q): split it across blocks and
  // combine with fp32 atomic adds.
  TilePick tp = (K >= 128 && CRS >= 128) ? TilePick{128, 128} : (CRS >= 128 ? TilePick{64, 128} : TilePick{64, 64});
  int64_t tiles = cdiv(K, tp.bm) * cdiv(CRS, tp.bn);
  int split = (int)cdiv(3 * (int64_t)g_num_cu, tiles);
  int max_split = (int)cdiv(red, 256); if (max_split < 1) max_split = 1;
  if (split > max_split) split = max_split;
  if (split < 1) split = 1;
  if (beta == 0.f) lh_fill(dw, 0.f, (int64_t)K * CRS);
  EpiRowMajor ep; ep.C = dw; ep.ldc = CRS; ep.alpha = 1.f; ep.beta = 1.f; ep.atomic = split > 1 ? 1 : 0;
  bool ok;
  if (tp.bm == 128) ok = igemm_launch<128, 128, 32>(al, bl, ep, K, CRS, (int)red, split);
  else if (tp.bn == 128) ok = igemm_launch<64, 128, 32>(al, bl, ep, K, CRS, (int)red, split);
  else ok = igemm_launch<64, 64, 32>(al, bl, ep, K, CRS, (int)red, split);
  if (!ok) return;
  if (db) hipLaunchKernelGGL(k_conv_bwd_bias, dim3(K), dim3(TPB), 0, g_stream, dy, db, N, K, PQ);
  LH_CHECK_LAUNCH();
}

}  // extern "C"
