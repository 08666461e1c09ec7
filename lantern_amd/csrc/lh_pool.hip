// Max pooling with argmax and average pooling, forward and backward (HBM-bound streaming).
// Reference semantics: CPU:848-1038 -- scan kernel rows then columns, strict '>' starting
// from -FLT_MAX so the first maximum wins; argmax is the global flat index into x.
#include "lh_common.h"
using namespace lh;

namespace {
constexpr int TPB = 256;

// One block row-slot per output row (n*C + c, p); threads run along q, so the only division is one per row.
// S2: stride (2,2), the common case, with the stride folded into shifts.
// K3: a 3x3 window, unrolled so that its nine loads are in flight together (with run-time bounds the loop serialises them).
template <bool S2, bool K3>
__global__ void __launch_bounds__(TPB) k_maxpool_fwd(const float* __restrict__ x, float* __restrict__ y, int* __restrict__ idx,
                                                     int H, int W, int oH, int oW, int kH, int kW, int sH, int sW, int pad, int64_t rows) {
  // A wavefront per output row; rows narrower than half a wavefront share one (G rows side by side), so that the
  // 16x16 and 8x8 maps of small networks still fill the lanes.
  const int ry = threadIdx.x / 64, lane = threadIdx.x & 63;
  const int G = oW > 32 ? 1 : 64 / oW;
  const int lr = G > 1 ? lane / oW : 0, lq = G > 1 ? lane - lr * oW : lane;
  for (int64_t row0 = ((int64_t)blockIdx.x * 4 + ry) * G; row0 < rows; row0 += (int64_t)gridDim.x * 4 * G) {
    const int64_t row = row0 + lr;
    if (lr >= G || row >= rows) continue;
    const int p = (int)(row % oH); const int64_t nc = row / oH;
    const int64_t base = nc * H * W;
    const int h0 = (S2 ? 2 * p : p * sH) - pad;
    for (int q = lq; q < oW; q += 64) {
      const int w0 = (S2 ? 2 * q : q * sW) - pad;
      float best = -3.402823466e+38f; int bi = 0;
      if (K3) {
        float v[9]; bool in[9];
#pragma unroll
        for (int r = 0; r < 3; r++)
#pragma unroll
          for (int t = 0; t < 3; t++) {
            const int h = h0 + r, w = w0 + t;
            in[r * 3 + t] = h >= 0 && h < H && w >= 0 && w < W;
            v[r * 3 + t] = in[r * 3 + t] ? x[base + (int64_t)h * W + w] : 0.f;
          }
#pragma unroll
        for (int e = 0; e < 9; e++)          // same visiting order and strict comparison as the loop below
          if (in[e] && v[e] > best) { best = v[e]; bi = (int)(base + (int64_t)(h0 + e / 3) * W + w0 + e % 3); }
      } else {
        for (int r = 0; r < kH; r++) {
          const int h = h0 + r;
          if (h < 0 || h >= H) continue;
          for (int t = 0; t < kW; t++) {
            const int w = w0 + t;
            if (w < 0 || w >= W) continue;
            const float v = x[base + (int64_t)h * W + w];
            if (v > best) { best = v; bi = (int)(base + (int64_t)h * W + w); }
          }
        }
      }
      const int64_t o = row * oW + q;
      y[o] = best; idx[o] = bi;
    }
  }
}
// Scatter-add.  Windows overlap when stride < kernel, so two outputs may hit the same input:
// atomic add (the sum has at most a few terms, all orders round the same to ~1 ulp).
__global__ void __launch_bounds__(TPB) k_maxpool_bwd_atomic(const float* __restrict__ dy, const int* __restrict__ idx, float* dx, int64_t n_out) {
  int64_t o = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; o < n_out; o += st) atomicAdd(dx + idx[o], dy[o]);
}
// Gather form: one thread per input pixel; the windows that contain (h, w) are p in [p_lo, p_hi] x q in
// [q_lo, q_hi]; a window contributes when its stored argmax is this pixel's flat index.
// W2: at most two windows per direction cover a pixel (kernel <= 2 * stride): the four candidates are fetched together.
template <bool ACC, bool S2, bool W2>
__global__ void __launch_bounds__(TPB) k_maxpool_bwd_dense(const float* __restrict__ dy, const int* __restrict__ idx, float* __restrict__ dx,
                                                           int H, int W, int oH, int oW, int kH, int kW, int sH, int sW, int pad, int64_t rows) {
  // a wavefront per input row (n*C + c, h), lanes along w: one division per row; S2 folds stride (2,2) into shifts
  const int ry = threadIdx.x / 64, lane = threadIdx.x & 63;
  const int G = W > 32 ? 1 : 64 / W;                      // narrow rows share a wavefront, as in the forward kernel
  const int lr = G > 1 ? lane / W : 0, lw = G > 1 ? lane - lr * W : lane;
  for (int64_t row0 = ((int64_t)blockIdx.x * 4 + ry) * G; row0 < rows; row0 += (int64_t)gridDim.x * 4 * G) {
    const int64_t row = row0 + lr;
    if (lr >= G || row >= rows) continue;
    const int h = (int)(row % H); const int64_t nc = row / H;
    const int hp = h + pad;
    const int p_hi = min(oH - 1, S2 ? hp >> 1 : hp / sH);
    const int p_lo = hp < kH ? 0 : (S2 ? (hp - kH) >> 1 : (hp - kH) / sH) + 1;
    const int64_t ob = nc * oH * oW;
    for (int w = lw; w < W; w += 64) {
      const int wp = w + pad;
      const int q_hi = min(oW - 1, S2 ? wp >> 1 : wp / sW);
      const int q_lo = wp < kW ? 0 : (S2 ? (wp - kW) >> 1 : (wp - kW) / sW) + 1;
      const int64_t i = row * W + w;
      float acc = 0.f;
      if (W2) {
        int id[4]; float g[4]; bool in[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int p = p_lo + (e >> 1), q = q_lo + (e & 1);
          in[e] = p <= p_hi && q <= q_hi;
          const int64_t o = ob + (int64_t)(in[e] ? p : p_hi) * oW + (in[e] ? q : q_hi);      // p_hi, q_hi are always valid windows
          id[e] = idx[o]; g[e] = dy[o];
        }
#pragma unroll
        for (int e = 0; e < 4; e++) if (in[e] && id[e] == (int)i) acc += g[e];        // same order as the loops below
      } else {
        for (int p = p_lo; p <= p_hi; p++)
          for (int q = q_lo; q <= q_hi; q++) {
            const int64_t o = ob + (int64_t)p * oW + q;
            if (idx[o] == (int)i) acc += dy[o];
          }
      }
      dx[i] = ACC ? dx[i] + acc : acc;
    }
  }
}
// The 3x3 / stride 2 / pad 1 pool of the ResNet stem, for even H and W % 4 == 0 (so oH = H/2, oW = W/2): a thread produces
// two neighbouring outputs from one 16-byte load and one scalar load per window row (input columns 4j-1 .. 4j+3) instead
// of nine strided scalar loads each.  Same scan order and strict comparison as the general kernel: the first maximum wins.
__global__ void __launch_bounds__(TPB) k_maxpool_fwd_k3s2p1(const float* __restrict__ x, float* __restrict__ y, int* __restrict__ idx,
                                                            int H, int W, int64_t total /* N*C*oH*(oW/2) */) {
  const int oW = W >> 1, oH = H >> 1, half = oW >> 1;
  for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < total; i += (int64_t)gridDim.x * TPB) {
    const int j = (int)(i % half); const int64_t row = i / half;
    const int p = (int)(row % oH); const int64_t nc = row / oH;
    const int64_t base = nc * H * W;
    float v[3][5]; bool in[3];
#pragma unroll
    for (int r = 0; r < 3; r++) {
      const int h = 2 * p - 1 + r;
      in[r] = h >= 0 && h < H;
      const int64_t o = base + (int64_t)(in[r] ? h : 0) * W + 4 * j;
      const float4 t = *reinterpret_cast<const float4*>(x + o);
      v[r][0] = j > 0 ? x[o - 1] : 0.f; v[r][1] = t.x; v[r][2] = t.y; v[r][3] = t.z; v[r][4] = t.w;
    }
    float b0 = -3.402823466e+38f, b1 = -3.402823466e+38f; int i0 = 0, i1 = 0;
#pragma unroll
    for (int r = 0; r < 3; r++) {
      if (!in[r]) continue;
      const int rowbase = (int)(base + (int64_t)(2 * p - 1 + r) * W + 4 * j);
#pragma unroll
      for (int t = 0; t < 3; t++) {
        if ((t > 0 || j > 0) && v[r][t] > b0) { b0 = v[r][t]; i0 = rowbase + t - 1; }       // output 2j: columns 4j-1 .. 4j+1
        if (v[r][t + 2] > b1) { b1 = v[r][t + 2]; i1 = rowbase + t + 1; }                     // output 2j+1: columns 4j+1 .. 4j+3
      }
    }
    const int64_t o = row * oW + 2 * j;
    *reinterpret_cast<float2*>(y + o) = make_float2(b0, b1);
    *reinterpret_cast<int2*>(idx + o) = make_int2(i0, i1);
  }
}
// Its backward as a gather: a thread owns the 2x2 input cell (2i..2i+1, 2j..2j+1), which only the windows (i..i+1, j..j+1)
// cover -- (2i,2j) lies in window (i,j) alone, (2i,2j+1) in (i,j),(i,j+1), (2i+1,2j) in (i,j),(i+1,j), the last pixel in all
// four -- so four (argmax, dy) pairs serve four pixels.  Sums run in window order, as in the general kernel.
template <bool ACC>
__global__ void __launch_bounds__(TPB) k_maxpool_bwd_k3s2p1(const float* __restrict__ dy, const int* __restrict__ idx, float* __restrict__ dx,
                                                            int H, int W, int64_t total /* N*C*(H/2)*(W/2) */) {
  const int oW = W >> 1, oH = H >> 1;
  for (int64_t t = (int64_t)blockIdx.x * TPB + threadIdx.x; t < total; t += (int64_t)gridDim.x * TPB) {
    const int j = (int)(t % oW); const int64_t r = t / oW;
    const int i = (int)(r % oH); const int64_t nc = r / oH;
    const int64_t ob = nc * oH * oW, ib = nc * H * W;
    const bool pd = i + 1 < oH, qd = j + 1 < oW;
    const int64_t o00 = ob + (int64_t)i * oW + j, o01 = qd ? o00 + 1 : o00, o10 = pd ? o00 + oW : o00, o11 = pd ? o01 + oW : o01;
    const int a00 = idx[o00], a01 = idx[o01], a10 = idx[o10], a11 = idx[o11];
    const float g00 = dy[o00], g01 = dy[o01], g10 = dy[o10], g11 = dy[o11];
    const int e00 = (int)(ib + (int64_t)(2 * i) * W + 2 * j), e01 = e00 + 1, e10 = e00 + W, e11 = e10 + 1;
    float s00 = 0.f, s01 = 0.f, s10 = 0.f, s11 = 0.f;
    if (a00 == e00) s00 += g00;
    if (a00 == e01) s01 += g00;
    if (qd && a01 == e01) s01 += g01;
    if (a00 == e10) s10 += g00;
    if (pd && a10 == e10) s10 += g10;
    if (a00 == e11) s11 += g00;
    if (qd && a01 == e11) s11 += g01;
    if (pd && a10 == e11) s11 += g10;
    if (pd && qd && a11 == e11) s11 += g11;
    float2* d0 = reinterpret_cast<float2*>(dx + e00); float2* d1 = reinterpret_cast<float2*>(dx + e10);
    if (ACC) { const float2 u0 = *d0, u1 = *d1; s00 += u0.x; s01 += u0.y; s10 += u1.x; s11 += u1.y; }
    *d0 = make_float2(s00, s01); *d1 = make_float2(s10, s11);
  }
}
__global__ void __launch_bounds__(TPB) k_avgpool_fwd(const float* __restrict__ x, float* __restrict__ y, int H, int W, int oH, int oW,
                                                     int kH, int kW, int sH, int sW, int64_t n_out) {
  const float ks = (float)(kH * kW);
  int64_t o = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; o < n_out; o += st) {
    int q = (int)(o % oW); int64_t t = o / oW; int p = (int)(t % oH); int64_t nc = t / oH;
    const float* xp = x + nc * H * W + (int64_t)(p * sH) * W + q * sW;
    float sum = 0.f;
    for (int r = 0; r < kH; r++) for (int s = 0; s < kW; s++) sum += xp[(int64_t)r * W + s];
    y[o] = sum / ks;
  }
}
// Gather form of the backward: each input element sums the windows that cover it.
__global__ void __launch_bounds__(TPB) k_avgpool_bwd(const float* __restrict__ dy, float* dx, int H, int W, int oH, int oW,
                                                     int kH, int kW, int sH, int sW, int64_t n_in) {
  const int ks = kH * kW;
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n_in; i += st) {
    int w = (int)(i % W); int64_t t = i / W; int h = (int)(t % H); int64_t nc = t / H;
    // windows p with p*sH <= h < p*sH + kH
    int p_lo = h - kH + 1 > 0 ? (h - kH + 1 + sH - 1) / sH : 0, p_hi = min(oH - 1, h / sH);
    int q_lo = w - kW + 1 > 0 ? (w - kW + 1 + sW - 1) / sW : 0, q_hi = min(oW - 1, w / sW);
    float acc = 0.f; bool any = false;
    for (int p = p_lo; p <= p_hi; p++) for (int q = q_lo; q <= q_hi; q++) { acc += dy[(nc * oH + p) * oW + q] / ks; any = true; }
    if (any) dx[i] += acc;
  }
}
// Global average pooling (the window is the whole map, one output per channel image): a wavefront per image with
// coalesced loads; the general kernel would walk each image with one thread.
__global__ void __launch_bounds__(TPB) k_avgpool_global_fwd(const float* __restrict__ x, float* __restrict__ y, int HW, int64_t rows) {
  const int lane = threadIdx.x & 63;
  const float ks = (float)HW;
  for (int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); row < rows; row += (int64_t)gridDim.x * 4) {
    const float* xp = x + row * HW;
    float a = 0.f;
    for (int l = lane; l < HW; l += 64) a += xp[l];
    a = lh_wave_sum(a);
    if (lane == 0) y[row] = a / ks;
  }
}
__global__ void __launch_bounds__(TPB) k_avgpool_global_bwd(const float* __restrict__ dy, float* dx, int HW, int64_t n_in) {
  const float ks = (float)HW;
  for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < n_in; i += (int64_t)gridDim.x * TPB) dx[i] += dy[i / HW] / ks;
}
}  // namespace

// Average pooling with zero padding, the divisor counting only the elements inside the image (the reference's cuDNN backend
// asks for CUDNN_POOLING_AVERAGE_COUNT_EXCLUDE_PADDING, TensorDslCudnn.scala:975-978).  One thread per output; the
// backward kernel gathers, one thread per input element over the windows that cover it, so nothing needs an atomic.
__global__ void __launch_bounds__(256) k_avgpool_pad_fwd(const float* __restrict__ x, float* __restrict__ y, int H, int W, int oH, int oW,
                                                         int kH, int kW, int sH, int sW, int pH, int pW, int64_t n_out) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, st = (int64_t)gridDim.x * blockDim.x;
  for (; i < n_out; i += st) {
    const int ow = (int)(i % oW), oh = (int)((i / oW) % oH);
    const int64_t nc = i / ((int64_t)oW * oH);
    const int h0 = max(oh * sH - pH, 0), h1 = min(oh * sH - pH + kH, H), w0 = max(ow * sW - pW, 0), w1 = min(ow * sW - pW + kW, W);
    const float* p = x + nc * H * W;
    float sum = 0.f;
    for (int h = h0; h < h1; h++) for (int w = w0; w < w1; w++) sum += p[h * W + w];
    const int cnt = (h1 - h0) * (w1 - w0);
    y[i] = cnt > 0 ? sum / (float)cnt : 0.f;
  }
}
__global__ void __launch_bounds__(256) k_avgpool_pad_bwd(const float* __restrict__ dy, float* __restrict__ dx, int H, int W, int oH, int oW,
                                                         int kH, int kW, int sH, int sW, int pH, int pW, int64_t n_in) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, st = (int64_t)gridDim.x * blockDim.x;
  for (; i < n_in; i += st) {
    const int w = (int)(i % W), h = (int)((i / W) % H);
    const int64_t nc = i / ((int64_t)W * H);
    const int a0 = h + pH - kH + 1, b0 = w + pW - kW + 1;
    const int oh0 = a0 <= 0 ? 0 : (a0 + sH - 1) / sH, oh1 = min((h + pH) / sH, oH - 1);
    const int ow0 = b0 <= 0 ? 0 : (b0 + sW - 1) / sW, ow1 = min((w + pW) / sW, oW - 1);
    const float* g = dy + nc * oH * oW;
    float acc = 0.f;
    for (int oh = oh0; oh <= oh1; oh++) {
      const int ch = min(oh * sH - pH + kH, H) - max(oh * sH - pH, 0);
      for (int ow = ow0; ow <= ow1; ow++) {
        const int cw = min(ow * sW - pW + kW, W) - max(ow * sW - pW, 0);
        acc += g[oh * oW + ow] / (float)(ch * cw);
      }
    }
    dx[i] += acc;
  }
}

extern "C" {

void lh_maxpool_fwd(const float* x, float* y, int* argmax, int N, int C, int H, int W, int kH, int kW, int sH, int sW, int pad) {
  LZ_ENTER();
  if (lazy::g_busy && kH >= 1 && kW >= 1 && sH >= 1 && sW >= 1 && pad >= 0 && H + 2 * pad >= kH && W + 2 * pad >= kW) {
    const int64_t no = (int64_t)N * C * ((H + 2 * pad - kH) / sH + 1) * ((W + 2 * pad - kW) / sW + 1);
    lazy::rd_f(x, (int64_t)N * C * H * W); lazy::wr_f(y, no); lazy::wr_f(argmax, no);
  }
  ProfScope prof_(CAT_POOL);
  LH_REQUIRE(kH >= 1 && kW >= 1 && sH >= 1 && sW >= 1 && pad >= 0, "lh_maxpool_fwd: kernel/stride must be >= 1 and pad >= 0");
  LH_REQUIRE(H + 2 * pad >= kH && W + 2 * pad >= kW, "Image too small for maxPool_k: %dx%d | (%d,%d)", H, W, kH, kW);
  LH_REQUIRE((int64_t)N * C * H * W < 2147483647LL, "lh_maxpool_fwd: input too large for int32 argmax");
  int oH = (H + 2 * pad - kH) / sH + 1, oW = (W + 2 * pad - kW) / sW + 1;
  int64_t n_out = (int64_t)N * C * oH * oW;
  if (n_out <= 0) return;
  if (kH == 3 && kW == 3 && sH == 2 && sW == 2 && pad == 1 && (H & 1) == 0 && (W & 3) == 0 && ((((uintptr_t)x | (uintptr_t)y | (uintptr_t)argmax) & 15) == 0)) {
    const int64_t total = (int64_t)N * C * oH * (oW / 2);
    hipLaunchKernelGGL(k_maxpool_fwd_k3s2p1, dim3(stream_grid(total, TPB)), dim3(TPB), 0, g_stream, x, y, argmax, H, W, total);
    LH_CHECK_LAUNCH();
    return;
  }
  const int64_t rows = (int64_t)N * C * oH;
  const int grid = stream_grid(rows, 4 * (oW > 32 ? 1 : 64 / oW));
#define GO(S, K) hipLaunchKernelGGL((k_maxpool_fwd<S, K>), dim3(grid), dim3(TPB), 0, g_stream, x, y, argmax, H, W, oH, oW, kH, kW, sH, sW, pad, rows)
  const bool k3 = kH == 3 && kW == 3;
  if (sH == 2 && sW == 2) { if (k3) GO(true, true); else GO(true, false); }
  else { if (k3) GO(false, true); else GO(false, false); }
#undef GO
  LH_CHECK_LAUNCH();
}
void lh_maxpool_bwd(const float* dy, const int* argmax, float* dx, int64_t n_out) {
  // the scatter form does not know how large dx is: everything deferred is brought up to date (ordered_stream() at depth 0)
  ProfScope prof_(CAT_POOL);
  if (n_out <= 0) return;
  hipLaunchKernelGGL(k_maxpool_bwd_atomic, dim3(stream_grid(n_out, TPB * 4)), dim3(TPB), 0, g_stream, dy, argmax, dx, n_out);
  LH_CHECK_LAUNCH();
}
void lh_maxpool_bwd_dense(const float* dy, const int* argmax, float* dx, float beta,
                          int N, int C, int H, int W, int kH, int kW, int sH, int sW, int pad) {
  LZ_ENTER();
  if (lazy::g_busy && kH >= 1 && kW >= 1 && sH >= 1 && sW >= 1 && pad >= 0 && H + 2 * pad >= kH && W + 2 * pad >= kW && (beta == 0.f || beta == 1.f)) {
    const int64_t no = (int64_t)N * C * ((H + 2 * pad - kH) / sH + 1) * ((W + 2 * pad - kW) / sW + 1);
    lazy::rd_f(dy, no); lazy::rd_f(argmax, no);
    beta = lazy::beta_f(dx, (int64_t)N * C * H * W, beta);
  }
  ProfScope prof_(CAT_POOL);
  LH_REQUIRE(kH >= 1 && kW >= 1 && sH >= 1 && sW >= 1 && pad >= 0, "lh_maxpool_bwd_dense: kernel/stride must be >= 1 and pad >= 0");
  LH_REQUIRE(H + 2 * pad >= kH && W + 2 * pad >= kW, "lh_maxpool_bwd_dense: image %dx%d too small for (%d,%d)", H, W, kH, kW);
  LH_REQUIRE(beta == 0.f || beta == 1.f, "lh_maxpool_bwd_dense: beta must be 0 or 1");
  const int64_t n_in = (int64_t)N * C * H * W;
  LH_REQUIRE(n_in < 2147483647LL, "lh_maxpool_bwd_dense: input too large for int32 argmax");
  if (n_in <= 0) return;
  const int oH = (H + 2 * pad - kH) / sH + 1, oW = (W + 2 * pad - kW) / sW + 1;
  if (kH == 3 && kW == 3 && sH == 2 && sW == 2 && pad == 1 && (H & 1) == 0 && (W & 1) == 0 && (((uintptr_t)dx & 7) == 0)) {
    const int64_t total = (int64_t)N * C * (H / 2) * (W / 2);
    if (beta == 0.f) hipLaunchKernelGGL((k_maxpool_bwd_k3s2p1<false>), dim3(stream_grid(total, TPB)), dim3(TPB), 0, g_stream, dy, argmax, dx, H, W, total);
    else hipLaunchKernelGGL((k_maxpool_bwd_k3s2p1<true>), dim3(stream_grid(total, TPB)), dim3(TPB), 0, g_stream, dy, argmax, dx, H, W, total);
    LH_CHECK_LAUNCH();
    return;
  }
  const int64_t rows = (int64_t)N * C * H;
  const int grid = stream_grid(rows, 4 * (W > 32 ? 1 : 64 / W));
  const bool s2 = sH == 2 && sW == 2;
  const bool w2 = kH <= 2 * sH && kW <= 2 * sW;
#define GO(A, S, T) hipLaunchKernelGGL((k_maxpool_bwd_dense<A, S, T>), dim3(grid), dim3(TPB), 0, g_stream, dy, argmax, dx, H, W, oH, oW, kH, kW, sH, sW, pad, rows)
#define GO2(A) do { if (s2) { if (w2) GO(A, true, true); else GO(A, true, false); } else { if (w2) GO(A, false, true); else GO(A, false, false); } } while (0)
  if (beta == 0.f) GO2(false); else GO2(true);
#undef GO2
#undef GO
  LH_CHECK_LAUNCH();
}
void lh_avgpool_fwd(const float* x, float* y, int N, int C, int H, int W, int kH, int kW, int sH, int sW) {
  LZ_ENTER();
  if (lazy::g_busy && kH >= 1 && kW >= 1 && sH >= 1 && sW >= 1 && H >= kH && W >= kW) {
    lazy::rd_f(x, (int64_t)N * C * H * W); lazy::wr_f(y, (int64_t)N * C * ((H - kH) / sH + 1) * ((W - kW) / sW + 1));
  }
  ProfScope prof_(CAT_POOL);
  LH_REQUIRE(kH >= 1 && kW >= 1 && sH >= 1 && sW >= 1 && H >= kH && W >= kW, "lh_avgpool_fwd: bad kernel/stride for %dx%d", H, W);
  int oH = (H - kH) / sH + 1, oW = (W - kW) / sW + 1;
  int64_t n_out = (int64_t)N * C * oH * oW;
  if (n_out <= 0) return;
  if (kH == H && kW == W) hipLaunchKernelGGL(k_avgpool_global_fwd, dim3(stream_grid(n_out, 4)), dim3(TPB), 0, g_stream, x, y, H * W, n_out);
  else hipLaunchKernelGGL(k_avgpool_fwd, dim3(stream_grid(n_out, TPB)), dim3(TPB), 0, g_stream, x, y, H, W, oH, oW, kH, kW, sH, sW, n_out);
  LH_CHECK_LAUNCH();
}
void lh_avgpool_bwd(const float* dy, float* dx, int N, int C, int H, int W, int kH, int kW, int sH, int sW) {
  LZ_ENTER();
  if (lazy::g_busy && kH >= 1 && kW >= 1 && sH >= 1 && sW >= 1 && H >= kH && W >= kW) {
    lazy::rd_f(dy, (int64_t)N * C * ((H - kH) / sH + 1) * ((W - kW) / sW + 1)); lazy::rw_f(dx, (int64_t)N * C * H * W);
  }
  ProfScope prof_(CAT_POOL);
  LH_REQUIRE(kH >= 1 && kW >= 1 && sH >= 1 && sW >= 1 && H >= kH && W >= kW, "lh_avgpool_bwd: bad kernel/stride for %dx%d", H, W);
  int oH = (H - kH) / sH + 1, oW = (W - kW) / sW + 1;
  int64_t n_in = (int64_t)N * C * H * W;
  if (n_in <= 0) return;
  if (kH == H && kW == W) hipLaunchKernelGGL(k_avgpool_global_bwd, dim3(stream_grid(n_in, TPB * 2)), dim3(TPB), 0, g_stream, dy, dx, H * W, n_in);
  else hipLaunchKernelGGL(k_avgpool_bwd, dim3(stream_grid(n_in, TPB * 2)), dim3(TPB), 0, g_stream, dy, dx, H, W, oH, oW, kH, kW, sH, sW, n_in);
  LH_CHECK_LAUNCH();
}

void lh_avgpool_pad_fwd(const float* x, float* y, int N, int C, int H, int W, int kH, int kW, int sH, int sW, int pH, int pW) {
  LZ_ENTER();
  if (lazy::g_busy && kH >= 1 && kW >= 1 && sH >= 1 && sW >= 1 && pH >= 0 && pW >= 0 && H + 2 * pH >= kH && W + 2 * pW >= kW) {
    lazy::rd_f(x, (int64_t)N * C * H * W); lazy::wr_f(y, (int64_t)N * C * ((H + 2 * pH - kH) / sH + 1) * ((W + 2 * pW - kW) / sW + 1));
  }
  ProfScope prof_(CAT_POOL);
  LH_REQUIRE(kH >= 1 && kW >= 1 && sH >= 1 && sW >= 1 && pH >= 0 && pW >= 0 && pH < kH && pW < kW, "lh_avgpool_pad_fwd: kernel (%d,%d) stride (%d,%d) pad (%d,%d)", kH, kW, sH, sW, pH, pW);
  LH_REQUIRE(H + 2 * pH >= kH && W + 2 * pW >= kW, "lh_avgpool_pad_fwd: image %dx%d too small for (%d,%d)", H, W, kH, kW);
  const int oH = (H + 2 * pH - kH) / sH + 1, oW = (W + 2 * pW - kW) / sW + 1;
  const int64_t n_out = (int64_t)N * C * oH * oW;
  if (n_out <= 0) return;
  hipLaunchKernelGGL(k_avgpool_pad_fwd, dim3(stream_grid(n_out, 256)), dim3(256), 0, g_stream, x, y, H, W, oH, oW, kH, kW, sH, sW, pH, pW, n_out);
  LH_CHECK_LAUNCH();
}
void lh_avgpool_pad_bwd(const float* dy, float* dx, int N, int C, int H, int W, int kH, int kW, int sH, int sW, int pH, int pW) {
  LZ_ENTER();
  if (lazy::g_busy && kH >= 1 && kW >= 1 && sH >= 1 && sW >= 1 && pH >= 0 && pW >= 0 && H + 2 * pH >= kH && W + 2 * pW >= kW) {
    lazy::rd_f(dy, (int64_t)N * C * ((H + 2 * pH - kH) / sH + 1) * ((W + 2 * pW - kW) / sW + 1)); lazy::rw_f(dx, (int64_t)N * C * H * W);
  }
  ProfScope prof_(CAT_POOL);
  LH_REQUIRE(kH >= 1 && kW >= 1 && sH >= 1 && sW >= 1 && pH >= 0 && pW >= 0 && pH < kH && pW < kW, "lh_avgpool_pad_bwd: kernel (%d,%d) stride (%d,%d) pad (%d,%d)", kH, kW, sH, sW, pH, pW);
  LH_REQUIRE(H + 2 * pH >= kH && W + 2 * pW >= kW, "lh_avgpool_pad_bwd: image %dx%d too small for (%d,%d)", H, W, kH, kW);
  const int oH = (H + 2 * pH - kH) / sH + 1, oW = (W + 2 * pW - kW) / sW + 1;
  const int64_t n_in = (int64_t)N * C * H * W;
  if (n_in <= 0) return;
  hipLaunchKernelGGL(k_avgpool_pad_bwd, dim3(stream_grid(n_in, 256)), dim3(256), 0, g_stream, dy, dx, H, W, oH, oW, kH, kW, sH, sW, pH, pW, n_in);
  LH_CHECK_LAUNCH();
}

}  // extern "C"
