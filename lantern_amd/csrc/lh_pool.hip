// Max pooling with argmax and average pooling, forward and backward (HBM-bound streaming).
// Reference semantics: CPU:848-1038 -- scan kernel rows then columns, strict '>' starting
// from -FLT_MAX so the first maximum wins; argmax is the global flat index into x.
#include "lh_common.h"
using namespace lh;

namespace {
constexpr int TPB = 256;

// IT: uint32_t when every flat index fits 32 bits (a 64-bit division costs several times a 32-bit one)
template <class IT>
__global__ void __launch_bounds__(TPB) k_maxpool_fwd(const float* __restrict__ x, float* __restrict__ y, int* __restrict__ idx,
                                                     int H, int W, int oH, int oW, int kH, int kW, int sH, int sW, int pad, int64_t n_out) {
  IT o = (IT)blockIdx.x * TPB + threadIdx.x; const IT st = (IT)gridDim.x * TPB;
  for (; o < (IT)n_out; o += st) {
    int q = (int)(o % (IT)oW); IT t = o / (IT)oW; int p = (int)(t % (IT)oH); IT nc = t / (IT)oH;
    const int64_t base = (int64_t)nc * H * W;
    float best = -3.402823466e+38f; int bi = 0;
    const int h0 = p * sH - pad, w0 = q * sW - pad;
    for (int r = 0; r < kH; r++) {
      int h = h0 + r;
      if (h < 0 || h >= H) continue;
      for (int s = 0; s < kW; s++) {
        int w = w0 + s;
        if (w < 0 || w >= W) continue;
        float v = x[base + (int64_t)h * W + w];
        if (v > best) { best = v; bi = (int)(base + (int64_t)h * W + w); }
      }
    }
    y[o] = best; idx[o] = bi;
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
template <bool ACC>
__global__ void __launch_bounds__(TPB) k_maxpool_bwd_dense(const float* __restrict__ dy, const int* __restrict__ idx, float* __restrict__ dx,
                                                           int H, int W, int oH, int oW, int kH, int kW, int sH, int sW, int pad, int64_t n_in) {
  // n_in < 2^31 (the argmax is an int32 flat index): 32-bit index arithmetic
  uint32_t i = blockIdx.x * TPB + threadIdx.x; const uint32_t st = gridDim.x * TPB;
  for (; i < (uint32_t)n_in; i += st) {
    const int w = (int)(i % (uint32_t)W); const uint32_t t = i / (uint32_t)W; const int h = (int)(t % (uint32_t)H); const int64_t nc = t / (uint32_t)H;
    const int hp = h + pad, wp = w + pad;
    const int p_hi = min(oH - 1, hp / sH), q_hi = min(oW - 1, wp / sW);
    const int p_lo = hp < kH ? 0 : (hp - kH) / sH + 1, q_lo = wp < kW ? 0 : (wp - kW) / sW + 1;
    const int64_t ob = nc * oH * oW;
    float acc = 0.f;
    for (int p = p_lo; p <= p_hi; p++)
      for (int q = q_lo; q <= q_hi; q++) {
        const int64_t o = ob + (int64_t)p * oW + q;
        if (idx[o] == (int)i) acc += dy[o];
      }
    dx[i] = ACC ? dx[i] + acc : acc;
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
}  // namespace

extern "C" {

void lh_maxpool_fwd(const float* x, float* y, int* argmax, int N, int C, int H, int W, int kH, int kW, int sH, int sW, int pad) {
  ProfScope prof_(CAT_POOL);
  LH_REQUIRE(kH >= 1 && kW >= 1 && sH >= 1 && sW >= 1 && pad >= 0, "lh_maxpool_fwd: kernel/stride must be >= 1 and pad >= 0");
  LH_REQUIRE(H + 2 * pad >= kH && W + 2 * pad >= kW, "Image too small for maxPool_k: %dx%d | (%d,%d)", H, W, kH, kW);
  LH_REQUIRE((int64_t)N * C * H * W < 2147483647LL, "lh_maxpool_fwd: input too large for int32 argmax");
  int oH = (H + 2 * pad - kH) / sH + 1, oW = (W + 2 * pad - kW) / sW + 1;
  int64_t n_out = (int64_t)N * C * oH * oW;
  if (n_out <= 0) return;
  if (n_out < 0x7fffffffLL) hipLaunchKernelGGL((k_maxpool_fwd<uint32_t>), dim3(stream_grid(n_out, TPB * 2)), dim3(TPB), 0, g_stream, x, y, argmax, H, W, oH, oW, kH, kW, sH, sW, pad, n_out);
  else hipLaunchKernelGGL((k_maxpool_fwd<int64_t>), dim3(stream_grid(n_out, TPB * 2)), dim3(TPB), 0, g_stream, x, y, argmax, H, W, oH, oW, kH, kW, sH, sW, pad, n_out);
  LH_CHECK_LAUNCH();
}
void lh_maxpool_bwd(const float* dy, const int* argmax, float* dx, int64_t n_out) {
  ProfScope prof_(CAT_POOL);
  if (n_out <= 0) return;
  hipLaunchKernelGGL(k_maxpool_bwd_atomic, dim3(stream_grid(n_out, TPB * 4)), dim3(TPB), 0, g_stream, dy, argmax, dx, n_out);
  LH_CHECK_LAUNCH();
}
void lh_maxpool_bwd_dense(const float* dy, const int* argmax, float* dx, float beta,
                          int N, int C, int H, int W, int kH, int kW, int sH, int sW, int pad) {
  ProfScope prof_(CAT_POOL);
  LH_REQUIRE(kH >= 1 && kW >= 1 && sH >= 1 && sW >= 1 && pad >= 0, "lh_maxpool_bwd_dense: kernel/stride must be >= 1 and pad >= 0");
  LH_REQUIRE(H + 2 * pad >= kH && W + 2 * pad >= kW, "lh_maxpool_bwd_dense: image %dx%d too small for (%d,%d)", H, W, kH, kW);
  LH_REQUIRE(beta == 0.f || beta == 1.f, "lh_maxpool_bwd_dense: beta must be 0 or 1");
  const int64_t n_in = (int64_t)N * C * H * W;
  LH_REQUIRE(n_in < 2147483647LL, "lh_maxpool_bwd_dense: input too large for int32 argmax");
  if (n_in <= 0) return;
  const int oH = (H + 2 * pad - kH) / sH + 1, oW = (W + 2 * pad - kW) / sW + 1;
  const int grid = stream_grid(n_in, TPB * 2);
  if (beta == 0.f) hipLaunchKernelGGL((k_maxpool_bwd_dense<false>), dim3(grid), dim3(TPB), 0, g_stream, dy, argmax, dx, H, W, oH, oW, kH, kW, sH, sW, pad, n_in);
  else hipLaunchKernelGGL((k_maxpool_bwd_dense<true>), dim3(grid), dim3(TPB), 0, g_stream, dy, argmax, dx, H, W, oH, oW, kH, kW, sH, sW, pad, n_in);
  LH_CHECK_LAUNCH();
}
void lh_avgpool_fwd(const float* x, float* y, int N, int C, int H, int W, int kH, int kW, int sH, int sW) {
  ProfScope prof_(CAT_POOL);
  LH_REQUIRE(kH >= 1 && kW >= 1 && sH >= 1 && sW >= 1 && H >= kH && W >= kW, "lh_avgpool_fwd: bad kernel/stride for %dx%d", H, W);
  int oH = (H - kH) / sH + 1, oW = (W - kW) / sW + 1;
  int64_t n_out = (int64_t)N * C * oH * oW;
  if (n_out <= 0) return;
  hipLaunchKernelGGL(k_avgpool_fwd, dim3(stream_grid(n_out, TPB)), dim3(TPB), 0, g_stream, x, y, H, W, oH, oW, kH, kW, sH, sW, n_out);
  LH_CHECK_LAUNCH();
}
void lh_avgpool_bwd(const float* dy, float* dx, int N, int C, int H, int W, int kH, int kW, int sH, int sW) {
  ProfScope prof_(CAT_POOL);
  LH_REQUIRE(kH >= 1 && kW >= 1 && sH >= 1 && sW >= 1 && H >= kH && W >= kW, "lh_avgpool_bwd: bad kernel/stride for %dx%d", H, W);
  int oH = (H - kH) / sH + 1, oW = (W - kW) / sW + 1;
  int64_t n_in = (int64_t)N * C * H * W;
  if (n_in <= 0) return;
  hipLaunchKernelGGL(k_avgpool_bwd, dim3(stream_grid(n_in, TPB * 2)), dim3(TPB), 0, g_stream, dy, dx, H, W, oH, oW, kH, kW, sH, sW, n_in);
  LH_CHECK_LAUNCH();
}

}  // extern "C"
