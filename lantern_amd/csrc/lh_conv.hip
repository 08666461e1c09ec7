// conv2D_batch forward, input gradient and filter gradient (NCHW fp32 cross-correlation).
#include "lh_common.h"
using namespace lh;

namespace {
constexpr int TPB = 256;

struct ConvDims { int N, C, H, W, K, R, S, sH, sW, pH, pW, P, Q; };

__global__ void __launch_bounds__(TPB) k_conv_fwd_direct(const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ bias,
                                                         float* __restrict__ y, ConvDims d, int64_t n_out) {
  int64_t o = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; o < n_out; o += st) {
    int q = (int)(o % d.Q); int64_t t = o / d.Q; int p = (int)(t % d.P); t /= d.P; int k = (int)(t % d.K); int n = (int)(t / d.K);
    float acc = bias ? bias[k] : 0.f;
    for (int c = 0; c < d.C; c++)
      for (int r = 0; r < d.R; r++) {
        int h = p * d.sH - d.pH + r;
        if (h < 0 || h >= d.H) continue;
        for (int s = 0; s < d.S; s++) {
          int ww = q * d.sW - d.pW + s;
          if (ww < 0 || ww >= d.W) continue;
          acc += x[(((int64_t)n * d.C + c) * d.H + h) * d.W + ww] * w[(((int64_t)k * d.C + c) * d.R + r) * d.S + s];
        }
      }
    y[o] = acc;
  }
}
__global__ void __launch_bounds__(TPB) k_conv_bwd_data_direct(const float* __restrict__ dy, const float* __restrict__ w, float* __restrict__ dx,
                                                              float beta, ConvDims d, int64_t n_in) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n_in; i += st) {
    int ww = (int)(i % d.W); int64_t t = i / d.W; int h = (int)(t % d.H); t /= d.H; int c = (int)(t % d.C); int n = (int)(t / d.C);
    float acc = 0.f;
    for (int r = 0; r < d.R; r++) {
      int hp = h + d.pH - r;
      if (hp < 0 || hp % d.sH) continue;
      int p = hp / d.sH; if (p >= d.P) continue;
      for (int s = 0; s < d.S; s++) {
        int wq = ww + d.pW - s;
        if (wq < 0 || wq % d.sW) continue;
        int q = wq / d.sW; if (q >= d.Q) continue;
        for (int k = 0; k < d.K; k++)
          acc += dy[(((int64_t)n * d.K + k) * d.P + p) * d.Q + q] * w[(((int64_t)k * d.C + c) * d.R + r) * d.S + s];
      }
    }
    dx[i] = acc + (beta == 0.f ? 0.f : beta * dx[i]);
  }
}
// one block per filter element (k, c, r, s): reduce over n, p, q
__global__ void __launch_bounds__(TPB) k_conv_bwd_filter_direct(const float* __restrict__ x, const float* __restrict__ dy, float* __restrict__ dw,
                                                                float beta, ConvDims d) {
  __shared__ float sm[17];
  int e = blockIdx.x;
  int s = e % d.S; int t = e / d.S; int r = t % d.R; t /= d.R; int c = t % d.C; int k = t / d.C;
  int64_t tot = (int64_t)d.N * d.P * d.Q;
  float acc = 0.f;
  for (int64_t j = threadIdx.x; j < tot; j += TPB) {
    int q = (int)(j % d.Q); int64_t u = j / d.Q; int p = (int)(u % d.P); int n = (int)(u / d.P);
    int h = p * d.sH - d.pH + r, ww = q * d.sW - d.pW + s;
    if (h < 0 || h >= d.H || ww < 0 || ww >= d.W) continue;
    acc += dy[(((int64_t)n * d.K + k) * d.P + p) * d.Q + q] * x[(((int64_t)n * d.C + c) * d.H + h) * d.W + ww];
  }
  acc = lh_block_sum(acc, sm);
  if (threadIdx.x == 0) dw[e] = acc + (beta == 0.f ? 0.f : beta * dw[e]);
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

static bool make_dims(ConvDims& d, int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW) {
  if (N < 1 || C < 1 || H < 1 || W < 1 || K < 1 || R < 1 || S < 1 || sH < 1 || sW < 1 || pH < 0 || pW < 0) return false;
  if (H + 2 * pH < R || W + 2 * pW < S) return false;
  d = {N, C, H, W, K, R, S, sH, sW, pH, pW, (H + 2 * pH - R) / sH + 1, (W + 2 * pW - S) / sW + 1};
  return true;
}
}  // namespace

extern "C" {

void lh_conv2d_fwd(const float* x, const float* w, const float* bias, float* y,
                   int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW) {
  ConvDims d;
  LH_REQUIRE(make_dims(d, N, C, H, W, K, R, S, sH, sW, pH, pW), "lh_conv2d_fwd: bad shape N%d C%d H%d W%d K%d R%d S%d s(%d,%d) p(%d,%d)", N, C, H, W, K, R, S, sH, sW, pH, pW);
  int64_t n_out = (int64_t)N * K * d.P * d.Q;
  hipLaunchKernelGGL(k_conv_fwd_direct, dim3(stream_grid(n_out, TPB)), dim3(TPB), 0, g_stream, x, w, bias, y, d, n_out);
  LH_CHECK_LAUNCH();
}
void lh_conv2d_bwd_data(const float* dy, const float* w, float* dx, float beta,
                        int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW) {
  ConvDims d;
  LH_REQUIRE(make_dims(d, N, C, H, W, K, R, S, sH, sW, pH, pW), "lh_conv2d_bwd_data: bad shape");
  int64_t n_in = (int64_t)N * C * H * W;
  hipLaunchKernelGGL(k_conv_bwd_data_direct, dim3(stream_grid(n_in, TPB)), dim3(TPB), 0, g_stream, dy, w, dx, beta, d, n_in);
  LH_CHECK_LAUNCH();
}
void lh_conv2d_bwd_filter(const float* x, const float* dy, float* dw, float* db, float beta,
                          int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW) {
  ConvDims d;
  LH_REQUIRE(make_dims(d, N, C, H, W, K, R, S, sH, sW, pH, pW), "lh_conv2d_bwd_filter: bad shape");
  hipLaunchKernelGGL(k_conv_bwd_filter_direct, dim3(K * C * R * S), dim3(TPB), 0, g_stream, x, dy, dw, beta, d);
  if (db) hipLaunchKernelGGL(k_conv_bwd_bias, dim3(K), dim3(TPB), 0, g_stream, dy, db, N, K, d.P * d.Q);
  LH_CHECK_LAUNCH();
}

}  // extern "C"
