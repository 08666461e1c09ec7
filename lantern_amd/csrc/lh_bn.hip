// Batch normalisation, training forward / backward and inference, for x viewed as [N, C, HW].
// HBM-bound: the forward reads x twice and writes y (12 B/element), the backward reads x and
// dy twice and writes dx (20 B/element, 24 when dx accumulates).  Each pass is a 2-D grid
// (channel, slice of the batch) so that even 64-channel layers fill 256 CUs; per-slice
// partial statistics go through a small device scratch and are combined (Chan's parallel
// variance formula, in double) by every block of the second pass.
#include "lh_common.h"
using namespace lh;

namespace {
constexpr int TPB = 256;
constexpr int MAX_PARTIALS = 1 << 16;           // C * slices upper bound
__device__ float g_bn_partial[3 * MAX_PARTIALS];
static float* g_partial_ptr = nullptr;

struct Plan { int slices; int n_per; bool vec4; };
static Plan make_plan(int N, int C, int HW, bool aligned) {
  Plan p;
  int want = (int)cdiv(8 * (int64_t)g_num_cu, C);          // aim at ~8 blocks per CU in total
  if (want < 1) want = 1;
  if (want > N) want = N;
  // keep at least ~4096 elements per block
  int64_t per_sample = HW;
  int min_n = (int)cdiv(4096, per_sample);
  int max_slices = N / (min_n < 1 ? 1 : min_n); if (max_slices < 1) max_slices = 1;
  if (want > max_slices) want = max_slices;
  while ((int64_t)want * C > MAX_PARTIALS && want > 1) want--;
  p.n_per = (int)cdiv(N, want);
  p.slices = (int)cdiv(N, p.n_per);
  p.vec4 = (HW % 4) == 0 && aligned;
  return p;
}

// Visit the elements of channel c in samples [n0, n1): f4(offset) per aligned group of four
// when VEC (HW % 4 == 0), else f1(offset) per element.
template <bool VEC, class F4, class F1>
__device__ __forceinline__ void bn_foreach(int n0, int n1, int C, int c, int HW, F4 f4, F1 f1) {
  if (VEC) {
    const int U = HW >> 2; const int64_t total = (int64_t)(n1 - n0) * U;
    for (int64_t u = threadIdx.x; u < total; u += TPB) {
      int dn = (int)(u / U); int q = (int)(u - (int64_t)dn * U);
      f4(((int64_t)(n0 + dn) * C + c) * HW + 4 * q);
    }
  } else {
    const int64_t total = (int64_t)(n1 - n0) * HW;
    for (int64_t u = threadIdx.x; u < total; u += TPB) {
      int dn = (int)(u / HW); int l = (int)(u - (int64_t)dn * HW);
      f1(((int64_t)(n0 + dn) * C + c) * HW + l);
    }
  }
}

// y = gamma * (x - mean) * invstd + beta with a fixed operation order (no contraction choices left to
// the compiler): the backward pass of a fused BN+relu recomputes it to rebuild the relu mask, and
// must get the forward's value bit for bit.
__device__ __forceinline__ float bn_affine(float v, float mean, float invstd, float g, float b) {
  return __fmaf_rn(__fmul_rn(__fsub_rn(v, mean), invstd), g, b);
}

template <bool VEC>
__global__ void __launch_bounds__(TPB) k_bn_stats(const float* __restrict__ x, float* __restrict__ partial, int N, int C, int HW, int n_per) {
  __shared__ float sm[17];
  const int c = blockIdx.x, s = blockIdx.y;
  const int n0 = s * n_per, n1 = min(N, n0 + n_per);
  const float K = x[((int64_t)n0 * C + c) * HW];      // shift: removes cancellation in sum of squares
  float s1 = 0.f, s2 = 0.f;
  bn_foreach<VEC>(n0, n1, C, c, HW,
    [&](int64_t off) { float4 v = *reinterpret_cast<const float4*>(x + off);
      float a = v.x - K, b = v.y - K, d = v.z - K, e = v.w - K;
      s1 += (a + b) + (d + e); s2 += (a * a + b * b) + (d * d + e * e); },
    [&](int64_t off) { float a = x[off] - K; s1 += a; s2 += a * a; });
  s1 = lh_block_sum(s1, sm);
  s2 = lh_block_sum(s2, sm);
  if (threadIdx.x == 0) {
    float cnt = (float)((int64_t)(n1 - n0) * HW);
    float* p = partial + 3 * ((int64_t)c * gridDim.y + s);
    p[0] = K + s1 / cnt;            // slice mean
    p[1] = s2 - s1 * s1 / cnt;      // slice M2
    p[2] = cnt;
  }
}

__device__ __forceinline__ void combine_stats(const float* partial, int c, int slices, double& mean, double& m2, double& cnt) {
  cnt = 0.0; double wsum = 0.0;
  for (int s = 0; s < slices; s++) { const float* p = partial + 3 * ((int64_t)c * slices + s); cnt += p[2]; wsum += (double)p[0] * p[2]; }
  mean = wsum / cnt; m2 = 0.0;
  for (int s = 0; s < slices; s++) { const float* p = partial + 3 * ((int64_t)c * slices + s); double d = p[0] - mean; m2 += p[1] + p[2] * d * d; }
}

template <bool VEC, bool RELU>
__global__ void __launch_bounds__(TPB) k_bn_fwd_apply(const float* __restrict__ x, float* __restrict__ y, const float* __restrict__ partial,
                                                      const float* gamma, const float* beta, float* run_mean, float* run_var,
                                                      float* save_mean, float* save_invstd, int N, int C, int HW, int n_per, float eps, float factor) {
  __shared__ float sh[2];
  const int c = blockIdx.x, s = blockIdx.y;
  if (threadIdx.x == 0) {
    double mean, m2, cnt;
    combine_stats(partial, c, gridDim.y, mean, m2, cnt);
    float var = (float)(m2 / cnt);
    float invstd = 1.0f / sqrtf(var + eps);
    sh[0] = (float)mean; sh[1] = invstd;
    if (s == 0) {
      if (save_mean) save_mean[c] = (float)mean;
      if (save_invstd) save_invstd[c] = invstd;
      if (run_mean) run_mean[c] = (1.0f - factor) * run_mean[c] + factor * (float)mean;
      if (run_var) { float unb = cnt > 1.0 ? (float)(m2 / (cnt - 1.0)) : var; run_var[c] = (1.0f - factor) * run_var[c] + factor * unb; }
    }
  }
  __syncthreads();
  const float mean = sh[0], invstd = sh[1], g = gamma[c], b = beta[c];
  const int n0 = s * n_per, n1 = min(N, n0 + n_per);
  bn_foreach<VEC>(n0, n1, C, c, HW,
    [&](int64_t off) { float4 v = *reinterpret_cast<const float4*>(x + off); float4 r;
      r.x = bn_affine(v.x, mean, invstd, g, b); r.y = bn_affine(v.y, mean, invstd, g, b);
      r.z = bn_affine(v.z, mean, invstd, g, b); r.w = bn_affine(v.w, mean, invstd, g, b);
      if (RELU) { r.x = r.x < 0.f ? 0.f : r.x; r.y = r.y < 0.f ? 0.f : r.y; r.z = r.z < 0.f ? 0.f : r.z; r.w = r.w < 0.f ? 0.f : r.w; }
      *reinterpret_cast<float4*>(y + off) = r; },
    [&](int64_t off) { float r = bn_affine(x[off], mean, invstd, g, b); if (RELU) r = r < 0.f ? 0.f : r; y[off] = r; });
}

// RELU: the layer's output y went through an in-place relu; the incoming gradient counts only where y > 0.
//   RELU == 1: the mask is read from the stored y;  RELU == 2: it is recomputed from x (y is not read).
template <bool VEC, int RELU>
__global__ void __launch_bounds__(TPB) k_bn_bwd_stats(const float* __restrict__ x, const float* __restrict__ yv, const float* __restrict__ dy,
                                                      const float* save_mean, const float* save_invstd, const float* gamma, const float* bias,
                                                      float* __restrict__ partial, int N, int C, int HW, int n_per) {
  __shared__ float sm[17];
  const int c = blockIdx.x, s = blockIdx.y;
  const int n0 = s * n_per, n1 = min(N, n0 + n_per);
  const float mean = save_mean[c], is = save_invstd[c];
  const float ga = RELU == 2 ? gamma[c] : 0.f, bi = RELU == 2 ? bias[c] : 0.f;
  float s1 = 0.f, s2 = 0.f;
  bn_foreach<VEC>(n0, n1, C, c, HW,
    [&](int64_t off) { float4 v = *reinterpret_cast<const float4*>(x + off); float4 g = *reinterpret_cast<const float4*>(dy + off);
      if (RELU) { float4 m;
        if (RELU == 1) m = *reinterpret_cast<const float4*>(yv + off);
        else { m.x = bn_affine(v.x, mean, is, ga, bi); m.y = bn_affine(v.y, mean, is, ga, bi); m.z = bn_affine(v.z, mean, is, ga, bi); m.w = bn_affine(v.w, mean, is, ga, bi); }
        g.x = m.x > 0.f ? g.x : 0.f; g.y = m.y > 0.f ? g.y : 0.f; g.z = m.z > 0.f ? g.z : 0.f; g.w = m.w > 0.f ? g.w : 0.f; }
      s1 += (g.x + g.y) + (g.z + g.w);
      s2 += (g.x * ((v.x - mean) * is) + g.y * ((v.y - mean) * is)) + (g.z * ((v.z - mean) * is) + g.w * ((v.w - mean) * is)); },
    [&](int64_t off) { float g = dy[off]; if (RELU) { float m = RELU == 1 ? yv[off] : bn_affine(x[off], mean, is, ga, bi); g = m > 0.f ? g : 0.f; }
      s1 += g; s2 += g * ((x[off] - mean) * is); });
  s1 = lh_block_sum(s1, sm);
  s2 = lh_block_sum(s2, sm);
  if (threadIdx.x == 0) { float* p = partial + 3 * ((int64_t)c * gridDim.y + s); p[0] = s1; p[1] = s2; }
}

template <bool VEC, bool ACC, int RELU>
__global__ void __launch_bounds__(TPB) k_bn_bwd_apply(const float* __restrict__ x, const float* __restrict__ yv, const float* __restrict__ dy, const float* __restrict__ partial,
                                                      const float* gamma, const float* bias, const float* save_mean, const float* save_invstd,
                                                      float* __restrict__ dx, float* dgamma, float* dbeta, int N, int C, int HW, int n_per, int from_end) {
  __shared__ float sh[2];
  // from_end: blocks walk the tensor from its end.  The statistics pass that ran just before read it front to back, so on
  // tensors beyond the last-level cache the part touched last is the part still there (measured: 5 % on 2 x 206 MB,
  // a loss on tensors that fit, hence the switch).
  const int c = from_end ? gridDim.x - 1 - blockIdx.x : blockIdx.x, s = from_end ? gridDim.y - 1 - blockIdx.y : blockIdx.y;
  if (threadIdx.x == 0) {
    double a = 0.0, b = 0.0;
    for (int t = 0; t < (int)gridDim.y; t++) { const float* p = partial + 3 * ((int64_t)c * gridDim.y + t); a += p[0]; b += p[1]; }
    double cnt = (double)N * HW;
    sh[0] = (float)(a / cnt); sh[1] = (float)(b / cnt);
    if (s == 0) { if (dgamma) dgamma[c] += (float)b; if (dbeta) dbeta[c] += (float)a; }
  }
  __syncthreads();
  if (dx == nullptr) return;
  const float m1 = sh[0], m2 = sh[1], mean = save_mean[c], is = save_invstd[c], ga = gamma[c], g = ga * is;
  const float bi = RELU == 2 ? bias[c] : 0.f;
  const int n0 = s * n_per, n1 = min(N, n0 + n_per);
  bn_foreach<VEC>(n0, n1, C, c, HW,
    [&](int64_t off) { float4 v = *reinterpret_cast<const float4*>(x + off); float4 d = *reinterpret_cast<const float4*>(dy + off); float4 r;
      if (RELU) { float4 m;
        if (RELU == 1) m = *reinterpret_cast<const float4*>(yv + off);
        else { m.x = bn_affine(v.x, mean, is, ga, bi); m.y = bn_affine(v.y, mean, is, ga, bi); m.z = bn_affine(v.z, mean, is, ga, bi); m.w = bn_affine(v.w, mean, is, ga, bi); }
        d.x = m.x > 0.f ? d.x : 0.f; d.y = m.y > 0.f ? d.y : 0.f; d.z = m.z > 0.f ? d.z : 0.f; d.w = m.w > 0.f ? d.w : 0.f; }
      r.x = g * (d.x - m1 - (v.x - mean) * is * m2); r.y = g * (d.y - m1 - (v.y - mean) * is * m2);
      r.z = g * (d.z - m1 - (v.z - mean) * is * m2); r.w = g * (d.w - m1 - (v.w - mean) * is * m2);
      if (ACC) { float4 o = *reinterpret_cast<const float4*>(dx + off); r.x += o.x; r.y += o.y; r.z += o.z; r.w += o.w; }
      *reinterpret_cast<float4*>(dx + off) = r; },
    [&](int64_t off) { float d = dy[off]; if (RELU) { float m = RELU == 1 ? yv[off] : bn_affine(x[off], mean, is, ga, bi); d = m > 0.f ? d : 0.f; }
      float r = g * (d - m1 - (x[off] - mean) * is * m2); if (ACC) r += dx[off]; dx[off] = r; });
}

// ---- small maps: a whole channel in one block ---------------------------------------------------------------------------------
// When a channel's N*HW elements fit the registers of one block (the 14x14 and 7x7 maps of a network's last stages at batch
// 64), the two passes of the kernels above (statistics, then apply, each a launch that re-reads the tensor and costs as much
// in launch latency as in traffic at these sizes) become one: every thread loads its PER units (groups of four elements when
// HW % 4 == 0, single elements otherwise) once, the block reduces, and the result is written from the registers.
// Forward 8 instead of 12 bytes per element, backward 12 instead of 20, one launch each.
constexpr int SMALL_PER = 16;
static bool small_fits(int N, int HW, bool vec) { return (int64_t)N * (vec ? HW / 4 : HW) <= (int64_t)SMALL_PER * TPB; }

template <bool VEC> struct SmallUnit { typedef float T; };
template <> struct SmallUnit<true> { typedef float4 T; };

template <bool VEC, bool RELU>
__global__ void __launch_bounds__(TPB) k_bn_small_fwd(const float* __restrict__ x, float* __restrict__ y, const float* gamma, const float* beta, float* run_mean, float* run_var,
                                                      float* save_mean, float* save_invstd, int N, int C, int HW, float eps, float factor) {
  __shared__ float sm[17];
  typedef typename SmallUnit<VEC>::T U;
  const int c = blockIdx.x, W = VEC ? HW >> 2 : HW, total = N * W;
  const float K = x[(int64_t)c * HW];                  // shift: removes cancellation in the sum of squares
  U v[SMALL_PER]; int64_t off[SMALL_PER];
#pragma unroll
  for (int k = 0; k < SMALL_PER; k++) {
    const int u = threadIdx.x + k * TPB;
    const int dn = u / W, q = u - dn * W;
    off[k] = u < total ? ((int64_t)dn * C + c) * HW + (VEC ? 4 * q : q) : -1;
    if (off[k] >= 0) v[k] = *reinterpret_cast<const U*>(x + off[k]);
  }
  float s1 = 0.f, s2 = 0.f;
#pragma unroll
  for (int k = 0; k < SMALL_PER; k++) if (off[k] >= 0) {
    if constexpr (VEC) { const float a = v[k].x - K, b = v[k].y - K, d = v[k].z - K, e = v[k].w - K; s1 += (a + b) + (d + e); s2 += (a * a + b * b) + (d * d + e * e); }
    else { const float a = v[k] - K; s1 += a; s2 += a * a; }
  }
  s1 = lh_block_sum(s1, sm);
  s2 = lh_block_sum(s2, sm);
  const float cnt = (float)((int64_t)N * HW);
  const float mean = K + s1 / cnt, m2 = s2 - s1 * s1 / cnt;
  const float var = m2 / cnt, invstd = 1.0f / sqrtf(var + eps);
  if (threadIdx.x == 0) {
    if (save_mean) save_mean[c] = mean;
    if (save_invstd) save_invstd[c] = invstd;
    if (run_mean) run_mean[c] = (1.0f - factor) * run_mean[c] + factor * mean;
    if (run_var) { const float unb = cnt > 1.0f ? m2 / (cnt - 1.0f) : var; run_var[c] = (1.0f - factor) * run_var[c] + factor * unb; }
  }
  const float g = gamma[c], b = beta[c];
#pragma unroll
  for (int k = 0; k < SMALL_PER; k++) if (off[k] >= 0) {
    if constexpr (VEC) {
      float4 r;
      r.x = bn_affine(v[k].x, mean, invstd, g, b); r.y = bn_affine(v[k].y, mean, invstd, g, b);
      r.z = bn_affine(v[k].z, mean, invstd, g, b); r.w = bn_affine(v[k].w, mean, invstd, g, b);
      if (RELU) { r.x = r.x < 0.f ? 0.f : r.x; r.y = r.y < 0.f ? 0.f : r.y; r.z = r.z < 0.f ? 0.f : r.z; r.w = r.w < 0.f ? 0.f : r.w; }
      *reinterpret_cast<float4*>(y + off[k]) = r;
    } else { float r = bn_affine(v[k], mean, invstd, g, b); if (RELU) r = r < 0.f ? 0.f : r; y[off[k]] = r; }
  }
}

// RELU as in k_bn_bwd_stats: 0 none, 1 mask from the stored y, 2 mask recomputed from x.
template <bool VEC, bool ACC, int RELU>
__global__ void __launch_bounds__(TPB) k_bn_small_bwd(const float* __restrict__ x, const float* __restrict__ yv, const float* __restrict__ dy, const float* gamma, const float* bias,
                                                      const float* save_mean, const float* save_invstd, float* __restrict__ dx, float* dgamma, float* dbeta,
                                                      int N, int C, int HW) {
  __shared__ float sm[17];
  typedef typename SmallUnit<VEC>::T U;
  const int c = blockIdx.x, W = VEC ? HW >> 2 : HW, total = N * W;
  const float mean = save_mean[c], is = save_invstd[c], ga = gamma[c];
  const float bi = RELU == 2 ? bias[c] : 0.f;
  U v[SMALL_PER], d[SMALL_PER]; int64_t off[SMALL_PER];
#pragma unroll
  for (int k = 0; k < SMALL_PER; k++) {
    const int u = threadIdx.x + k * TPB;
    const int dn = u / W, q = u - dn * W;
    off[k] = u < total ? ((int64_t)dn * C + c) * HW + (VEC ? 4 * q : q) : -1;
    if (off[k] >= 0) {
      v[k] = *reinterpret_cast<const U*>(x + off[k]); d[k] = *reinterpret_cast<const U*>(dy + off[k]);
      if (RELU == 1) {
        const U m = *reinterpret_cast<const U*>(yv + off[k]);
        if constexpr (VEC) { d[k].x = m.x > 0.f ? d[k].x : 0.f; d[k].y = m.y > 0.f ? d[k].y : 0.f; d[k].z = m.z > 0.f ? d[k].z : 0.f; d[k].w = m.w > 0.f ? d[k].w : 0.f; }
        else d[k] = m > 0.f ? d[k] : 0.f;
      }
    }
  }
  float s1 = 0.f, s2 = 0.f;
#pragma unroll
  for (int k = 0; k < SMALL_PER; k++) if (off[k] >= 0) {
    if constexpr (VEC) {
      if (RELU == 2) {
        d[k].x = bn_affine(v[k].x, mean, is, ga, bi) > 0.f ? d[k].x : 0.f; d[k].y = bn_affine(v[k].y, mean, is, ga, bi) > 0.f ? d[k].y : 0.f;
        d[k].z = bn_affine(v[k].z, mean, is, ga, bi) > 0.f ? d[k].z : 0.f; d[k].w = bn_affine(v[k].w, mean, is, ga, bi) > 0.f ? d[k].w : 0.f;
      }
      s1 += (d[k].x + d[k].y) + (d[k].z + d[k].w);
      s2 += (d[k].x * ((v[k].x - mean) * is) + d[k].y * ((v[k].y - mean) * is)) + (d[k].z * ((v[k].z - mean) * is) + d[k].w * ((v[k].w - mean) * is));
    } else {
      if (RELU == 2) d[k] = bn_affine(v[k], mean, is, ga, bi) > 0.f ? d[k] : 0.f;
      s1 += d[k]; s2 += d[k] * ((v[k] - mean) * is);
    }
  }
  s1 = lh_block_sum(s1, sm);
  s2 = lh_block_sum(s2, sm);
  if (threadIdx.x == 0) { if (dgamma) dgamma[c] += s2; if (dbeta) dbeta[c] += s1; }
  if (dx == nullptr) return;
  const float cnt = (float)((int64_t)N * HW), m1 = s1 / cnt, m2 = s2 / cnt, g = ga * is;
#pragma unroll
  for (int k = 0; k < SMALL_PER; k++) if (off[k] >= 0) {
    if constexpr (VEC) {
      float4 r;
      r.x = g * (d[k].x - m1 - (v[k].x - mean) * is * m2); r.y = g * (d[k].y - m1 - (v[k].y - mean) * is * m2);
      r.z = g * (d[k].z - m1 - (v[k].z - mean) * is * m2); r.w = g * (d[k].w - m1 - (v[k].w - mean) * is * m2);
      if (ACC) { const float4 o = *reinterpret_cast<const float4*>(dx + off[k]); r.x += o.x; r.y += o.y; r.z += o.z; r.w += o.w; }
      *reinterpret_cast<float4*>(dx + off[k]) = r;
    } else { float r = g * (d[k] - m1 - (v[k] - mean) * is * m2); if (ACC) r += dx[off[k]]; dx[off[k]] = r; }
  }
}

// Backward of out = relu(bn(x) + shortcut) for a small map, one launch: the incoming gradient masked with out > 0 goes to the
// shortcut's gradient (DS 1: written, DS 2: added, DS 0: the shortcut is an input) and through the batch norm into dx.
template <bool VEC, bool ACC, int DS>
__global__ void __launch_bounds__(TPB) k_bn_small_bwd_join(const float* __restrict__ x, const float* __restrict__ out, const float* __restrict__ dout, float* __restrict__ ds,
                                                           const float* gamma, const float* save_mean, const float* save_invstd, float* __restrict__ dx,
                                                           float* dgamma, float* dbeta, int N, int C, int HW) {
  __shared__ float sm[17];
  typedef typename SmallUnit<VEC>::T U;
  const int c = blockIdx.x, W = VEC ? HW >> 2 : HW, total = N * W;
  const float mean = save_mean[c], is = save_invstd[c], ga = gamma[c];
  U v[SMALL_PER], d[SMALL_PER]; int64_t off[SMALL_PER];
#pragma unroll
  for (int k = 0; k < SMALL_PER; k++) {
    const int u = threadIdx.x + k * TPB;
    const int dn = u / W, q = u - dn * W;
    off[k] = u < total ? ((int64_t)dn * C + c) * HW + (VEC ? 4 * q : q) : -1;
    if (off[k] >= 0) {
      v[k] = *reinterpret_cast<const U*>(x + off[k]); d[k] = *reinterpret_cast<const U*>(dout + off[k]);
      const U m = *reinterpret_cast<const U*>(out + off[k]);
      if constexpr (VEC) { d[k].x = m.x > 0.f ? d[k].x : 0.f; d[k].y = m.y > 0.f ? d[k].y : 0.f; d[k].z = m.z > 0.f ? d[k].z : 0.f; d[k].w = m.w > 0.f ? d[k].w : 0.f; }
      else d[k] = m > 0.f ? d[k] : 0.f;
      if (DS == 1) *reinterpret_cast<U*>(ds + off[k]) = d[k];
      if (DS == 2) {
        U o = *reinterpret_cast<const U*>(ds + off[k]);
        if constexpr (VEC) { o.x += d[k].x; o.y += d[k].y; o.z += d[k].z; o.w += d[k].w; } else o += d[k];
        *reinterpret_cast<U*>(ds + off[k]) = o;
      }
    }
  }
  float s1 = 0.f, s2 = 0.f;
#pragma unroll
  for (int k = 0; k < SMALL_PER; k++) if (off[k] >= 0) {
    if constexpr (VEC) {
      s1 += (d[k].x + d[k].y) + (d[k].z + d[k].w);
      s2 += (d[k].x * ((v[k].x - mean) * is) + d[k].y * ((v[k].y - mean) * is)) + (d[k].z * ((v[k].z - mean) * is) + d[k].w * ((v[k].w - mean) * is));
    } else { s1 += d[k]; s2 += d[k] * ((v[k] - mean) * is); }
  }
  s1 = lh_block_sum(s1, sm);
  s2 = lh_block_sum(s2, sm);
  if (threadIdx.x == 0) { if (dgamma) dgamma[c] += s2; if (dbeta) dbeta[c] += s1; }
  if (dx == nullptr) return;
  const float cnt = (float)((int64_t)N * HW), m1 = s1 / cnt, m2 = s2 / cnt, g = ga * is;
#pragma unroll
  for (int k = 0; k < SMALL_PER; k++) if (off[k] >= 0) {
    if constexpr (VEC) {
      float4 r;
      r.x = g * (d[k].x - m1 - (v[k].x - mean) * is * m2); r.y = g * (d[k].y - m1 - (v[k].y - mean) * is * m2);
      r.z = g * (d[k].z - m1 - (v[k].z - mean) * is * m2); r.w = g * (d[k].w - m1 - (v[k].w - mean) * is * m2);
      if (ACC) { const float4 o = *reinterpret_cast<const float4*>(dx + off[k]); r.x += o.x; r.y += o.y; r.z += o.z; r.w += o.w; }
      *reinterpret_cast<float4*>(dx + off[k]) = r;
    } else { float r = g * (d[k] - m1 - (v[k] - mean) * is * m2); if (ACC) r += dx[off[k]]; dx[off[k]] = r; }
  }
}

__global__ void __launch_bounds__(TPB) k_bn_infer(const float* __restrict__ x, float* __restrict__ y, const float* gamma, const float* beta,
                                                  const float* rmean, const float* rvar, int C, int HW, int64_t n, float eps) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n; i += st) {
    int c = (int)((i / HW) % C);
    y[i] = (x[i] - rmean[c]) / sqrtf(rvar[c] + eps) * gamma[c] + beta[c];
  }
}

// ---- HW == 1 (BatchNorm1D over [rows, C]): the elements of a channel lie C floats apart, so the (channel, slice) blocks
// above would touch one cache line per element.  Here a block takes 64 neighbouring channels (a 256-byte row segment per
// load, coalesced) times a slice of the rows; four row lanes per channel are combined through LDS.  The partial sums have
// the layout of the kernels above, so statistics finalisation and the other passes are shared.
constexpr int C1 = 64;                          // channels per block
struct Plan1 { int slices, rows_per; };
static Plan1 make_plan1(int N, int C) {
  const int colb = (int)cdiv(C, C1);
  int want = (int)cdiv(2 * (int64_t)g_num_cu, colb);
  if (want > 16) want = 16;                  // every thread of the second pass walks the slices' partial sums
  int max_slices = N / 32; if (max_slices < 1) max_slices = 1;         // at least 32 rows per block
  if (want > max_slices) want = max_slices;
  if (want < 1) want = 1;
  while ((int64_t)want * C > MAX_PARTIALS && want > 1) want--;
  Plan1 p; p.rows_per = (int)cdiv(N, want); p.slices = (int)cdiv(N, p.rows_per);
  return p;
}
__global__ void __launch_bounds__(TPB) k_bn1d_stats(const float* __restrict__ x, float* __restrict__ partial, int N, int C, int rows_per) {
  __shared__ float sh[2][4][C1];
  const int cx = threadIdx.x & (C1 - 1), ry = threadIdx.x >> 6;
  const int c = blockIdx.x * C1 + cx, s = blockIdx.y;
  const int n0 = s * rows_per, n1 = min(N, n0 + rows_per);
  const bool ok = c < C;
  const float K = ok ? x[(int64_t)n0 * C + c] : 0.f;          // shift, as k_bn_stats
  float s1 = 0.f, s2 = 0.f;
  float t1 = 0.f, t2 = 0.f;                     // two independent chains: the loads of neighbouring iterations overlap
  if (ok) {
    int n = n0 + ry;
    for (; n + 4 < n1; n += 8) {
      const float a = x[(int64_t)n * C + c] - K, b = x[(int64_t)(n + 4) * C + c] - K;
      s1 += a; s2 += a * a; t1 += b; t2 += b * b;
    }
    if (n < n1) { const float a = x[(int64_t)n * C + c] - K; s1 += a; s2 += a * a; }
    s1 += t1; s2 += t2;
  }
  sh[0][ry][cx] = s1; sh[1][ry][cx] = s2;
  __syncthreads();
  if (ry == 0 && ok) {
    s1 = (sh[0][0][cx] + sh[0][1][cx]) + (sh[0][2][cx] + sh[0][3][cx]);
    s2 = (sh[1][0][cx] + sh[1][1][cx]) + (sh[1][2][cx] + sh[1][3][cx]);
    const float cnt = (float)(n1 - n0);
    float* p = partial + 3 * ((int64_t)c * gridDim.y + s);
    p[0] = K + s1 / cnt; p[1] = s2 - s1 * s1 / cnt; p[2] = cnt;
  }
}
__global__ void __launch_bounds__(TPB) k_bn1d_fwd_apply(const float* __restrict__ x, float* __restrict__ y, const float* __restrict__ partial,
                                                        const float* gamma, const float* beta, float* run_mean, float* run_var,
                                                        float* save_mean, float* save_invstd, int N, int C, int rows_per, float eps, float factor) {
  const int cx = threadIdx.x & (C1 - 1), ry = threadIdx.x >> 6;
  const int c = blockIdx.x * C1 + cx, s = blockIdx.y;
  if (c >= C) return;
  double mean, m2, cnt;
  combine_stats(partial, c, gridDim.y, mean, m2, cnt);        // every row lane of a channel gets the same bits
  const float var = (float)(m2 / cnt), invstd = 1.0f / sqrtf(var + eps), mu = (float)mean;
  if (s == 0 && ry == 0) {
    if (save_mean) save_mean[c] = mu;
    if (save_invstd) save_invstd[c] = invstd;
    if (run_mean) run_mean[c] = (1.0f - factor) * run_mean[c] + factor * mu;
    if (run_var) { float unb = cnt > 1.0 ? (float)(m2 / (cnt - 1.0)) : var; run_var[c] = (1.0f - factor) * run_var[c] + factor * unb; }
  }
  const float g = gamma[c], b = beta[c];
  const int n0 = s * rows_per, n1 = min(N, n0 + rows_per);
#pragma unroll 4
  for (int n = n0 + ry; n < n1; n += 4) { const int64_t o = (int64_t)n * C + c; y[o] = bn_affine(x[o], mu, invstd, g, b); }
}
__global__ void __launch_bounds__(TPB) k_bn1d_bwd_stats(const float* __restrict__ x, const float* __restrict__ dy, const float* save_mean, const float* save_invstd,
                                                        float* __restrict__ partial, int N, int C, int rows_per) {
  __shared__ float sh[2][4][C1];
  const int cx = threadIdx.x & (C1 - 1), ry = threadIdx.x >> 6;
  const int c = blockIdx.x * C1 + cx, s = blockIdx.y;
  const int n0 = s * rows_per, n1 = min(N, n0 + rows_per);
  const bool ok = c < C;
  const float mean = ok ? save_mean[c] : 0.f, is = ok ? save_invstd[c] : 0.f;
  float s1 = 0.f, s2 = 0.f;
  float t1 = 0.f, t2 = 0.f;
  if (ok) {
    int n = n0 + ry;
    for (; n + 4 < n1; n += 8) {
      const int64_t o = (int64_t)n * C + c, o2 = (int64_t)(n + 4) * C + c;
      const float g = dy[o], g2 = dy[o2], xa = x[o], xb = x[o2];
      s1 += g; s2 += g * ((xa - mean) * is); t1 += g2; t2 += g2 * ((xb - mean) * is);
    }
    if (n < n1) { const int64_t o = (int64_t)n * C + c; const float g = dy[o]; s1 += g; s2 += g * ((x[o] - mean) * is); }
    s1 += t1; s2 += t2;
  }
  sh[0][ry][cx] = s1; sh[1][ry][cx] = s2;
  __syncthreads();
  if (ry == 0 && ok) {
    float* p = partial + 3 * ((int64_t)c * gridDim.y + s);
    p[0] = (sh[0][0][cx] + sh[0][1][cx]) + (sh[0][2][cx] + sh[0][3][cx]);
    p[1] = (sh[1][0][cx] + sh[1][1][cx]) + (sh[1][2][cx] + sh[1][3][cx]);
  }
}
template <bool ACC>
__global__ void __launch_bounds__(TPB) k_bn1d_bwd_apply(const float* __restrict__ x, const float* __restrict__ dy, const float* __restrict__ partial,
                                                        const float* gamma, const float* save_mean, const float* save_invstd,
                                                        float* __restrict__ dx, float* dgamma, float* dbeta, int N, int C, int rows_per) {
  const int cx = threadIdx.x & (C1 - 1), ry = threadIdx.x >> 6;
  const int c = blockIdx.x * C1 + cx, s = blockIdx.y;
  if (c >= C) return;
  double a = 0.0, b = 0.0;
  for (int t = 0; t < (int)gridDim.y; t++) { const float* p = partial + 3 * ((int64_t)c * gridDim.y + t); a += p[0]; b += p[1]; }
  const double cnt = (double)N;
  const float m1 = (float)(a / cnt), m2 = (float)(b / cnt);
  if (s == 0 && ry == 0) { if (dgamma) dgamma[c] += (float)b; if (dbeta) dbeta[c] += (float)a; }
  if (dx == nullptr) return;
  const float mean = save_mean[c], is = save_invstd[c], g = gamma[c] * is;
  const int n0 = s * rows_per, n1 = min(N, n0 + rows_per);
#pragma unroll 4
  for (int n = n0 + ry; n < n1; n += 4) {
    const int64_t o = (int64_t)n * C + c;
    float r = g * (dy[o] - m1 - (x[o] - mean) * is * m2);
    if (ACC) r += dx[o];
    dx[o] = r;
  }
}

// Channel statistics from classic per-slice partials (mean, M2, count): one thread per channel.
__global__ void __launch_bounds__(TPB) k_bn_finalize(const float* __restrict__ partial, int C, int slices, float* save_mean, float* save_invstd,
                                                     float* run_mean, float* run_var, float eps, float factor) {
  const int c = blockIdx.x * TPB + threadIdx.x;
  if (c >= C) return;
  double mean, m2, cnt;
  combine_stats(partial, c, slices, mean, m2, cnt);
  const float var = (float)(m2 / cnt);
  if (save_mean) save_mean[c] = (float)mean;
  if (save_invstd) save_invstd[c] = 1.0f / sqrtf(var + eps);
  if (run_mean) run_mean[c] = (1.0f - factor) * run_mean[c] + factor * (float)mean;
  if (run_var) { float unb = cnt > 1.0 ? (float)(m2 / (cnt - 1.0)) : var; run_var[c] = (1.0f - factor) * run_var[c] + factor * unb; }
}

// Channel statistics from the (sum, sum of squares) pieces of a convolution epilogue: one block per channel adds the
// pieces up in double (they are fp32 sums of at most 64 values each, so double carries them exactly enough:
// M2 = sum q - (sum a)^2 / n loses about log2(n mean^2 / M2) of 53 bits) and finishes the channel.
__global__ void __launch_bounds__(TPB) k_bn_finalize_conv(const float* __restrict__ partial, int C, int ncols, int col1, int g_main, int slots_main, int g_rem,
                                                          int slots, float* save_mean, float* save_invstd, float* run_mean, float* run_var, float eps, float factor) {
  __shared__ double sa_[TPB], sq_[TPB];
  const int c = blockIdx.x;
  const float2* pc = reinterpret_cast<const float2*>(partial) + (size_t)c * slots;
  double sa = 0.0, sq = 0.0;
  for (int s = threadIdx.x; s < slots; s += TPB) {
    const int j0 = s < slots_main ? s * g_main : col1 + (s - slots_main) * g_rem;
    const int n = s < slots_main ? min(g_main, col1 - j0) : min(g_rem, ncols - j0);
    if (n <= 0) continue;                       // a slot behind the last column holds nothing
    const float2 pv = pc[s];
    sa += (double)pv.x; sq += (double)pv.y;
  }
  sa_[threadIdx.x] = sa; sq_[threadIdx.x] = sq;
  __syncthreads();
  for (int off = TPB / 2; off > 0; off >>= 1) {
    if (threadIdx.x < off) { sa_[threadIdx.x] += sa_[threadIdx.x + off]; sq_[threadIdx.x] += sq_[threadIdx.x + off]; }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    const double n = (double)ncols, mu = sa_[0] / n;
    double M2 = sq_[0] - sa_[0] * mu; if (M2 < 0.0) M2 = 0.0;
    const float var = (float)(M2 / n);
    if (save_mean) save_mean[c] = (float)mu;
    if (save_invstd) save_invstd[c] = 1.0f / sqrtf(var + eps);
    if (run_mean) run_mean[c] = (1.0f - factor) * run_mean[c] + factor * (float)mu;
    if (run_var) { float unb = n > 1.0 ? (float)(M2 / (n - 1.0)) : var; run_var[c] = (1.0f - factor) * run_var[c] + factor * unb; }
  }
}

// Mean and 1/sqrt(var + eps) of channel c from the pieces a convolution epilogue left, computed by the whole block exactly as
// k_bn_finalize_conv does (same partition over threads, same tree), so every block of a channel gets the same bits; the
// owner block also stores the saved and running statistics.
__device__ __forceinline__ void bn_stats_from_pieces(const ConvPieces& P, int c, bool owner, float& mean_out, float& invstd_out) {
  __shared__ double sa_[TPB], sq_[TPB];
  __shared__ float res_[2];
  const float2* pc = reinterpret_cast<const float2*>(P.partial) + (size_t)c * P.slots;
  double sa = 0.0, sq = 0.0;
  for (int s = threadIdx.x; s < P.slots; s += TPB) {
    const int j0 = s < P.slots_main ? s * P.g_main : P.col1 + (s - P.slots_main) * P.g_rem;
    const int n = s < P.slots_main ? min(P.g_main, P.col1 - j0) : min(P.g_rem, P.ncols - j0);
    if (n <= 0) continue;
    const float2 pv = pc[s];
    sa += (double)pv.x; sq += (double)pv.y;
  }
  sa_[threadIdx.x] = sa; sq_[threadIdx.x] = sq;
  __syncthreads();
  for (int off = TPB / 2; off > 0; off >>= 1) {
    if (threadIdx.x < off) { sa_[threadIdx.x] += sa_[threadIdx.x + off]; sq_[threadIdx.x] += sq_[threadIdx.x + off]; }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    const double n = (double)P.ncols, mu = sa_[0] / n;
    double M2 = sq_[0] - sa_[0] * mu; if (M2 < 0.0) M2 = 0.0;
    const float var = (float)(M2 / n);
    const float is = 1.0f / sqrtf(var + P.eps);
    res_[0] = (float)mu; res_[1] = is;
    if (owner) {
      if (P.save_mean) P.save_mean[c] = (float)mu;
      if (P.save_invstd) P.save_invstd[c] = is;
      if (P.run_mean) P.run_mean[c] = (1.0f - P.factor) * P.run_mean[c] + P.factor * (float)mu;
      if (P.run_var) { float unb = n > 1.0 ? (float)(M2 / (n - 1.0)) : var; P.run_var[c] = (1.0f - P.factor) * P.run_var[c] + P.factor * unb; }
    }
  }
  __syncthreads();
  mean_out = res_[0]; invstd_out = res_[1];
}

// y = gamma * (x - mean) * invstd + beta from given statistics (optionally followed by relu); PIECES: the statistics come
// from a convolution's pieces instead of save_mean / save_invstd
template <bool VEC, bool RELU, bool PIECES = false>
__global__ void __launch_bounds__(TPB) k_bn_apply(const float* __restrict__ x, float* __restrict__ y, const float* gamma, const float* beta,
                                                  const float* save_mean, const float* save_invstd, int N, int C, int HW, int n_per, ConvPieces P = ConvPieces()) {
  const int c = blockIdx.x, s = blockIdx.y;
  float mean, invstd;
  if (PIECES) bn_stats_from_pieces(P, c, s == 0, mean, invstd); else { mean = save_mean[c]; invstd = save_invstd[c]; }
  const float g = gamma[c], b = beta[c];
  const int n0 = s * n_per, n1 = min(N, n0 + n_per);
  bn_foreach<VEC>(n0, n1, C, c, HW,
    [&](int64_t off) { float4 v = *reinterpret_cast<const float4*>(x + off); float4 r;
      r.x = bn_affine(v.x, mean, invstd, g, b); r.y = bn_affine(v.y, mean, invstd, g, b);
      r.z = bn_affine(v.z, mean, invstd, g, b); r.w = bn_affine(v.w, mean, invstd, g, b);
      if (RELU) { r.x = r.x < 0.f ? 0.f : r.x; r.y = r.y < 0.f ? 0.f : r.y; r.z = r.z < 0.f ? 0.f : r.z; r.w = r.w < 0.f ? 0.f : r.w; }
      *reinterpret_cast<float4*>(y + off) = r; },
    [&](int64_t off) { float r = bn_affine(x[off], mean, invstd, g, b); if (RELU) r = r < 0.f ? 0.f : r; y[off] = r; });
}

// out = relu(gamma * (x - mean) * invstd + beta + shortcut): the residual join behind a batch norm, one read of x and of
// the shortcut and one write.
template <bool VEC, bool PIECES = false>
__global__ void __launch_bounds__(TPB) k_bn_apply_add_relu(const float* __restrict__ x, const float* __restrict__ sc, float* __restrict__ y, const float* gamma, const float* beta,
                                                           const float* save_mean, const float* save_invstd, int N, int C, int HW, int n_per, ConvPieces P = ConvPieces()) {
  const int c = blockIdx.x, s = blockIdx.y;
  float mean, invstd;
  if (PIECES) bn_stats_from_pieces(P, c, s == 0, mean, invstd); else { mean = save_mean[c]; invstd = save_invstd[c]; }
  const float g = gamma[c], b = beta[c];
  const int n0 = s * n_per, n1 = min(N, n0 + n_per);
  bn_foreach<VEC>(n0, n1, C, c, HW,
    [&](int64_t off) { float4 v = *reinterpret_cast<const float4*>(x + off); float4 a = *reinterpret_cast<const float4*>(sc + off); float4 r;
      r.x = __fadd_rn(bn_affine(v.x, mean, invstd, g, b), a.x); r.y = __fadd_rn(bn_affine(v.y, mean, invstd, g, b), a.y);
      r.z = __fadd_rn(bn_affine(v.z, mean, invstd, g, b), a.z); r.w = __fadd_rn(bn_affine(v.w, mean, invstd, g, b), a.w);
      r.x = r.x < 0.f ? 0.f : r.x; r.y = r.y < 0.f ? 0.f : r.y; r.z = r.z < 0.f ? 0.f : r.z; r.w = r.w < 0.f ? 0.f : r.w;
      *reinterpret_cast<float4*>(y + off) = r; },
    [&](int64_t off) { float r = __fadd_rn(bn_affine(x[off], mean, invstd, g, b), sc[off]); y[off] = r < 0.f ? 0.f : r; });
}

// First pass of the backward of out = relu(bn(x) + shortcut): g = dout where out > 0 else 0; per-slice sums of g and
// of g * xhat; g goes to the shortcut's gradient.  INPLACE: ds accumulates (or is absent), so g is also written over
// dout, where the second pass reads it; otherwise ds = g and the second pass reads ds.
template <bool VEC, bool INPLACE, bool HAS_DS>
__global__ void __launch_bounds__(TPB) k_bn_bwd_stats_add(const float* __restrict__ x, const float* __restrict__ out, float* dout, float* ds,
                                                          const float* save_mean, const float* save_invstd, float* __restrict__ partial, int N, int C, int HW, int n_per) {
  __shared__ float sm[17];
  const int c = blockIdx.x, s = blockIdx.y;
  const int n0 = s * n_per, n1 = min(N, n0 + n_per);
  const float mean = save_mean[c], is = save_invstd[c];
  float s1 = 0.f, s2 = 0.f;
  bn_foreach<VEC>(n0, n1, C, c, HW,
    [&](int64_t off) { float4 v = *reinterpret_cast<const float4*>(x + off); float4 g = *reinterpret_cast<const float4*>(dout + off);
      const float4 m = *reinterpret_cast<const float4*>(out + off);
      g.x = m.x > 0.f ? g.x : 0.f; g.y = m.y > 0.f ? g.y : 0.f; g.z = m.z > 0.f ? g.z : 0.f; g.w = m.w > 0.f ? g.w : 0.f;
      if (INPLACE) {
        *reinterpret_cast<float4*>(dout + off) = g;
        if (HAS_DS) { float4 o = *reinterpret_cast<const float4*>(ds + off); o.x += g.x; o.y += g.y; o.z += g.z; o.w += g.w; *reinterpret_cast<float4*>(ds + off) = o; }
      } else {
        *reinterpret_cast<float4*>(ds + off) = g;
      }
      s1 += (g.x + g.y) + (g.z + g.w);
      s2 += (g.x * ((v.x - mean) * is) + g.y * ((v.y - mean) * is)) + (g.z * ((v.z - mean) * is) + g.w * ((v.w - mean) * is)); },
    [&](int64_t off) { float g = out[off] > 0.f ? dout[off] : 0.f;
      if (INPLACE) { dout[off] = g; if (HAS_DS) ds[off] += g; } else ds[off] = g;
      s1 += g; s2 += g * ((x[off] - mean) * is); });
  s1 = lh_block_sum(s1, sm);
  s2 = lh_block_sum(s2, sm);
  if (threadIdx.x == 0) { float* p = partial + 3 * ((int64_t)c * gridDim.y + s); p[0] = s1; p[1] = s2; }
}

static bool get_partial() {
  if (g_partial_ptr) return true;
  if (hipGetSymbolAddress((void**)&g_partial_ptr, HIP_SYMBOL(g_bn_partial)) != hipSuccess) { LH_FAIL("bn scratch symbol lookup failed"); return false; }
  return true;
}
}  // namespace

namespace lh {
void bn_finalize_conv_partials(const float* partial, int C, int ncols, int col1, int g_main, int slots_main, int g_rem,
                               float* save_mean, float* save_invstd, float* run_mean, float* run_var, float eps, float factor) {
  const int slots_rem = col1 < ncols ? (int)cdiv(ncols - col1, g_rem) : 0;
  hipLaunchKernelGGL(k_bn_finalize_conv, dim3(C), dim3(TPB), 0, g_stream, partial, C, ncols, col1, g_main, slots_main, g_rem, slots_main + slots_rem,
                     save_mean, save_invstd, run_mean, run_var, eps, factor);
}
void bn_apply_from_pieces(const float* y, const ConvPieces& pieces, const float* gamma, const float* beta, const float* shortcut, float* out, int relu,
                          int N, int C, int HW) {
  ProfScope prof_(CAT_BN_FWD);
  work_add(CAT_BN_FWD, (shortcut ? 12.0 : 8.0) * N * C * (double)HW);      // y (and the shortcut) read, out written
  Plan p = make_plan(N, C, HW, (((uintptr_t)y | (uintptr_t)out | (uintptr_t)shortcut) & 15) == 0);
  dim3 grid(C, p.slices);
  const float* none = nullptr;
  if (shortcut) {
    if (p.vec4) hipLaunchKernelGGL((k_bn_apply_add_relu<true, true>), grid, dim3(TPB), 0, g_stream, y, shortcut, out, gamma, beta, none, none, N, C, HW, p.n_per, pieces);
    else hipLaunchKernelGGL((k_bn_apply_add_relu<false, true>), grid, dim3(TPB), 0, g_stream, y, shortcut, out, gamma, beta, none, none, N, C, HW, p.n_per, pieces);
  } else {
#define GO(V, R) hipLaunchKernelGGL((k_bn_apply<V, R, true>), grid, dim3(TPB), 0, g_stream, y, out, gamma, beta, none, none, N, C, HW, p.n_per, pieces)
    if (p.vec4) { if (relu) GO(true, true); else GO(true, false); }
    else { if (relu) GO(false, true); else GO(false, false); }
#undef GO
  }
}
}  // namespace lh

// What a batch-norm call reads and writes, stated to the deferred-work bookkeeping (lh_defer.hip); launches whatever is parked.
static void bn_fwd_declare(const float* x, const float* gamma, const float* beta, float* run_mean, float* run_var, float* y,
                           float* save_mean, float* save_invstd, int N, int C, int HW) {
  if (!lazy::g_busy || lazy::g_replay) return;
  const int64_t n = (int64_t)N * C * HW;
  lazy::flush_parked();
  lazy::rd_f(x, n); lazy::rd_f(gamma, C); lazy::rd_f(beta, C); lazy::rw_f(run_mean, C); lazy::rw_f(run_var, C);
  lazy::out_f(y, n, y == x);
  lazy::wr_f(save_mean, C); lazy::wr_f(save_invstd, C);
}
// returns the beta to run with: 1 on a gradient buffer nobody has touched since lh_malloc becomes 0
static float bn_bwd_declare(const float* x, const float* y, const float* dy, const float* gamma, const float* bias, const float* save_mean, const float* save_invstd,
                            float* dx, float beta_dx, float* dgamma, float* dbeta, int N, int C, int HW) {
  if (!lazy::g_busy || lazy::g_replay) return beta_dx;
  const int64_t n = (int64_t)N * C * HW;
  lazy::flush_parked();
  lazy::rd_f(x, n); lazy::rd_f(y, n); lazy::rd_f(dy, n); lazy::rd_f(gamma, C); lazy::rd_f(bias, C); lazy::rd_f(save_mean, C); lazy::rd_f(save_invstd, C);
  if (dx && (beta_dx == 0.f || beta_dx == 1.f)) beta_dx = lazy::beta_f(dx, n, beta_dx);
  lazy::rw_f(dgamma, C); lazy::rw_f(dbeta, C);
  return beta_dx;
}

extern "C" {

void lh_bn_stats(const float* x, float* save_mean, float* save_invstd, float* run_mean, float* run_var, int N, int C, int HW, float eps, float factor) {
  LH_REQUIRE(N > 0 && C > 0 && HW > 0, "lh_bn_stats: empty shape [%d,%d,%d]", N, C, HW);
  LZ_ENTER(); lazy::rd_f(x, (int64_t)N * C * HW); lazy::wr_f(save_mean, C); lazy::wr_f(save_invstd, C); lazy::rw_f(run_mean, C); lazy::rw_f(run_var, C);
  ProfScope prof_(CAT_BN_FWD);
  LH_REQUIRE(C <= MAX_PARTIALS, "lh_bn_stats: %d channels exceed the scratch (%d)", C, MAX_PARTIALS);
  if (!get_partial()) return;
  work_add(CAT_BN_FWD, 4.0 * N * C * (double)HW);
  Plan p = make_plan(N, C, HW, ((uintptr_t)x & 15) == 0);
  dim3 grid(C, p.slices);
  if (p.vec4) hipLaunchKernelGGL((k_bn_stats<true>), grid, dim3(TPB), 0, g_stream, x, g_partial_ptr, N, C, HW, p.n_per);
  else hipLaunchKernelGGL((k_bn_stats<false>), grid, dim3(TPB), 0, g_stream, x, g_partial_ptr, N, C, HW, p.n_per);
  hipLaunchKernelGGL(k_bn_finalize, dim3((unsigned)cdiv(C, TPB)), dim3(TPB), 0, g_stream, (const float*)g_partial_ptr, C, p.slices, save_mean, save_invstd,
                     run_mean, run_var, eps, factor);
  LH_CHECK_LAUNCH();
}

void lh_bn_apply(const float* x, const float* gamma, const float* beta, const float* save_mean, const float* save_invstd, float* y,
                 int N, int C, int HW, int relu) {
  LH_REQUIRE(N > 0 && C > 0 && HW > 0, "lh_bn_apply: empty shape [%d,%d,%d]", N, C, HW);
  LZ_ENTER(); lazy::rd_f(x, (int64_t)N * C * HW); lazy::rd_f(gamma, C); lazy::rd_f(beta, C); lazy::rd_f(save_mean, C); lazy::rd_f(save_invstd, C);
  lazy::out_f(y, (int64_t)N * C * HW, y == x);
  ProfScope prof_(CAT_BN_FWD);
  work_add(CAT_BN_FWD, 8.0 * N * C * (double)HW);
  Plan p = make_plan(N, C, HW, (((uintptr_t)x | (uintptr_t)y) & 15) == 0);
  dim3 grid(C, p.slices);
#define GO(V, R) hipLaunchKernelGGL((k_bn_apply<V, R>), grid, dim3(TPB), 0, g_stream, x, y, gamma, beta, save_mean, save_invstd, N, C, HW, p.n_per)
  if (p.vec4) { if (relu) GO(true, true); else GO(true, false); }
  else { if (relu) GO(false, true); else GO(false, false); }
#undef GO
  LH_CHECK_LAUNCH();
}

void lh_bn_infer(const float* x, const float* gamma, const float* beta, const float* run_mean, const float* run_var,
                 float* y, int N, int C, int HW, float eps) {
  int64_t n = (int64_t)N * C * HW;
  if (n <= 0) return;
  LZ_ENTER(); lazy::rd_f(x, n); lazy::rd_f(gamma, C); lazy::rd_f(beta, C); lazy::rd_f(run_mean, C); lazy::rd_f(run_var, C);
  lazy::out_f(y, n, y == x);
  ProfScope prof_(CAT_BN_FWD);
  work_add(CAT_BN_FWD, 8.0 * (double)n);
  hipLaunchKernelGGL(k_bn_infer, dim3(stream_grid(n, TPB * 4)), dim3(TPB), 0, g_stream, x, y, gamma, beta, run_mean, run_var, C, HW, n, eps);
  LH_CHECK_LAUNCH();
}

static void bn_train_fwd_impl(bool relu, const float* x, const float* gamma, const float* beta, float* run_mean, float* run_var, float* y,
                              float* save_mean, float* save_invstd, int N, int C, int HW, float eps, float factor) {
  LH_REQUIRE(N > 0 && C > 0 && HW > 0, "lh_bn_train_fwd: empty shape [%d,%d,%d]", N, C, HW);
  LH_REQUIRE(C <= MAX_PARTIALS, "lh_bn_train_fwd: %d channels exceed the scratch (%d)", C, MAX_PARTIALS);
  if (!get_partial()) return;
  if (HW == 1 && !relu && C >= 32) {          // rows of channels: the column kernels
    work_add(CAT_BN_FWD, 12.0 * N * (double)C);
    const Plan1 p1 = make_plan1(N, C);
    dim3 g1((unsigned)cdiv(C, C1), p1.slices);
    hipLaunchKernelGGL(k_bn1d_stats, g1, dim3(TPB), 0, g_stream, x, g_partial_ptr, N, C, p1.rows_per);
    hipLaunchKernelGGL(k_bn1d_fwd_apply, g1, dim3(TPB), 0, g_stream, x, y, (const float*)g_partial_ptr, gamma, beta, run_mean, run_var,
                       save_mean, save_invstd, N, C, p1.rows_per, eps, factor);
    LH_CHECK_LAUNCH();
    return;
  }
  Plan p = make_plan(N, C, HW, (((uintptr_t)x | (uintptr_t)y) & 15) == 0);
  work_add(CAT_BN_FWD, ((C >= 128 && small_fits(N, HW, p.vec4)) ? 8.0 : 12.0) * N * C * (double)HW);    // x read once (twice: statistics pass, then the apply pass), y written
  if (C >= 128 && small_fits(N, HW, p.vec4)) {          // a channel per block, one launch (given enough channels to occupy the chip)
#define SMALL(V, R) hipLaunchKernelGGL((k_bn_small_fwd<V, R>), dim3(C), dim3(TPB), 0, g_stream, x, y, gamma, beta, run_mean, run_var, save_mean, save_invstd, N, C, HW, eps, factor)
    if (p.vec4) { if (relu) SMALL(true, true); else SMALL(true, false); }
    else { if (relu) SMALL(false, true); else SMALL(false, false); }
#undef SMALL
    LH_CHECK_LAUNCH();
    return;
  }
  dim3 grid(C, p.slices);
#define FWD(V, R) hipLaunchKernelGGL((k_bn_fwd_apply<V, R>), grid, dim3(TPB), 0, g_stream, x, y, (const float*)g_partial_ptr, gamma, beta, run_mean, run_var, \
                                     save_mean, save_invstd, N, C, HW, p.n_per, eps, factor)
  if (p.vec4) {
    hipLaunchKernelGGL((k_bn_stats<true>), grid, dim3(TPB), 0, g_stream, x, g_partial_ptr, N, C, HW, p.n_per);
    if (relu) FWD(true, true); else FWD(true, false);
  } else {
    hipLaunchKernelGGL((k_bn_stats<false>), grid, dim3(TPB), 0, g_stream, x, g_partial_ptr, N, C, HW, p.n_per);
    if (relu) FWD(false, true); else FWD(false, false);
  }
#undef FWD
  LH_CHECK_LAUNCH();
}

static void bn_bwd_impl(const float* x, const float* y_relu, const float* dy, const float* gamma, const float* bias, int relu,
                        const float* save_mean, const float* save_invstd,
                        float* dx, float beta_dx, float* dgamma, float* dbeta, int N, int C, int HW) {
  LH_REQUIRE(N > 0 && C > 0 && HW > 0, "lh_bn_bwd: empty shape [%d,%d,%d]", N, C, HW);
  LH_REQUIRE(C <= MAX_PARTIALS, "lh_bn_bwd: %d channels exceed the scratch (%d)", C, MAX_PARTIALS);
  LH_REQUIRE(beta_dx == 0.0f || beta_dx == 1.0f, "lh_bn_bwd: beta must be 0 or 1");
  if (!get_partial()) return;
  if (HW == 1 && relu == 0 && C >= 32) {
    work_add(CAT_BN_BWD, (20.0 + (beta_dx != 0.0f ? 4.0 : 0.0)) * N * (double)C);
    const Plan1 p1 = make_plan1(N, C);
    dim3 g1((unsigned)cdiv(C, C1), p1.slices);
    hipLaunchKernelGGL(k_bn1d_bwd_stats, g1, dim3(TPB), 0, g_stream, x, dy, save_mean, save_invstd, g_partial_ptr, N, C, p1.rows_per);
    if (beta_dx != 0.0f) hipLaunchKernelGGL((k_bn1d_bwd_apply<true>), g1, dim3(TPB), 0, g_stream, x, dy, (const float*)g_partial_ptr, gamma, save_mean, save_invstd, dx, dgamma, dbeta, N, C, p1.rows_per);
    else hipLaunchKernelGGL((k_bn1d_bwd_apply<false>), g1, dim3(TPB), 0, g_stream, x, dy, (const float*)g_partial_ptr, gamma, save_mean, save_invstd, dx, dgamma, dbeta, N, C, p1.rows_per);
    LH_CHECK_LAUNCH();
    return;
  }
  Plan p = make_plan(N, C, HW, (((uintptr_t)x | (uintptr_t)dy | (uintptr_t)dx | (uintptr_t)y_relu) & 15) == 0);
  const bool acc = beta_dx != 0.0f;
  {
    // x and dy (and y, when the relu mask is read from it) read once, or twice with the statistics pass; dx written, and read first when it accumulates
    const bool one = C >= 128 && small_fits(N, HW, p.vec4);
    const double per = (one ? 8.0 : 16.0) + (relu == 1 ? (one ? 4.0 : 8.0) : 0.0) + (dx ? 4.0 + (acc ? 4.0 : 0.0) : 0.0);
    work_add(CAT_BN_BWD, per * N * C * (double)HW);
  }
  if (C >= 128 && small_fits(N, HW, p.vec4)) {          // a channel per block, one launch
#define SMALL(V, A, R) hipLaunchKernelGGL((k_bn_small_bwd<V, A, R>), dim3(C), dim3(TPB), 0, g_stream, x, y_relu, dy, gamma, bias, save_mean, save_invstd, dx, dgamma, dbeta, N, C, HW)
#define SMALL_R(V, A) do { if (relu == 2) SMALL(V, A, 2); else if (relu == 1) SMALL(V, A, 1); else SMALL(V, A, 0); } while (0)
    if (p.vec4) { if (acc) SMALL_R(true, true); else SMALL_R(true, false); }
    else { if (acc) SMALL_R(false, true); else SMALL_R(false, false); }
#undef SMALL_R
#undef SMALL
    LH_CHECK_LAUNCH();
    return;
  }
  dim3 grid(C, p.slices);
  const int from_end = 8.0 * N * C * (double)HW > 192e6;      // x and dy together beyond most of the 256 MB last-level cache
#define STATS(V, R) hipLaunchKernelGGL((k_bn_bwd_stats<V, R>), grid, dim3(TPB), 0, g_stream, x, y_relu, dy, save_mean, save_invstd, gamma, bias, g_partial_ptr, N, C, HW, p.n_per)
#define APPLY(V, A, R) hipLaunchKernelGGL((k_bn_bwd_apply<V, A, R>), grid, dim3(TPB), 0, g_stream, x, y_relu, dy, (const float*)g_partial_ptr, gamma, bias, save_mean, save_invstd, dx, dgamma, dbeta, N, C, HW, p.n_per, from_end)
#define BOTH(V, R) do { STATS(V, R); if (acc) APPLY(V, true, R); else APPLY(V, false, R); } while (0)
  if (p.vec4) { if (relu == 2) BOTH(true, 2); else if (relu == 1) BOTH(true, 1); else BOTH(true, 0); }
  else { if (relu == 2) BOTH(false, 2); else if (relu == 1) BOTH(false, 1); else BOTH(false, 0); }
#undef BOTH
#undef STATS
#undef APPLY
  LH_CHECK_LAUNCH();
}

void lh_bn_train_fwd(const float* x, const float* gamma, const float* beta, float* run_mean, float* run_var, float* y,
                     float* save_mean, float* save_invstd, int N, int C, int HW, float eps, float factor) {
  LZ_SCOPE();
  // waits for the call behind it: relu in place or the residual join fuse with it; right behind a parked convolution the
  // statistics come from that convolution's epilogue
  if (lazy::park_bn_train_fwd(x, gamma, beta, run_mean, run_var, y, save_mean, save_invstd, N, C, HW, eps, factor)) return;
  bn_fwd_declare(x, gamma, beta, run_mean, run_var, y, save_mean, save_invstd, N, C, HW);
  ProfScope prof_(CAT_BN_FWD);
  bn_train_fwd_impl(false, x, gamma, beta, run_mean, run_var, y, save_mean, save_invstd, N, C, HW, eps, factor);
}
void lh_bn_train_fwd_relu(const float* x, const float* gamma, const float* beta, float* run_mean, float* run_var, float* y,
                          float* save_mean, float* save_invstd, int N, int C, int HW, float eps, float factor) {
  LZ_SCOPE();
  bn_fwd_declare(x, gamma, beta, run_mean, run_var, y, save_mean, save_invstd, N, C, HW);
  ProfScope prof_(CAT_BN_FWD);
  bn_train_fwd_impl(true, x, gamma, beta, run_mean, run_var, y, save_mean, save_invstd, N, C, HW, eps, factor);
}
void lh_bn_bwd(const float* x, const float* dy, const float* gamma, const float* save_mean, const float* save_invstd,
               float* dx, float beta_dx, float* dgamma, float* dbeta, int N, int C, int HW) {
  LZ_SCOPE();
  // right behind a parked relu_grad (and the gradient of a `+`): one fused backward instead of two or three passes
  if (lazy::g_busy && !lazy::g_replay && lazy::take_bn_bwd(x, dy, gamma, save_mean, save_invstd, dx, beta_dx, dgamma, dbeta, N, C, HW)) return;
  beta_dx = bn_bwd_declare(x, nullptr, dy, gamma, nullptr, save_mean, save_invstd, dx, beta_dx, dgamma, dbeta, N, C, HW);
  ProfScope prof_(CAT_BN_BWD);
  bn_bwd_impl(x, nullptr, dy, gamma, nullptr, 0, save_mean, save_invstd, dx, beta_dx, dgamma, dbeta, N, C, HW);
}
void lh_bn_bwd_relu(const float* x, const float* y, const float* dy, const float* gamma, const float* bias, const float* save_mean, const float* save_invstd,
                    float* dx, float beta_dx, float* dgamma, float* dbeta, int N, int C, int HW) {
  LH_REQUIRE(y != nullptr || bias != nullptr, "lh_bn_bwd_relu: y or the layer's bias is required");
  LZ_SCOPE();
  beta_dx = bn_bwd_declare(x, bias ? nullptr : y, dy, gamma, bias, save_mean, save_invstd, dx, beta_dx, dgamma, dbeta, N, C, HW);
  ProfScope prof_(CAT_BN_BWD);
  bn_bwd_impl(x, bias ? nullptr : y, dy, gamma, bias, bias ? 2 : 1, save_mean, save_invstd, dx, beta_dx, dgamma, dbeta, N, C, HW);
}

void lh_bn_apply_add_relu(const float* x, const float* gamma, const float* beta, const float* save_mean, const float* save_invstd,
                          const float* shortcut, float* out, int N, int C, int HW) {
  LH_REQUIRE(N > 0 && C > 0 && HW > 0, "lh_bn_apply_add_relu: empty shape [%d,%d,%d]", N, C, HW);
  LH_REQUIRE(x && shortcut && out && gamma && beta && save_mean && save_invstd, "lh_bn_apply_add_relu: null operand");
  LZ_ENTER(); lazy::rd_f(x, (int64_t)N * C * HW); lazy::rd_f(shortcut, (int64_t)N * C * HW); lazy::rd_f(gamma, C); lazy::rd_f(beta, C); lazy::rd_f(save_mean, C); lazy::rd_f(save_invstd, C);
  lazy::out_f(out, (int64_t)N * C * HW, out == x || out == shortcut);
  ProfScope prof_(CAT_BN_FWD);
  work_add(CAT_BN_FWD, 12.0 * N * C * (double)HW);
  Plan p = make_plan(N, C, HW, (((uintptr_t)x | (uintptr_t)out | (uintptr_t)shortcut) & 15) == 0);
  dim3 grid(C, p.slices);
  if (p.vec4) hipLaunchKernelGGL((k_bn_apply_add_relu<true>), grid, dim3(TPB), 0, g_stream, x, shortcut, out, gamma, beta, save_mean, save_invstd, N, C, HW, p.n_per);
  else hipLaunchKernelGGL((k_bn_apply_add_relu<false>), grid, dim3(TPB), 0, g_stream, x, shortcut, out, gamma, beta, save_mean, save_invstd, N, C, HW, p.n_per);
  LH_CHECK_LAUNCH();
}

void lh_bn_bwd_add_relu(const float* x, const float* out, float* dout, const float* gamma, const float* save_mean, const float* save_invstd,
                        float* dx, float beta_dx, float* ds, float beta_ds, float* dgamma, float* dbeta, int N, int C, int HW) {
  LH_REQUIRE(N > 0 && C > 0 && HW > 0, "lh_bn_bwd_add_relu: empty shape [%d,%d,%d]", N, C, HW);
  LZ_SCOPE();
  if (lazy::g_busy && !lazy::g_replay) {
    const int64_t n = (int64_t)N * C * HW;
    lazy::flush_parked();
    lazy::rd_f(x, n); lazy::rd_f(out, n); lazy::rw_f(dout, n); lazy::rd_f(gamma, C); lazy::rd_f(save_mean, C); lazy::rd_f(save_invstd, C);
    if (dx && (beta_dx == 0.f || beta_dx == 1.f)) beta_dx = lazy::beta_f(dx, n, beta_dx);
    if (ds && (beta_ds == 0.f || beta_ds == 1.f)) beta_ds = lazy::beta_f(ds, n, beta_ds);
    lazy::rw_f(dgamma, C); lazy::rw_f(dbeta, C);
  }
  ProfScope prof_(CAT_BN_BWD);
  LH_REQUIRE(C <= MAX_PARTIALS, "lh_bn_bwd_add_relu: %d channels exceed the scratch (%d)", C, MAX_PARTIALS);
  LH_REQUIRE((beta_dx == 0.0f || beta_dx == 1.0f) && (beta_ds == 0.0f || beta_ds == 1.0f), "lh_bn_bwd_add_relu: beta must be 0 or 1");
  LH_REQUIRE(x && out && dout && gamma && save_mean && save_invstd, "lh_bn_bwd_add_relu: null operand");
  LH_REQUIRE(ds != dout && dx != dout, "lh_bn_bwd_add_relu: dout may not alias a gradient output");
  LH_REQUIRE(dx == nullptr || dx != ds, "lh_bn_bwd_add_relu: dx and ds are the same buffer (a batch norm whose input is also the shortcut): the first pass would add into what the second overwrites; run lh_add_relu_grad and lh_bn_bwd instead");
  if (!get_partial()) return;
  Plan p = make_plan(N, C, HW, (((uintptr_t)x | (uintptr_t)out | (uintptr_t)dout | (uintptr_t)dx | (uintptr_t)ds) & 15) == 0);
  {
    // one launch: x, out, dout read once; two passes: pass 1 reads x, out, dout and writes the masked gradient (to the shortcut's
    // buffer, or over dout), pass 2 reads x and the masked gradient; dx and ds written, each read first when it accumulates
    const bool one = C >= 128 && small_fits(N, HW, p.vec4);
    const double per = one ? 12.0 + (ds ? 4.0 + (beta_ds != 0.0f ? 4.0 : 0.0) : 0.0) + (dx ? 4.0 + (beta_dx != 0.0f ? 4.0 : 0.0) : 0.0)
                           : 24.0 + (ds && beta_ds != 0.0f ? 8.0 : 0.0) + (dx ? 4.0 + (beta_dx != 0.0f ? 4.0 : 0.0) : 0.0);
    work_add(CAT_BN_BWD, per * N * C * (double)HW);
  }
  if (C >= 128 && small_fits(N, HW, p.vec4)) {          // a channel per block, one launch; dout is left as it is
    const int dsm = ds == nullptr ? 0 : (beta_ds != 0.0f ? 2 : 1);
#define SMALL(V, A, D) hipLaunchKernelGGL((k_bn_small_bwd_join<V, A, D>), dim3(C), dim3(TPB), 0, g_stream, x, out, (const float*)dout, ds, gamma, save_mean, save_invstd, dx, dgamma, dbeta, N, C, HW)
#define SMALL_D(V, A) do { if (dsm == 2) SMALL(V, A, 2); else if (dsm == 1) SMALL(V, A, 1); else SMALL(V, A, 0); } while (0)
    if (p.vec4) { if (beta_dx != 0.0f) SMALL_D(true, true); else SMALL_D(true, false); }
    else { if (beta_dx != 0.0f) SMALL_D(false, true); else SMALL_D(false, false); }
#undef SMALL_D
#undef SMALL
    LH_CHECK_LAUNCH();
    return;
  }
  dim3 grid(C, p.slices);
  const bool inplace = ds == nullptr || beta_ds != 0.0f, acc = beta_dx != 0.0f;
  const float* g = inplace ? dout : ds;            // where the masked gradient lies after the first pass
  const int from_end = 8.0 * N * C * (double)HW > 192e6;
#define STATS(V, I, H) hipLaunchKernelGGL((k_bn_bwd_stats_add<V, I, H>), grid, dim3(TPB), 0, g_stream, x, out, dout, ds, save_mean, save_invstd, g_partial_ptr, N, C, HW, p.n_per)
#define APPLY(V, A) hipLaunchKernelGGL((k_bn_bwd_apply<V, A, 0>), grid, dim3(TPB), 0, g_stream, x, (const float*)nullptr, g, (const float*)g_partial_ptr, gamma, (const float*)nullptr, save_mean, save_invstd, dx, dgamma, dbeta, N, C, HW, p.n_per, from_end)
  if (p.vec4) {
    if (!inplace) STATS(true, false, true); else if (ds) STATS(true, true, true); else STATS(true, true, false);
    if (acc) APPLY(true, true); else APPLY(true, false);
  } else {
    if (!inplace) STATS(false, false, true); else if (ds) STATS(false, true, true); else STATS(false, true, false);
    if (acc) APPLY(false, true); else APPLY(false, false);
  }
#undef STATS
#undef APPLY
  LH_CHECK_LAUNCH();
}

}  // extern "C"
