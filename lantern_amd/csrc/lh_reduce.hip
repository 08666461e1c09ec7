// Reductions and the loss head: full sum / mean, sum over one axis, softmax / logSoftmax
// over the middle axis of an [outer, c, inner] view, nllLoss.  Wavefront-shuffle (64 lanes)
// reductions with one LDS hop across the waves of a block.
#include "lh_common.h"
using namespace lh;

namespace {
constexpr int TPB = 256;

// ---- full reduction: two stages through a fixed scratch of partials --------------------
constexpr int SUM_BLOCKS = 1024;
__device__ float g_sum_partials[SUM_BLOCKS];

__global__ void __launch_bounds__(TPB) k_sum_stage1(const float* __restrict__ x, int64_t n, float* partials) {
  __shared__ float sm[17];
  float acc = 0.f;
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n; i += st) acc += x[i];
  acc = lh_block_sum(acc, sm);
  if (threadIdx.x == 0) partials[blockIdx.x] = acc;
}
__global__ void __launch_bounds__(TPB) k_sum_stage2(const float* partials, int np, float* out, float scale) {
  __shared__ float sm[17];
  float acc = 0.f;
  for (int i = threadIdx.x; i < np; i += TPB) acc += partials[i];
  acc = lh_block_sum(acc, sm);
  if (threadIdx.x == 0) out[0] = acc * scale;
}
__global__ void __launch_bounds__(TPB) k_sum_small(const float* x, int64_t n, float* out, float scale) {
  __shared__ float sm[17];
  float acc = 0.f;
  for (int64_t i = threadIdx.x; i < n; i += TPB) acc += x[i];
  acc = lh_block_sum(acc, sm);
  if (threadIdx.x == 0) out[0] = acc * scale;
}
static void sum_impl(const float* x, float* out, int64_t n, float scale) {
  if (n <= 16384) {
    hipLaunchKernelGGL(k_sum_small, dim3(1), dim3(TPB), 0, g_stream, x, n, out, scale);
    return;
  }
  float* partials = nullptr;
  if (hipGetSymbolAddress((void**)&partials, HIP_SYMBOL(g_sum_partials)) != hipSuccess) { LH_FAIL("partials symbol lookup failed"); return; }
  int grid = (int)cdiv(n, TPB * 16); if (grid > SUM_BLOCKS) grid = SUM_BLOCKS;
  hipLaunchKernelGGL(k_sum_stage1, dim3(grid), dim3(TPB), 0, g_stream, x, n, partials);
  hipLaunchKernelGGL(k_sum_stage2, dim3(1), dim3(TPB), 0, g_stream, (const float*)partials, grid, out, scale);
}

__global__ void __launch_bounds__(TPB) k_add_scalar_from(float* dx, const float* dy1, float scale, int64_t n) {
  float v = dy1[0] * scale;
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n; i += st) dx[i] += v;
}

// ---- sum over the middle axis of [outer, dim, inner] -----------------------------------
// inner > 1: thread per (outer, inner) output, coalesced along inner.  inner == 1: wave per row.
__global__ void __launch_bounds__(TPB) k_sum_dim_inner(const float* __restrict__ x, float* y, int outer, int dim, int inner) {
  int64_t n = (int64_t)outer * inner;
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n; i += st) {
    int64_t h = i / inner, l = i - h * inner;
    const float* p = x + h * dim * inner + l;
    float acc = 0.f;
    for (int s = 0; s < dim; s++) acc += p[(int64_t)s * inner];
    y[i] = acc;
  }
}
// Few outputs, long reduction: a block sums a slice of `dim` for 64 consecutive inner positions (4 threads per
// position, combined in LDS) and adds its partial sum into y, which the host has zeroed.
__global__ void __launch_bounds__(TPB) k_sum_dim_split(const float* __restrict__ x, float* y, int dim, int inner, int per_slice) {
  __shared__ float sm[4][64];
  const int l = blockIdx.x * 64 + (threadIdx.x & 63), q = threadIdx.x >> 6;
  const int s0 = blockIdx.y * per_slice, s1 = min(dim, s0 + per_slice);
  const int64_t h = blockIdx.z;
  float acc = 0.f;
  if (l < inner) {
    const float* p = x + h * dim * inner + l;
    for (int s = s0 + q; s < s1; s += 4) acc += p[(int64_t)s * inner];
  }
  sm[q][threadIdx.x & 63] = acc;
  __syncthreads();
  if (q == 0 && l < inner) atomicAdd(y + h * inner + l, (sm[0][threadIdx.x] + sm[1][threadIdx.x]) + (sm[2][threadIdx.x] + sm[3][threadIdx.x]));
}
__global__ void __launch_bounds__(TPB) k_sum_rows(const float* __restrict__ x, float* y, int rows, int cols) {
  const int lane = threadIdx.x & 63;
  int64_t w = ((int64_t)blockIdx.x * TPB + threadIdx.x) >> 6, nw = ((int64_t)gridDim.x * TPB) >> 6;
  for (; w < rows; w += nw) {
    float acc = 0.f;
    for (int j = lane; j < cols; j += 64) acc += x[w * cols + j];
    acc = lh_wave_sum(acc);
    if (lane == 0) y[w] = acc;
  }
}
__global__ void __launch_bounds__(TPB) k_sum_dim_grad(float* dx, const float* __restrict__ dy, int64_t n, int dim, int inner) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n; i += st) {
    int64_t l = i % inner, h = i / ((int64_t)dim * inner);
    dx[i] += dy[h * inner + l];
  }
}

// ---- softmax / logSoftmax --------------------------------------------------------------
// inner == 1: one block per row when c is large, one wave per row when c <= 1024.
template <bool LOG>
__global__ void __launch_bounds__(TPB) k_softmax_rows_wave(const float* __restrict__ x, float* __restrict__ y, int rows, int c) {
  const int lane = threadIdx.x & 63;
  int64_t w = ((int64_t)blockIdx.x * TPB + threadIdx.x) >> 6, nw = ((int64_t)gridDim.x * TPB) >> 6;
  for (; w < rows; w += nw) {
    const float* xp = x + w * c; float* yp = y + w * c;
    float mx = -3.402823466e+38f;
    for (int j = lane; j < c; j += 64) mx = fmaxf(mx, xp[j]);
    mx = lh_wave_max(mx); mx = __shfl(mx, 0, 64);
    float sum = 0.f;
    for (int j = lane; j < c; j += 64) sum += expf(xp[j] - mx);
    sum = lh_wave_sum(sum); sum = __shfl(sum, 0, 64);
    if (LOG) { float ls = mx + logf(sum); for (int j = lane; j < c; j += 64) yp[j] = xp[j] - ls; }
    else { for (int j = lane; j < c; j += 64) yp[j] = expf(xp[j] - mx) / sum; }
  }
}
template <bool LOG>
__global__ void __launch_bounds__(TPB) k_softmax_rows_block(const float* __restrict__ x, float* __restrict__ y, int c) {
  __shared__ float sm[17];
  const float* xp = x + (int64_t)blockIdx.x * c; float* yp = y + (int64_t)blockIdx.x * c;
  float mx = -3.402823466e+38f;
  for (int j = threadIdx.x; j < c; j += TPB) mx = fmaxf(mx, xp[j]);
  mx = lh_block_max(mx, sm);
  float sum = 0.f;
  for (int j = threadIdx.x; j < c; j += TPB) sum += expf(xp[j] - mx);
  sum = lh_block_sum(sum, sm);
  if (LOG) { float ls = mx + logf(sum); for (int j = threadIdx.x; j < c; j += TPB) yp[j] = xp[j] - ls; }
  else { for (int j = threadIdx.x; j < c; j += TPB) yp[j] = expf(xp[j] - mx) / sum; }
}
// inner > 1: thread per (outer, inner) pair, strided walk over c (coalesced along inner).
template <bool LOG>
__global__ void __launch_bounds__(TPB) k_softmax_inner(const float* __restrict__ x, float* __restrict__ y, int outer, int c, int inner) {
  int64_t n = (int64_t)outer * inner;
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n; i += st) {
    int64_t o = i / inner, l = i - o * inner, base = o * c * inner + l;
    float mx = -3.402823466e+38f;
    for (int j = 0; j < c; j++) mx = fmaxf(mx, x[base + (int64_t)j * inner]);
    float sum = 0.f;
    for (int j = 0; j < c; j++) sum += expf(x[base + (int64_t)j * inner] - mx);
    if (LOG) { float ls = mx + logf(sum); for (int j = 0; j < c; j++) y[base + (int64_t)j * inner] = x[base + (int64_t)j * inner] - ls; }
    else { for (int j = 0; j < c; j++) y[base + (int64_t)j * inner] = expf(x[base + (int64_t)j * inner] - mx) / sum; }
  }
}
// gradients: log: dx += dy - exp(y)*sum(dy);  plain: dx += y*(dy - sum(dy*y))
template <bool LOG>
__global__ void __launch_bounds__(TPB) k_softmax_grad_wave(const float* __restrict__ y, const float* __restrict__ dy, float* dx, int64_t groups, int c, int inner) {
  const int lane = threadIdx.x & 63;
  int64_t w = ((int64_t)blockIdx.x * TPB + threadIdx.x) >> 6, nw = ((int64_t)gridDim.x * TPB) >> 6;
  for (; w < groups; w += nw) {
    int64_t o = w / inner, l = w - o * inner, base = o * c * inner + l;
    float acc = 0.f;
    for (int j = lane; j < c; j += 64) { int64_t i = base + (int64_t)j * inner; acc += LOG ? dy[i] : dy[i] * y[i]; }
    acc = lh_wave_sum(acc); acc = __shfl(acc, 0, 64);
    for (int j = lane; j < c; j += 64) {
      int64_t i = base + (int64_t)j * inner;
      dx[i] += LOG ? dy[i] - expf(y[i]) * acc : y[i] * (dy[i] - acc);
    }
  }
}

__global__ void k_nll(const float* x, const int* target, float* y, int batch, int stride) {
  int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b < batch) y[b] = -1.0f * x[(int64_t)b * stride + target[b]];
}
__global__ void k_nll_grad(float* dx, const int* target, const float* dy, int batch, int stride) {
  int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b < batch) dx[(int64_t)b * stride + target[b]] += -1.0f * dy[b];
}
}  // namespace

extern "C" {

void lh_sum_all(const float* x, float* out, int64_t n) { LZ_ENTER(); lazy::rd_f(x, n); lazy::wr_f(out, 1); ProfScope prof_(CAT_REDUCE); sum_impl(x, out, n, 1.0f); if (!failed()) LH_CHECK_LAUNCH(); }
void lh_mean_all(const float* x, float* out, int64_t n) { LZ_ENTER(); lazy::rd_f(x, n); lazy::wr_f(out, 1); ProfScope prof_(CAT_REDUCE);
  LH_REQUIRE(n > 0, "lh_mean_all of an empty tensor");
  sum_impl(x, out, n, 1.0f / (float)n);
  if (!failed()) LH_CHECK_LAUNCH();
}
void lh_add_scalar_from(float* dx, const float* dy1, float scale, int64_t n) { LZ_ENTER(); lazy::rd_f(dy1, 1); lazy::rw_f(dx, n); ProfScope prof_(CAT_REDUCE);
  if (n <= 0) return;
  hipLaunchKernelGGL(k_add_scalar_from, dim3(stream_grid(n, TPB * 4)), dim3(TPB), 0, g_stream, dx, dy1, scale, n);
  LH_CHECK_LAUNCH();
}
void lh_sum_dim(const float* x, float* y, int outer, int dim, int inner) { LZ_ENTER(); lazy::rd_f(x, (int64_t)outer * dim * inner); lazy::wr_f(y, (int64_t)outer * inner); ProfScope prof_(CAT_REDUCE);
  if ((int64_t)outer * inner <= 0) return;
  if (inner == 1) hipLaunchKernelGGL(k_sum_rows, dim3(stream_grid((int64_t)outer * 64, TPB)), dim3(TPB), 0, g_stream, x, y, outer, dim);
  else if (!g_deterministic && (int64_t)outer * inner < 64 * (int64_t)g_num_cu && dim >= 512 && outer <= 65535) {      // slices add atomically
    const int64_t base = (int64_t)outer * cdiv(inner, 64);
    int slices = (int)cdiv(4 * (int64_t)g_num_cu, base);
    if (slices > dim / 64) slices = dim / 64;
    if (slices < 1) slices = 1;
    const int per = (int)cdiv(dim, slices);
    slices = (int)cdiv(dim, per);
    lh_fill(y, 0.f, (int64_t)outer * inner);
    hipLaunchKernelGGL(k_sum_dim_split, dim3((unsigned)cdiv(inner, 64), slices, outer), dim3(TPB), 0, g_stream, x, y, dim, inner, per);
  }
  else hipLaunchKernelGGL(k_sum_dim_inner, dim3(stream_grid((int64_t)outer * inner, TPB)), dim3(TPB), 0, g_stream, x, y, outer, dim, inner);
  LH_CHECK_LAUNCH();
}
void lh_sum_dim_grad(float* dx, const float* dy, int outer, int dim, int inner) { LZ_ENTER(); lazy::rd_f(dy, (int64_t)outer * inner); lazy::rw_f(dx, (int64_t)outer * dim * inner); ProfScope prof_(CAT_REDUCE);
  int64_t n = (int64_t)outer * dim * inner;
  if (n <= 0) return;
  hipLaunchKernelGGL(k_sum_dim_grad, dim3(stream_grid(n, TPB * 4)), dim3(TPB), 0, g_stream, dx, dy, n, dim, inner);
  LH_CHECK_LAUNCH();
}

void lh_softmax(int is_log, const float* x, float* y, int outer, int c, int inner) { LZ_ENTER(); lazy::rd_f(x, (int64_t)outer * c * inner); lazy::out_f(y, (int64_t)outer * c * inner, y == x); ProfScope prof_(CAT_REDUCE);
  if ((int64_t)outer * c * inner <= 0) return;
  if (inner == 1 && rec_ok((int64_t)outer * c)) { rec_cmd(CL_SOFTMAX, outer, c, is_log ? 1 : 0, 0.f, 0.f, 0.f, 0.f, y, x, nullptr, nullptr); return; }
  if (inner == 1) {
    if (c <= 1024 || outer >= 4 * g_num_cu) {
      int grid = stream_grid((int64_t)outer * 64, TPB);
      if (is_log) hipLaunchKernelGGL((k_softmax_rows_wave<true>), dim3(grid), dim3(TPB), 0, g_stream, x, y, outer, c);
      else hipLaunchKernelGGL((k_softmax_rows_wave<false>), dim3(grid), dim3(TPB), 0, g_stream, x, y, outer, c);
    } else {
      if (is_log) hipLaunchKernelGGL((k_softmax_rows_block<true>), dim3(outer), dim3(TPB), 0, g_stream, x, y, c);
      else hipLaunchKernelGGL((k_softmax_rows_block<false>), dim3(outer), dim3(TPB), 0, g_stream, x, y, c);
    }
  } else {
    int grid = stream_grid((int64_t)outer * inner, TPB);
    if (is_log) hipLaunchKernelGGL((k_softmax_inner<true>), dim3(grid), dim3(TPB), 0, g_stream, x, y, outer, c, inner);
    else hipLaunchKernelGGL((k_softmax_inner<false>), dim3(grid), dim3(TPB), 0, g_stream, x, y, outer, c, inner);
  }
  LH_CHECK_LAUNCH();
}
void lh_softmax_grad(int is_log, const float* y, const float* dy, float* dx, int outer, int c, int inner) { LZ_ENTER(); lazy::rd_f(y, (int64_t)outer * c * inner); lazy::rd_f(dy, (int64_t)outer * c * inner); lazy::rw_f(dx, (int64_t)outer * c * inner); ProfScope prof_(CAT_REDUCE);
  int64_t groups = (int64_t)outer * inner;
  if (groups * c <= 0) return;
  if (inner == 1 && rec_ok(groups * c)) { rec_cmd(CL_SOFTMAX_GRAD, outer, c, is_log ? 1 : 0, 0.f, 0.f, 0.f, 0.f, dx, y, dy, nullptr); return; }
  int grid = stream_grid(groups * 64, TPB);
  if (is_log) hipLaunchKernelGGL((k_softmax_grad_wave<true>), dim3(grid), dim3(TPB), 0, g_stream, y, dy, dx, groups, c, inner);
  else hipLaunchKernelGGL((k_softmax_grad_wave<false>), dim3(grid), dim3(TPB), 0, g_stream, y, dy, dx, groups, c, inner);
  LH_CHECK_LAUNCH();
}
void lh_nll(const float* x, const int* target, float* y, int batch, int stride) { LZ_ENTER(); lazy::rd_f(x, (int64_t)batch * stride); lazy::rd_f(target, batch); lazy::wr_f(y, batch); ProfScope prof_(CAT_REDUCE);
  if (batch <= 0) return;
  if (rec_ok(batch)) { rec_cmd(CL_NLL, batch, stride, 0, 0.f, 0.f, 0.f, 0.f, y, x, target, nullptr); return; }
  hipLaunchKernelGGL(k_nll, dim3(cdiv(batch, 64)), dim3(64), 0, g_stream, x, target, y, batch, stride);
  LH_CHECK_LAUNCH();
}
void lh_nll_grad(float* dx, const int* target, const float* dy, int batch, int stride) { LZ_ENTER(); lazy::rd_f(dy, batch); lazy::rd_f(target, batch); lazy::rw_f(dx, (int64_t)batch * stride); ProfScope prof_(CAT_REDUCE);
  if (batch <= 0) return;
  if (rec_ok(batch)) { rec_cmd(CL_NLL_GRAD, batch, stride, 0, 0.f, 0.f, 0.f, 0.f, dx, dy, target, nullptr); return; }
  hipLaunchKernelGGL(k_nll_grad, dim3(cdiv(batch, 64)), dim3(64), 0, g_stream, dx, target, dy, batch, stride);
  LH_CHECK_LAUNCH();
}

}  // extern "C"
