// Streaming (HBM-bound) operators: fills, activations and their gradients, scalar and
// broadcast arithmetic, permute, dropout, concat and the optimizer updates.
// All are grid-stride kernels over float4 where the pointers allow it; each element is
// read and written once, so the bound is bytes moved / HBM bandwidth.
#include "lh_common.h"
using namespace lh;

namespace {

constexpr int TPB = 256;

__global__ void __launch_bounds__(TPB) k_fill(float* __restrict__ y, float v, int64_t n) {
  // vector body (y 16-byte aligned at its base is required by the caller) + scalar tail
  int64_t n4 = n >> 2;
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (int64_t j = i; j < n4; j += st) reinterpret_cast<float4*>(y)[j] = make_float4(v, v, v, v);
  for (int64_t j = 4 * n4 + i; j < n; j += st) y[j] = v;
}
__global__ void __launch_bounds__(TPB) k_fill_scalar(float* y, float v, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n; i += st) y[i] = v;
}
__global__ void __launch_bounds__(TPB) k_fill_bias(float* y, const float* bias, int64_t c, int64_t inner, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n; i += st) y[i] = bias[(i / inner) % c];
}

static inline bool al16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// ---- generic vectorised elementwise driver: out[i] = f(a[i], b[i], c[i]) --------------
template <int NIN, class F>
__global__ void __launch_bounds__(TPB) k_ew_vec(float* out /* may be one of the inputs (in-place forms): no restrict */, const float* a, const float* b, const float* c, int64_t n, F f) {
  int64_t n4 = n >> 2;
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (int64_t j = i; j < n4; j += st) {
    float4 va = reinterpret_cast<const float4*>(a)[j];
    float4 vb = NIN > 1 ? reinterpret_cast<const float4*>(b)[j] : va;
    float4 vc = NIN > 2 ? reinterpret_cast<const float4*>(c)[j] : va;
    float4 r;
    r.x = f(va.x, vb.x, vc.x); r.y = f(va.y, vb.y, vc.y); r.z = f(va.z, vb.z, vc.z); r.w = f(va.w, vb.w, vc.w);
    reinterpret_cast<float4*>(out)[j] = r;
  }
  for (int64_t j = 4 * n4 + i; j < n; j += st) out[j] = f(a[j], NIN > 1 ? b[j] : 0.f, NIN > 2 ? c[j] : 0.f);
}
template <int NIN, class F>
__global__ void __launch_bounds__(TPB) k_ew_scalar(float* out, const float* a, const float* b, const float* c, int64_t n, F f) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (int64_t j = i; j < n; j += st) out[j] = f(a[j], NIN > 1 ? b[j] : 0.f, NIN > 2 ? c[j] : 0.f);
}
// g = dy where y > 0 else 0, delivered to two gradient buffers in one pass
template <bool ACC_A, bool ACC_B>
__global__ void __launch_bounds__(TPB) k_add_relu_grad2(const float* __restrict__ y, const float* __restrict__ dy, float* __restrict__ ad, float* __restrict__ bd, int64_t n) {
  int64_t n4 = n >> 2;
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (int64_t j = i; j < n4; j += st) {
    float4 vy = reinterpret_cast<const float4*>(y)[j], g = reinterpret_cast<const float4*>(dy)[j];
    g.x = vy.x > 0.f ? g.x : 0.f; g.y = vy.y > 0.f ? g.y : 0.f; g.z = vy.z > 0.f ? g.z : 0.f; g.w = vy.w > 0.f ? g.w : 0.f;
    float4 ra = g, rb = g;
    if (ACC_A) { float4 o = reinterpret_cast<const float4*>(ad)[j]; ra.x += o.x; ra.y += o.y; ra.z += o.z; ra.w += o.w; }
    if (ACC_B) { float4 o = reinterpret_cast<const float4*>(bd)[j]; rb.x += o.x; rb.y += o.y; rb.z += o.z; rb.w += o.w; }
    reinterpret_cast<float4*>(ad)[j] = ra; reinterpret_cast<float4*>(bd)[j] = rb;
  }
  for (int64_t j = 4 * n4 + i; j < n; j += st) {
    float g = y[j] > 0.f ? dy[j] : 0.f;
    ad[j] = ACC_A ? ad[j] + g : g; bd[j] = ACC_B ? bd[j] + g : g;
  }
}
template <int NIN, class F>
void ew(float* out, const float* a, const float* b, const float* c, int64_t n, F f) {
  if (n <= 0) return;
  work_add(CAT_ELEMENTWISE, 4.0 * (NIN + 1) * (double)n);
  bool vec = al16(out) && al16(a) && (NIN < 2 || al16(b)) && (NIN < 3 || al16(c));
  int grid = stream_grid(n, TPB * 8);
  if (vec) hipLaunchKernelGGL((k_ew_vec<NIN, F>), dim3(grid), dim3(TPB), 0, g_stream, out, a, b, c, n, f);
  else hipLaunchKernelGGL((k_ew_scalar<NIN, F>), dim3(grid), dim3(TPB), 0, g_stream, out, a, b, c, n, f);
}

__device__ __forceinline__ float bop(int op, float a, float b) {
  switch (op) { case LH_ADD: return a + b; case LH_SUB: return a - b; case LH_MUL: return a * b; default: return a / b; }
}

struct Dims4 { int d[4]; int64_t sa[4]; int64_t sb[4]; };

}  // namespace

// Records of one label byte and `count` pixel bytes (CIFAR-10's .bin layout) -> x[n, count] = byte / 255.0f, y[n] = byte.
// A thread turns 4 consecutive pixels into one 16-byte store; a wave reads 256 consecutive record bytes.  The division
// is the correctly rounded one, so the floats carry the bits the host loop `(float)(unsigned char)b / 255.0f` gives.
template <int V>
__global__ void k_cifar_decode(const unsigned char* __restrict__ rec, float* __restrict__ x, int* __restrict__ y,
                               int64_t n_groups, int count) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, st = (int64_t)gridDim.x * blockDim.x;
  for (; i < n_groups; i += st) {
    const int64_t e = i * V, r = e / count;
    const int j = (int)(e - r * count);
    const unsigned char* src = rec + r * ((int64_t)count + 1) + 1 + j;
    if (j == 0) y[r] = (int)src[-1];
    if constexpr (V == 4) {
      float4 o;
      o.x = __fdiv_rn((float)src[0], 255.0f); o.y = __fdiv_rn((float)src[1], 255.0f);
      o.z = __fdiv_rn((float)src[2], 255.0f); o.w = __fdiv_rn((float)src[3], 255.0f);
      *reinterpret_cast<float4*>(x + e) = o;
    } else {
      x[e] = __fdiv_rn((float)src[0], 255.0f);
    }
  }
}

// repeat0 (the sliding window of the Lookahead layer): out[i0, i1, j] = in[i0 + i1, j] for i0 < rows - context, i1 <= context.
__global__ void k_repeat0(const float* __restrict__ in, float* __restrict__ out, int c1, int64_t inner, int64_t n_out) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, st = (int64_t)gridDim.x * blockDim.x;
  for (; i < n_out; i += st) {
    const int64_t j = i % inner, r = i / inner;
    const int64_t i0 = r / c1, i1 = r - i0 * c1;
    out[i] = in[(i0 + i1) * inner + j];
  }
}
// ind[r, j] += sum over the windows that hold row r: outd[r - i1, i1, j] for 0 <= i1 <= context, 0 <= r - i1 < out_rows (a gather)
__global__ void k_repeat0_grad(float* __restrict__ ind, const float* __restrict__ outd, int c1, int64_t out_rows, int64_t inner, int64_t n_in) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, st = (int64_t)gridDim.x * blockDim.x;
  for (; i < n_in; i += st) {
    const int64_t j = i % inner, r = i / inner;
    float acc = 0.f;
    for (int i1 = 0; i1 < c1; i1++) {
      const int64_t i0 = r - i1;
      if (i0 >= 0 && i0 < out_rows) acc += outd[(i0 * c1 + i1) * inner + j];
    }
    ind[i] += acc;
  }
}

extern "C" {

void lh_fill(float* x, float v, int64_t n) { LZ_ENTER(); lazy::wr_f(x, n); ProfScope prof_(CAT_FILL);
  if (n > 0 && rec_ok(n)) { rec_cmd(CL_FILL, (int)n, 0, 0, v, 0.f, 0.f, 0.f, x, nullptr, nullptr, nullptr); return; }
  if (n <= 0) return;
  if (al16(x)) hipLaunchKernelGGL(k_fill, dim3(stream_grid(n, TPB * 8)), dim3(TPB), 0, g_stream, x, v, n);
  else hipLaunchKernelGGL(k_fill_scalar, dim3(stream_grid(n, TPB * 4)), dim3(TPB), 0, g_stream, x, v, n);
  LH_CHECK_LAUNCH();
}

void lh_fill_with_bias(float* y, const float* bias, int64_t outer, int64_t c, int64_t inner) {
  int64_t n = outer * c * inner;
  if (n <= 0) return;
  LZ_ENTER(); lazy::rd_f(bias, c); lazy::wr_f(y, n);
  hipLaunchKernelGGL(k_fill_bias, dim3(stream_grid(n, TPB * 4)), dim3(TPB), 0, g_stream, y, bias, c, inner, n);
  LH_CHECK_LAUNCH();
}

void lh_clip(float* x, float bound, int64_t n) {
  LZ_ENTER(); lazy::rw_f(x, n);
  side_join();      // clips gradients, which may still be in flight on the side stream
  ew<1>(x, x, nullptr, nullptr, n, [bound] __device__(float v, float, float) { return v > bound ? bound : (v < -bound ? -bound : v); });
  LH_CHECK_LAUNCH();
}

__global__ void k_mask4d(float* x, const int* lengths, int64_t n, int cd, int t) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, st = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += st) {
    int u = (int)(i % t);
    int b = (int)(i / ((int64_t)cd * t));
    if (u >= lengths[b]) x[i] = 0.f;
  }
}
void lh_mask4d(float* x, const int* lengths, int n, int c, int d, int t) {
  int64_t tot = (int64_t)n * c * d * t;
  if (tot <= 0) return;
  LZ_ENTER(); lazy::rd_f(lengths, n); lazy::rw_f(x, tot);
  hipLaunchKernelGGL(k_mask4d, dim3(stream_grid(tot, TPB * 4)), dim3(TPB), 0, g_stream, x, lengths, tot, c * d, t);
  LH_CHECK_LAUNCH();
}

void lh_repeat0(const float* in, float* out, int rows, int context, int64_t inner) {
  if (rows < 1 || context < 0 || context >= rows || inner < 1) { LH_FAIL("lh_repeat0: rows %d, context %d, inner %lld", rows, context, (long long)inner); return; }
  const int64_t n_out = (int64_t)(rows - context) * (context + 1) * inner;
  LZ_ENTER(); lazy::rd_f(in, (int64_t)rows * inner); lazy::wr_f(out, n_out);
  hipLaunchKernelGGL(k_repeat0, dim3(stream_grid(n_out, TPB * 4)), dim3(TPB), 0, g_stream, in, out, context + 1, inner, n_out);
  LH_CHECK_LAUNCH();
}
void lh_repeat0_grad(float* ind, const float* outd, int rows, int context, int64_t inner) {
  if (rows < 1 || context < 0 || context >= rows || inner < 1) { LH_FAIL("lh_repeat0_grad: rows %d, context %d, inner %lld", rows, context, (long long)inner); return; }
  const int64_t n_in = (int64_t)rows * inner;
  LZ_ENTER(); lazy::rd_f(outd, (int64_t)(rows - context) * (context + 1) * inner); lazy::rw_f(ind, n_in);
  hipLaunchKernelGGL(k_repeat0_grad, dim3(stream_grid(n_in, TPB * 2)), dim3(TPB), 0, g_stream, ind, outd, context + 1, (int64_t)(rows - context), inner, n_in);
  LH_CHECK_LAUNCH();
}

void lh_cifar_decode(const unsigned char* records, float* x, int* y, int n, int count) {
  if (n < 0 || count <= 0) { LH_FAIL("lh_cifar_decode: n %d, count %d", n, count); return; }
  if (n == 0) return;
  const int64_t tot = (int64_t)n * count;
  LZ_ENTER(); lazy::rd(records, (size_t)n * ((size_t)count + 1)); lazy::wr_f(x, tot); lazy::wr_f(y, n);
  if (count % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
    hipLaunchKernelGGL(k_cifar_decode<4>, dim3(stream_grid(tot / 4, TPB)), dim3(TPB), 0, g_stream, records, x, y, tot / 4, count);
  } else {
    hipLaunchKernelGGL(k_cifar_decode<1>, dim3(stream_grid(tot, TPB * 4)), dim3(TPB), 0, g_stream, records, x, y, tot, count);
  }
  LH_CHECK_LAUNCH();
}

void lh_unary(int op, const float* x, float* y, int64_t n, float lo, float hi) {
  LZ_SCOPE();
  // relu in place behind a parked batch norm, residual join or `+`: the chain runs as its fused kernel
  if (op == LH_RELU && x == y && lazy::g_busy && !lazy::g_replay && lazy::take_relu_inplace(y, n)) return;
  if (lazy::g_busy && !lazy::g_replay) { lazy::flush_parked(); if (x == y) lazy::rw_f(y, n); else { lazy::rd_f(x, n); lazy::wr_f(y, n); } }
  ProfScope prof_(CAT_ELEMENTWISE);
  if (n > 0 && op >= LH_RELU && op <= LH_HARDTANH && rec_ok(n)) { rec_cmd(CL_UNARY, (int)n, op, 0, lo, hi, 0.f, 0.f, y, x, nullptr, nullptr); return; }
  switch (op) {
    case LH_RELU: ew<1>(y, x, nullptr, nullptr, n, [] __device__(float v, float, float) { return v < 0.f ? 0.f : v; }); break;
    case LH_TANH: ew<1>(y, x, nullptr, nullptr, n, [] __device__(float v, float, float) { return tanhf(v); }); break;
    case LH_SIGMOID: ew<1>(y, x, nullptr, nullptr, n, [] __device__(float v, float, float) { return 1.0f / (expf(-v) + 1.0f); }); break;
    case LH_EXP: ew<1>(y, x, nullptr, nullptr, n, [] __device__(float v, float, float) { return expf(v); }); break;
    case LH_LOG: ew<1>(y, x, nullptr, nullptr, n, [] __device__(float v, float, float) { return logf(v); }); break;
    case LH_SQRT: ew<1>(y, x, nullptr, nullptr, n, [] __device__(float v, float, float) { return sqrtf(v); }); break;
    case LH_SQUARE: ew<1>(y, x, nullptr, nullptr, n, [] __device__(float v, float, float) { return v * v; }); break;
    case LH_HARDTANH: ew<1>(y, x, nullptr, nullptr, n, [lo, hi] __device__(float v, float, float) { return v < lo ? lo : (v > hi ? hi : v); }); break;
    default: LH_FAIL("lh_unary: unknown op %d", op); return;
  }
  LH_CHECK_LAUNCH();
}

void lh_unary_grad(int op, const float* x, const float* y, const float* dy, float* dx, int64_t n, int inplace, float lo, float hi) {
  LZ_SCOPE();
  // relu_grad in place waits for the call behind it: a batch-norm gradient (or `+`'s gradient, then a batch norm's) takes the mask along
  if (op == LH_RELU && inplace && dy == dx && lazy::park_relu_grad_inplace(y, dx, n)) return;
  bool fresh = false;
  if (lazy::g_busy && !lazy::g_replay) {
    lazy::flush_parked();
    if (inplace) { lazy::rd_f(y, n); lazy::rw_f(dx, n); }
    else {
      if (op == LH_RELU || op == LH_HARDTANH || op == LH_LOG || op == LH_SQUARE) lazy::rd_f(x, n); else lazy::rd_f(y, n);
      lazy::rd_f(dy, n);
      if (op == LH_RELU) fresh = lazy::acc_f(dx, n); else lazy::rw_f(dx, n);
    }
  }
  ProfScope prof_(CAT_ELEMENTWISE);
  if (n > 0 && op >= LH_RELU && op <= LH_HARDTANH && rec_ok(n)) { rec_cmd(CL_UNARY_GRAD, (int)n, op, inplace ? 1 : 0, lo, hi, 0.f, 0.f, dx, x, y, dy); return; }
  // out = dx; inputs (a, b, c) chosen per op.  All forms are dx (+)= g(x|y, dy).
  switch (op) {
    case LH_RELU:
      if (inplace) ew<2>(dx, dx, y, nullptr, n, [] __device__(float d, float yv, float) { return yv > 0.f ? d : 0.f; });
      else if (fresh) ew<2>(dx, x, dy, nullptr, n, [] __device__(float xv, float g, float) { return 0.f + (xv < 0.f ? 0.f : g); });     // dx is an untouched zero block
      else ew<3>(dx, dx, x, dy, n, [] __device__(float d, float xv, float g) { return d + (xv < 0.f ? 0.f : g); });
      break;
    case LH_HARDTANH:
      if (inplace) ew<2>(dx, dx, y, nullptr, n, [lo, hi] __device__(float d, float yv, float) { return (yv > lo && yv < hi) ? d : 0.f; });
      else ew<3>(dx, dx, x, dy, n, [lo, hi] __device__(float d, float xv, float g) { return d + ((xv < lo || xv > hi) ? 0.f : g); });
      break;
    case LH_TANH: ew<3>(dx, dx, y, dy, n, [] __device__(float d, float yv, float g) { return d + (1.0f - yv * yv) * g; }); break;
    case LH_SIGMOID: ew<3>(dx, dx, y, dy, n, [] __device__(float d, float yv, float g) { return d + ((1.0f - yv) * yv) * g; }); break;
    case LH_EXP: ew<3>(dx, dx, y, dy, n, [] __device__(float d, float yv, float g) { return d + g * yv; }); break;
    case LH_LOG: ew<3>(dx, dx, x, dy, n, [] __device__(float d, float xv, float g) { return d + g / xv; }); break;
    case LH_SQRT: ew<3>(dx, dx, y, dy, n, [] __device__(float d, float yv, float g) { return d + g / yv / 2.0f; }); break;
    case LH_SQUARE: ew<3>(dx, dx, x, dy, n, [] __device__(float d, float xv, float g) { return d + g * xv * 2.0f; }); break;
    default: LH_FAIL("lh_unary_grad: unknown op %d", op); return;
  }
  LH_CHECK_LAUNCH();
}

void lh_scalar_op(int op, const float* x, float* y, float s, int64_t n) {
  LZ_ENTER(); if (x == y) lazy::rw_f(y, n); else { lazy::rd_f(x, n); lazy::wr_f(y, n); }
  ProfScope prof_(CAT_ELEMENTWISE);
  LH_REQUIRE(op >= LH_ADD && op <= LH_DIV, "lh_scalar_op: unknown op %d", op);
  if (n > 0 && rec_ok(n)) { rec_cmd(CL_SCALAR, (int)n, op, 0, s, 0.f, 0.f, 0.f, y, x, nullptr, nullptr); return; }
  ew<1>(y, x, nullptr, nullptr, n, [op, s] __device__(float v, float, float) { return bop(op, v, s); });
  LH_CHECK_LAUNCH();
}

void lh_add_relu(const float* a, const float* b, float* out, int64_t n) {
  LZ_ENTER(); lazy::rd_f(a, n); lazy::rd_f(b, n); lazy::out_f(out, n, out == a || out == b);
  ProfScope prof_(CAT_ELEMENTWISE);
  ew<2>(out, a, b, nullptr, n, [] __device__(float x, float y, float) { float r = x + y; return r < 0.f ? 0.f : r; });
  LH_CHECK_LAUNCH();
}
void lh_add_relu_grad(const float* y, const float* dy, float* ad, float abeta, float* bd, float bbeta, int64_t n) {
  // g = dy where y > 0 else 0 ; ad = abeta*ad + g ; bd = bbeta*bd + g   (either target may be NULL)
  if (n <= 0) return;
  LH_REQUIRE((abeta == 0.f || abeta == 1.f) && (bbeta == 0.f || bbeta == 1.f), "lh_add_relu_grad: beta must be 0 or 1");
  LZ_ENTER(); lazy::rd_f(y, n); lazy::rd_f(dy, n);
  if (ad) abeta = lazy::beta_f(ad, n, abeta);
  if (bd && bd != ad) bbeta = lazy::beta_f(bd, n, bbeta);
  ProfScope prof_(CAT_ELEMENTWISE);
  if (ad && bd && ad != bd && al16(y) && al16(dy) && al16(ad) && al16(bd)) {
    const int grid = stream_grid(n, TPB * 8);
    work_add(CAT_ELEMENTWISE, (16.0 + (abeta != 0.f ? 4.0 : 0.0) + (bbeta != 0.f ? 4.0 : 0.0)) * (double)n);
#define GO(A, B) hipLaunchKernelGGL((k_add_relu_grad2<A, B>), dim3(grid), dim3(TPB), 0, g_stream, y, dy, ad, bd, n)
    if (abeta != 0.f) { if (bbeta != 0.f) GO(true, true); else GO(true, false); }
    else { if (bbeta != 0.f) GO(false, true); else GO(false, false); }
#undef GO
    LH_CHECK_LAUNCH();
    return;
  }
  if (ad) {
    if (abeta == 0.f) ew<2>(ad, y, dy, nullptr, n, [] __device__(float yv, float g, float) { return yv > 0.f ? g : 0.f; });
    else ew<3>(ad, ad, y, dy, n, [] __device__(float d, float yv, float g) { return d + (yv > 0.f ? g : 0.f); });
  }
  if (bd) {
    if (bbeta == 0.f) ew<2>(bd, y, dy, nullptr, n, [] __device__(float yv, float g, float) { return yv > 0.f ? g : 0.f; });
    else ew<3>(bd, bd, y, dy, n, [] __device__(float d, float yv, float g) { return d + (yv > 0.f ? g : 0.f); });
  }
  LH_CHECK_LAUNCH();
}

void lh_geam(const float* x, float alpha, const float* y, float beta, float* out, int64_t n) {
  LZ_ENTER(); lazy::rd_f(x, n); lazy::rd_f(y, n); lazy::out_f(out, n, out == x || out == y);
  ProfScope prof_(CAT_ELEMENTWISE);
  if (n > 0 && rec_ok(n)) { rec_cmd(CL_GEAM, (int)n, 0, 0, alpha, beta, 0.f, 0.f, out, x, y, nullptr); return; }
  ew<2>(out, x, y, nullptr, n, [alpha, beta] __device__(float a, float b, float) { return a * alpha + b * beta; });
  LH_CHECK_LAUNCH();
}

}  // extern "C"

// ---------------------------------------------------------------- broadcast -----------
namespace {

static bool same_dims(const int* a, const int* b, int rank) { for (int i = 0; i < rank; i++) if (a[i] != b[i]) return false; return true; }
static int64_t prod(const int* d, int rank) { int64_t p = 1; for (int i = 0; i < rank; i++) p *= d[i]; return p; }

static bool make_dims4(Dims4& D, const int* adims, const int* bdims, const int* odims, int rank) {
  if (rank < 1 || rank > 4) return false;
  int pad = 4 - rank;
  int ad[4] = {1, 1, 1, 1}, bd[4] = {1, 1, 1, 1};
  for (int i = 0; i < 4; i++) D.d[i] = 1;
  for (int i = 0; i < rank; i++) { ad[pad + i] = adims[i]; bd[pad + i] = bdims[i]; D.d[pad + i] = odims[i]; }
  int64_t s = 1; for (int i = 3; i >= 0; i--) { D.sa[i] = ad[i] == 1 ? 0 : s; s *= ad[i]; }
  s = 1; for (int i = 3; i >= 0; i--) { D.sb[i] = bd[i] == 1 ? 0 : s; s *= bd[i]; }
  for (int i = 0; i < 4; i++) {
    if (ad[i] != 1 && ad[i] != D.d[i]) return false;
    if (bd[i] != 1 && bd[i] != D.d[i]) return false;
  }
  return true;
}

__global__ void __launch_bounds__(TPB) k_bcast_op(int op, const float* a, const float* b, float* out, Dims4 D, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n; i += st) {
    int64_t r = i;
    int i3 = (int)(r % D.d[3]); r /= D.d[3];
    int i2 = (int)(r % D.d[2]); r /= D.d[2];
    int i1 = (int)(r % D.d[1]); r /= D.d[1];
    int i0 = (int)r;
    int64_t ia = i0 * D.sa[0] + i1 * D.sa[1] + i2 * D.sa[2] + i3 * D.sa[3];
    int64_t ib = i0 * D.sb[0] + i1 * D.sb[1] + i2 * D.sb[2] + i3 * D.sb[3];
    out[i] = bop(op, a[ia], b[ib]);
  }
}

// small[j] (op)= reduce over the broadcast positions of g(...).  One wave per small element.
// mode 0: value = big[i]                       (bcast_update with reduction, ADD/SUB)
// mode 1: value = grad wrt operand `which` of out = a op b, with outd = big
template <int MODE>
__global__ void __launch_bounds__(TPB) k_bcast_reduce(int op, int which, float* small, const float* a, const float* b, const float* big,
                                                      Dims4 D /* d = out dims, sa = strides of small, sb = strides of other */,
                                                      int64_t nsmall, int64_t nred, int rd0, int rd1, int rd2, int rd3) {
  // rdX = size of the reduced index space along axis X (out dim where small dim == 1, else 1)
  const int lane = threadIdx.x & 63;
  int64_t w = ((int64_t)blockIdx.x * TPB + threadIdx.x) >> 6, nw = ((int64_t)gridDim.x * TPB) >> 6;
  for (; w < nsmall; w += nw) {
    // decode the kept coordinates of small element w (axes where small dim != 1)
    int k[4]; int64_t r = w;
    int kd3 = rd3 == 1 ? D.d[3] : 1, kd2 = rd2 == 1 ? D.d[2] : 1, kd1 = rd1 == 1 ? D.d[1] : 1;
    k[3] = (int)(r % kd3); r /= kd3; k[2] = (int)(r % kd2); r /= kd2; k[1] = (int)(r % kd1); r /= kd1; k[0] = (int)r;
    float acc = 0.f;
    for (int64_t q = lane; q < nred; q += 64) {
      int64_t t = q; int c[4];
      c[3] = k[3] + (int)(t % rd3); t /= rd3; c[2] = k[2] + (int)(t % rd2); t /= rd2; c[1] = k[1] + (int)(t % rd1); t /= rd1; c[0] = k[0] + (int)t;
      int64_t io = ((int64_t)(c[0] * D.d[1] + c[1]) * D.d[2] + c[2]) * D.d[3] + c[3];
      float v = big[io];
      if (MODE == 1) {
        int64_t is = c[0] * D.sa[0] + c[1] * D.sa[1] + c[2] * D.sa[2] + c[3] * D.sa[3];   // index in small's own tensor
        int64_t it = c[0] * D.sb[0] + c[1] * D.sb[1] + c[2] * D.sb[2] + c[3] * D.sb[3];   // index in the other operand
        // which == 0: small is `a` (x), other is `b`; which == 1: small is `b`, other is `a`
        float av = which == 0 ? a[is] : a[it];
        float bv = which == 0 ? b[it] : b[is];
        switch (op) {
          case LH_ADD: break;
          case LH_SUB: v = which == 0 ? v : 0.0f - v; break;
          case LH_MUL: v = which == 0 ? v * bv : v * av; break;
          default: v = which == 0 ? v / bv : -1.0f * av * v / (bv * bv); break;
        }
      }
      acc += v;
    }
    acc = lh_wave_sum(acc);
    if (lane == 0) {
      if (MODE == 0 && op == LH_SUB) small[w] -= acc; else small[w] += acc;
    }
  }
}

// Elementwise part of a broadcast gradient for an operand that has the full output shape.
__global__ void __launch_bounds__(TPB) k_bcast_grad_full(int op, int which, float* gd, const float* a, const float* b, const float* od, Dims4 D, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n; i += st) {
    int64_t r = i;
    int i3 = (int)(r % D.d[3]); r /= D.d[3];
    int i2 = (int)(r % D.d[2]); r /= D.d[2];
    int i1 = (int)(r % D.d[1]); r /= D.d[1];
    int i0 = (int)r;
    int64_t ia = i0 * D.sa[0] + i1 * D.sa[1] + i2 * D.sa[2] + i3 * D.sa[3];
    int64_t ib = i0 * D.sb[0] + i1 * D.sb[1] + i2 * D.sb[2] + i3 * D.sb[3];
    float c = od[i], g;
    switch (op) {
      case LH_ADD: g = c; break;
      case LH_SUB: g = which == 0 ? c : 0.0f - c; break;
      case LH_MUL: g = which == 0 ? c * b[ib] : c * a[ia]; break;
      default: g = which == 0 ? c / b[ib] : -1.0f * a[ia] * c / (b[ib] * b[ib]); break;
    }
    gd[i] += g;
  }
}

// Launch the reduction of `big`-shaped values into the operand whose dims are sdims.
template <int MODE>
void launch_reduce(int op, int which, float* small, const int* sdims4, const float* a, const float* b, const float* big, const Dims4& Dsmall_other) {
  int rd[4]; int64_t nred = 1, nsmall = 1;
  for (int i = 0; i < 4; i++) {
    rd[i] = (sdims4[i] == 1 && Dsmall_other.d[i] > 1) ? Dsmall_other.d[i] : 1;
    nred *= rd[i];
    nsmall *= (rd[i] == 1 ? Dsmall_other.d[i] : 1);
  }
  int grid = (int)cdiv(nsmall * 64, TPB); if (grid > g_num_cu * 16) grid = g_num_cu * 16; if (grid < 1) grid = 1;
  hipLaunchKernelGGL((k_bcast_reduce<MODE>), dim3(grid), dim3(TPB), 0, g_stream, op, which, small, a, b, big, Dsmall_other, nsmall, nred, rd[0], rd[1], rd[2], rd[3]);
}

}  // namespace

extern "C" {

void lh_bcast_op(int op, const float* a, const int* adims, const float* b, const int* bdims, float* out, const int* odims, int rank) {
  LH_REQUIRE(op >= LH_ADD && op <= LH_DIV, "lh_bcast_op: unknown op %d", op);
  int64_t n = prod(odims, rank);
  if (n <= 0) return;
  LZ_SCOPE();
  const bool same = same_dims(adims, odims, rank) && same_dims(bdims, odims, rank);
  // a same-shape `+` waits for the call behind it: relu in place makes it one kernel, behind a parked batch norm the residual join
  if (same && op == LH_ADD && !rec_ok(n) && lazy::park_add(a, b, out, n)) return;
  if (lazy::g_busy && !lazy::g_replay) { lazy::flush_parked(); lazy::rd_f(a, prod(adims, rank)); lazy::rd_f(b, prod(bdims, rank)); lazy::out_f(out, n, out == a || out == b); }
  ProfScope prof_(CAT_ELEMENTWISE);
  if (same) {
    if (rec_ok(n)) { rec_cmd(CL_BIN, (int)n, op, 0, 0.f, 0.f, 0.f, 0.f, out, a, b, nullptr); return; }
    ew<2>(out, a, b, nullptr, n, [op] __device__(float x, float y, float) { return bop(op, x, y); });
  } else {
    Dims4 D;
    LH_REQUIRE(make_dims4(D, adims, bdims, odims, rank), "lh_bcast_op: shapes do not broadcast (rank %d)", rank);
    hipLaunchKernelGGL(k_bcast_op, dim3(stream_grid(n, TPB * 4)), dim3(TPB), 0, g_stream, op, a, b, out, D, n);
  }
  LH_CHECK_LAUNCH();
}

void lh_bcast_op_grad(int op, const float* a, float* ad, const int* adims, int a_is_input,
                      const float* b, float* bd, const int* bdims, int b_is_input,
                      const float* outd, const int* odims, int rank) {
  LH_REQUIRE(op >= LH_ADD && op <= LH_DIV, "lh_bcast_op_grad: unknown op %d", op);
  int64_t n = prod(odims, rank);
  if (n <= 0) return;
  Dims4 D;
  LH_REQUIRE(make_dims4(D, adims, bdims, odims, rank), "lh_bcast_op_grad: shapes do not broadcast (rank %d)", rank);
  int pad = 4 - rank; int a4[4] = {1, 1, 1, 1}, b4[4] = {1, 1, 1, 1};
  for (int i = 0; i < rank; i++) { a4[pad + i] = adims[i]; b4[pad + i] = bdims[i]; }
  bool a_full = same_dims(adims, odims, rank), b_full = same_dims(bdims, odims, rank);
  LZ_SCOPE();
  // the gradient of a same-shape `+` right behind a parked relu_grad: both wait for a batch-norm gradient (the residual join's backward)
  if (a_full && b_full && op == LH_ADD && lazy::g_busy && !lazy::g_replay && !rec_ok(n) &&
      lazy::park_add_grad(a_is_input ? nullptr : ad, b_is_input ? nullptr : bd, outd, n)) return;
  bool a_fresh = false, b_fresh = false;
  if (lazy::g_busy && !lazy::g_replay) {
    lazy::flush_parked();
    lazy::rd_f(outd, n);
    lazy::rd_f(a, prod(adims, rank)); lazy::rd_f(b, prod(bdims, rank));
    const bool plain = a_full && b_full && (op == LH_ADD || op == LH_SUB);      // d += g / d -= g: an untouched zero block takes a copy
    if (!a_is_input) { if (plain) a_fresh = lazy::acc_f(ad, n); else lazy::rw_f(ad, prod(adims, rank)); }
    if (!b_is_input && !(bd == ad && !a_is_input)) { if (plain) b_fresh = lazy::acc_f(bd, n); else lazy::rw_f(bd, prod(bdims, rank)); }
  }
  ProfScope prof_(CAT_ELEMENTWISE);
  if (a_full && b_full && op != LH_DIV && rec_ok(n)) {       // same shapes: d += g, d += -g or d += g * other
    if (!a_is_input) rec_cmd(op == LH_MUL ? CL_ACCMUL : CL_ACC, (int)n, 0, 0, 0.f, 0.f, 0.f, 0.f, ad, outd, b, nullptr);
    if (!b_is_input) rec_cmd(op == LH_MUL ? CL_ACCMUL : (op == LH_SUB ? CL_ACCNEG : CL_ACC), (int)n, 0, 0, 0.f, 0.f, 0.f, 0.f, bd, outd, a, nullptr);
    return;
  }
  if (!a_is_input) {
    if (a_full) {
      if (b_full && (op == LH_ADD || op == LH_SUB) && a_fresh) ew<1>(ad, outd, nullptr, nullptr, n, [] __device__(float g, float, float) { return 0.f + g; });
      else if (b_full && op == LH_ADD) ew<2>(ad, ad, outd, nullptr, n, [] __device__(float d, float g, float) { return d + g; });
      else if (b_full && op == LH_SUB) ew<2>(ad, ad, outd, nullptr, n, [] __device__(float d, float g, float) { return d + g; });
      else if (b_full && op == LH_MUL) ew<3>(ad, ad, outd, b, n, [] __device__(float d, float g, float bv) { return d + g * bv; });
      else hipLaunchKernelGGL(k_bcast_grad_full, dim3(stream_grid(n, TPB * 4)), dim3(TPB), 0, g_stream, op, 0, ad, a, b, outd, D, n);
    } else {
      launch_reduce<1>(op, 0, ad, a4, a, b, outd, D);
    }
  }
  if (!b_is_input) {
    if (b_full) {
      if (a_full && op == LH_ADD && b_fresh) ew<1>(bd, outd, nullptr, nullptr, n, [] __device__(float g, float, float) { return 0.f + g; });
      else if (a_full && op == LH_SUB && b_fresh) ew<1>(bd, outd, nullptr, nullptr, n, [] __device__(float g, float, float) { return 0.f + (0.0f - g); });
      else if (a_full && op == LH_ADD) ew<2>(bd, bd, outd, nullptr, n, [] __device__(float d, float g, float) { return d + g; });
      else if (a_full && op == LH_SUB) ew<2>(bd, bd, outd, nullptr, n, [] __device__(float d, float g, float) { return d + (0.0f - g); });
      else if (a_full && op == LH_MUL) ew<3>(bd, bd, outd, a, n, [] __device__(float d, float g, float av) { return d + g * av; });
      else hipLaunchKernelGGL(k_bcast_grad_full, dim3(stream_grid(n, TPB * 4)), dim3(TPB), 0, g_stream, op, 1, bd, a, b, outd, D, n);
    } else {
      Dims4 Ds = D;  // small = b: swap stride roles so sa = strides of small (b), sb = strides of other (a)
      for (int i = 0; i < 4; i++) { Ds.sa[i] = D.sb[i]; Ds.sb[i] = D.sa[i]; }
      launch_reduce<1>(op, 1, bd, b4, a, b, outd, Ds);
    }
  }
  LH_CHECK_LAUNCH();
}

void lh_bcast_update(int op, float* a, const int* adims, const float* b, const int* bdims, int rank) {
  LH_REQUIRE(op >= LH_ADD && op <= LH_DIV, "lh_bcast_update: unknown op %d", op);
  LH_REQUIRE(rank >= 1 && rank <= 4, "lh_bcast_update: rank %d not in 1..4", rank);
  LZ_ENTER(); lazy::rd_f(b, prod(bdims, rank)); lazy::rw_f(a, prod(adims, rank));
  ProfScope prof_(CAT_ELEMENTWISE);
  int od[4];
  for (int i = 0; i < rank; i++) od[i] = adims[i] > bdims[i] ? adims[i] : bdims[i];
  int64_t n = prod(od, rank);
  if (n <= 0) return;
  if (same_dims(adims, od, rank)) {  // a has the full shape: a = a op broadcast(b)
    if (same_dims(bdims, od, rank)) {
      if (rec_ok(n)) { rec_cmd(CL_BIN, (int)n, op, 0, 0.f, 0.f, 0.f, 0.f, a, a, b, nullptr); return; }
      ew<2>(a, a, b, nullptr, n, [op] __device__(float x, float y, float) { return bop(op, x, y); });
    } else {
      Dims4 D;
      LH_REQUIRE(make_dims4(D, adims, bdims, od, rank), "lh_bcast_update: shapes do not broadcast");
      hipLaunchKernelGGL(k_bcast_op, dim3(stream_grid(n, TPB * 4)), dim3(TPB), 0, g_stream, op, (const float*)a, b, a, D, n);
    }
  } else {  // a is the smaller one: reduce b into a (the reference's loop applies op once per broadcast position)
    LH_REQUIRE(op == LH_ADD || op == LH_SUB, "lh_bcast_update: reducing update supports += and -= only");
    LH_REQUIRE(same_dims(bdims, od, rank), "lh_bcast_update: reduce source must have the full shape");
    Dims4 D;
    LH_REQUIRE(make_dims4(D, adims, bdims, od, rank), "lh_bcast_update: shapes do not broadcast");
    int pad = 4 - rank; int a4[4] = {1, 1, 1, 1};
    for (int i = 0; i < rank; i++) a4[pad + i] = adims[i];
    launch_reduce<0>(op, 0, a, a4, nullptr, nullptr, b, D);
  }
  LH_CHECK_LAUNCH();
}

}  // extern "C"

// ------------------------------------------------------------- permute / trans --------
namespace {
struct Perm4 { int yd[4]; int64_t sx[4]; };   // y dims and, for each y axis, the stride in x

// 32x32 LDS-tiled transpose of the two fastest axes when the permutation moves x's fastest
// axis; otherwise a plain gather keeps reads and writes contiguous along the last axis.
template <bool GRAD>
__global__ void __launch_bounds__(TPB) k_permute(const float* __restrict__ src, float* __restrict__ dst, Perm4 P, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n; i += st) {
    int64_t r = i;
    int i3 = (int)(r % P.yd[3]); r /= P.yd[3];
    int i2 = (int)(r % P.yd[2]); r /= P.yd[2];
    int i1 = (int)(r % P.yd[1]); r /= P.yd[1];
    int i0 = (int)r;
    int64_t ix = i0 * P.sx[0] + i1 * P.sx[1] + i2 * P.sx[2] + i3 * P.sx[3];
    if (GRAD) dst[ix] += src[i]; else dst[i] = src[ix];
  }
}
template <bool GRAD>
__global__ void __launch_bounds__(256) k_trans_tile(const float* __restrict__ src, float* __restrict__ dst, int rows, int cols, int64_t batch_stride) {
  // !GRAD: dst[c][r] = src[r][c] (src rows x cols).  GRAD: dst is rows x cols, src is cols x rows: dst[r][c] += src[c][r].
  __shared__ float tile[32][33];
  const float* s = src + (int64_t)blockIdx.z * batch_stride;
  float* d = dst + (int64_t)blockIdx.z * batch_stride;
  int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
  if (!GRAD) {
    for (int j = ty; j < 32; j += 8) { int r = r0 + j, c = c0 + tx; if (r < rows && c < cols) tile[j][tx] = s[(int64_t)r * cols + c]; }
    __syncthreads();
    for (int j = ty; j < 32; j += 8) { int c = c0 + j, r = r0 + tx; if (r < rows && c < cols) d[(int64_t)c * rows + r] = tile[tx][j]; }
  } else {
    for (int j = ty; j < 32; j += 8) { int c = c0 + j, r = r0 + tx; if (r < rows && c < cols) tile[tx][j] = s[(int64_t)c * rows + r]; }
    __syncthreads();
    for (int j = ty; j < 32; j += 8) { int r = r0 + j, c = c0 + tx; if (r < rows && c < cols) d[(int64_t)r * cols + c] += tile[j][tx]; }
  }
}
static bool make_perm(Perm4& P, const int* dims, const int* perm, int rank) {
  if (rank < 1 || rank > 4) return false;
  int pad = 4 - rank; int xd[4] = {1, 1, 1, 1}, pm[4] = {0, 1, 2, 3};
  for (int i = 0; i < rank; i++) { xd[pad + i] = dims[i]; pm[pad + i] = perm[i] + pad; }
  bool seen[4] = {false, false, false, false};
  for (int i = 0; i < 4; i++) { if (pm[i] < 0 || pm[i] > 3 || seen[pm[i]]) return false; seen[pm[i]] = true; }
  int64_t sx[4]; int64_t s = 1; for (int i = 3; i >= 0; i--) { sx[i] = s; s *= xd[i]; }
  for (int i = 0; i < 4; i++) { P.yd[i] = xd[pm[i]]; P.sx[i] = sx[pm[i]]; }
  return true;
}
}  // namespace

extern "C" {

void lh_trans(const float* x, float* y, int rows, int cols) {
  if (rows <= 0 || cols <= 0) return;
  LZ_ENTER(); lazy::rd_f(x, (int64_t)rows * cols); lazy::wr_f(y, (int64_t)rows * cols);
  hipLaunchKernelGGL((k_trans_tile<false>), dim3(cdiv(cols, 32), cdiv(rows, 32), 1), dim3(256), 0, g_stream, x, y, rows, cols, (int64_t)0);
  LH_CHECK_LAUNCH();
}
void lh_trans_grad(float* xd, const float* yd, int rows, int cols) {
  if (rows <= 0 || cols <= 0) return;
  LZ_ENTER(); lazy::rd_f(yd, (int64_t)rows * cols); lazy::rw_f(xd, (int64_t)rows * cols);
  hipLaunchKernelGGL((k_trans_tile<true>), dim3(cdiv(cols, 32), cdiv(rows, 32), 1), dim3(256), 0, g_stream, yd, xd, rows, cols, (int64_t)0);
  LH_CHECK_LAUNCH();
}
void lh_permute(const float* x, float* y, const int* dims, const int* perm, int rank) {
  Perm4 P;
  LH_REQUIRE(make_perm(P, dims, perm, rank), "lh_permute: bad rank/permutation");
  int64_t n = 1; for (int i = 0; i < rank; i++) n *= dims[i];
  if (n <= 0) return;
  LZ_ENTER(); lazy::rd_f(x, n); lazy::wr_f(y, n);
  hipLaunchKernelGGL((k_permute<false>), dim3(stream_grid(n, TPB * 4)), dim3(TPB), 0, g_stream, x, y, P, n);
  LH_CHECK_LAUNCH();
}
void lh_permute_grad(float* xd, const float* yd, const int* dims, const int* perm, int rank) {
  Perm4 P;
  LH_REQUIRE(make_perm(P, dims, perm, rank), "lh_permute_grad: bad rank/permutation");
  int64_t n = 1; for (int i = 0; i < rank; i++) n *= dims[i];
  if (n <= 0) return;
  LZ_ENTER(); lazy::rd_f(yd, n); lazy::rw_f(xd, n);
  hipLaunchKernelGGL((k_permute<true>), dim3(stream_grid(n, TPB * 4)), dim3(TPB), 0, g_stream, yd, xd, P, n);
  LH_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- dropout -------------
__device__ __forceinline__ float ctr_uniform(uint64_t seed, uint64_t index) {
  uint64_t z = seed + 0x9E3779B97F4A7C15ULL * (index + 1);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
  z = z ^ (z >> 31);
  return (float)(z >> 40) * (1.0f / 16777216.0f);
}
__global__ void __launch_bounds__(TPB) k_dropout(const float* x, float* y, float* mask, int64_t n, float p, float scale, uint64_t seed, uint64_t offset,
                                                 const unsigned long long* advance) {
  if (advance) offset += *advance;      // a replayed graph: positions move on by what the earlier replays drew
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n; i += st) {
    bool keep = ctr_uniform(seed, offset + (uint64_t)i) > p;
    y[i] = keep ? x[i] * scale : 0.f;
    mask[i] = keep ? scale : 0.f;
  }
}
void lh_dropout_fwd(const float* x, float* y, float* mask, int64_t n, float p, uint64_t seed, uint64_t offset) {
  LH_REQUIRE(p >= 0.f && p < 1.f, "dropout rate should be [0.0, 1), got %f", p);
  if (n <= 0) return;
  LZ_ENTER(); lazy::rd_f(x, n); lazy::wr_f(y, n); lazy::wr_f(mask, n);
  hipLaunchKernelGGL(k_dropout, dim3(stream_grid(n, TPB * 4)), dim3(TPB), 0, g_stream, x, y, mask, n, p, 1.0f / (1.0f - p), seed, offset,
                     g_capturing ? (const unsigned long long*)g_capture_advance : (const unsigned long long*)nullptr);
  if (g_capturing) g_capture_drawn += (unsigned long long)n;
  LH_CHECK_LAUNCH();
}
void lh_dropout_bwd(const float* dy, const float* mask, float* dx, int64_t n) {
  LZ_ENTER(); lazy::rd_f(dy, n); lazy::rd_f(mask, n);
  if (lazy::acc_f(dx, n)) ew<2>(dx, mask, dy, nullptr, n, [] __device__(float m, float g, float) { return 0.f + m * g; });      // dx is an untouched zero block
  else
  ew<3>(dx, dx, mask, dy, n, [] __device__(float d, float m, float g) { return d + m * g; });
  LH_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- concat --------------
// Up to four tensors per launch: a thread walks the strided side (the concatenated tensor), finds the tensor its position
// belongs to, and copies from (or, for the gradient, adds or copies into) that tensor's packed rows of `st = sizes[t]*inner` floats.
}  // extern "C"
namespace {
constexpr int CAT_MAX = 4;
struct CatArgs { float* p[CAT_MAX]; int64_t st[CAT_MAX]; int64_t off[CAT_MAX]; int add[CAT_MAX]; int n; int64_t lo, width; };
// GRAD: false = forward copy into the concatenated tensor, true = gradient into the packed ones (added where add[t], else overwriting)
// T = float4: every row length, offset and pointer is a multiple of four floats; the lengths in CatArgs, row and total count float4s then.
__device__ __forceinline__ float cat_add(float a, float b) { return a + b; }
__device__ __forceinline__ float4 cat_add(float4 a, float4 b) { return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w); }
template <bool GRAD, class T>
__global__ void __launch_bounds__(TPB) k_concat(CatArgs a, float* cat_, int64_t row, int64_t total) {
  T* cat = reinterpret_cast<T*>(cat_);
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, s = (int64_t)gridDim.x * TPB;
  const bool narrow = total < 0x7fffffffLL && row < 0x7fffffffLL;      // 32-bit divisions where they suffice
  for (; i < total; i += s) {
    int64_t h, l;
    if (narrow) { const uint32_t hh = (uint32_t)i / (uint32_t)a.width; h = hh; l = a.lo + ((uint32_t)i - hh * (uint32_t)a.width); }
    else { h = i / a.width; l = a.lo + (i - h * a.width); }
    int t = 0;
#pragma unroll
    for (int u = 1; u < CAT_MAX; u++) if (u < a.n && l >= a.off[u]) t = u;
    T* q = reinterpret_cast<T*>(a.p[t]);
    if (q == nullptr) continue;
    const int64_t o = h * row + l, e = h * a.st[t] + (l - a.off[t]);
    if (GRAD) q[e] = a.add[t] ? cat_add(q[e], cat[o]) : cat[o]; else cat[o] = q[e];
  }
}
// shrinks the lengths to float4 units when everything is a multiple of four floats and 16-byte aligned
static bool cat_vectorize(CatArgs& a, const float* cat, int64_t& row, int64_t& tot) {
  if ((row | a.lo | a.width) & 3 || ((uintptr_t)cat & 15)) return false;
  for (int u = 0; u < a.n; u++) if ((a.st[u] | a.off[u]) & 3 || ((uintptr_t)a.p[u] & 15)) return false;
  for (int u = 0; u < a.n; u++) { a.st[u] >>= 2; a.off[u] >>= 2; }
  a.lo >>= 2; a.width >>= 2; row >>= 2; tot >>= 2;
  return true;
}
template <bool GRAD>
static void cat_launch(CatArgs a, float* cat, int64_t row, int64_t tot) {
  if (cat_vectorize(a, cat, row, tot)) hipLaunchKernelGGL((k_concat<GRAD, float4>), dim3(stream_grid(tot, TPB * 2)), dim3(TPB), 0, g_stream, a, cat, row, tot);
  else hipLaunchKernelGGL((k_concat<GRAD, float>), dim3(stream_grid(tot, TPB * 4)), dim3(TPB), 0, g_stream, a, cat, row, tot);
}
}  // namespace
extern "C" {
void lh_concat(int n, const float* const* h_in, const int* sizes, float* out, int outer, int inner) {
  int64_t row = 0; for (int t = 0; t < n; t++) row += (int64_t)sizes[t] * inner;
  LZ_ENTER();
  for (int t = 0; t < n; t++) lazy::rd_f(h_in[t], (int64_t)sizes[t] * inner * outer);
  lazy::wr_f(out, row * outer);
  int64_t off = 0;
  for (int t0 = 0; t0 < n; t0 += CAT_MAX) {
    CatArgs a{}; a.n = n - t0 < CAT_MAX ? n - t0 : CAT_MAX; a.lo = off;
    for (int u = 0; u < a.n; u++) { a.p[u] = const_cast<float*>(h_in[t0 + u]); a.st[u] = (int64_t)sizes[t0 + u] * inner; a.off[u] = off; off += a.st[u]; }
    a.width = off - a.lo;
    const int64_t tot = a.width * outer;
    if (tot > 0) cat_launch<false>(a, out, row, tot);
  }
  LH_CHECK_LAUNCH();
}
void lh_concat_grad_beta(int n, float* const* h_ind, const float* h_beta, const int* sizes, const float* outd, int outer, int inner) {
  int64_t row = 0; for (int t = 0; t < n; t++) row += (int64_t)sizes[t] * inner;
  for (int t = 0; t < n && h_beta; t++) LH_REQUIRE(h_beta[t] == 0.f || h_beta[t] == 1.f, "lh_concat_grad_beta: beta must be 0 or 1");
  LZ_ENTER(); lazy::rd_f(outd, row * outer);
  int64_t off = 0;
  for (int t0 = 0; t0 < n; t0 += CAT_MAX) {
    CatArgs a{}; a.n = n - t0 < CAT_MAX ? n - t0 : CAT_MAX; a.lo = off;
    bool any = false;
    for (int u = 0; u < a.n; u++) {
      const int t = t0 + u;
      a.p[u] = h_ind[t]; a.st[u] = (int64_t)sizes[t] * inner; a.off[u] = off; off += a.st[u];
      if (a.p[u] && a.st[u] > 0) { a.add[u] = lazy::beta_f(a.p[u], a.st[u] * outer, h_beta ? h_beta[t] : 1.f) != 0.f; any = true; }
    }
    a.width = off - a.lo;
    const int64_t tot = a.width * outer;
    if (tot > 0 && any) cat_launch<true>(a, const_cast<float*>(outd), row, tot);
  }
  LH_CHECK_LAUNCH();
}
void lh_concat_grad(int n, float* const* h_ind, const int* sizes, const float* outd, int outer, int inner) {
  lh_concat_grad_beta(n, h_ind, nullptr, sizes, outd, outer, inner);
}

}  // extern "C"

// ---------------------------------------------------------------- optimizers ----------
namespace {
__device__ __forceinline__ void momentum_elem(float& x, float& d, float& v, float lr, float mu, float clip, int nesterov) {
  float t = d;
  if (t > clip) t = clip;
  if (t < -clip) t = -clip;
  float vv = v * mu; vv += t;
  if (nesterov) t += mu * vv; else t = vv;
  x -= lr * t; v = vv; d = 0.f;
}
__global__ void __launch_bounds__(TPB) k_momentum(float* x, float* d, float* v, float lr, float mu, float clip, int nesterov, int64_t n) {
  int64_t n4 = n >> 2;
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (int64_t j = i; j < n4; j += st) {
    float4 X = reinterpret_cast<float4*>(x)[j], D = reinterpret_cast<float4*>(d)[j], V = reinterpret_cast<float4*>(v)[j];
    momentum_elem(X.x, D.x, V.x, lr, mu, clip, nesterov); momentum_elem(X.y, D.y, V.y, lr, mu, clip, nesterov);
    momentum_elem(X.z, D.z, V.z, lr, mu, clip, nesterov); momentum_elem(X.w, D.w, V.w, lr, mu, clip, nesterov);
    reinterpret_cast<float4*>(x)[j] = X; reinterpret_cast<float4*>(d)[j] = D; reinterpret_cast<float4*>(v)[j] = V;
  }
  for (int64_t j = 4 * n4 + i; j < n; j += st) momentum_elem(x[j], d[j], v[j], lr, mu, clip, nesterov);
}
__global__ void __launch_bounds__(TPB) k_adagrad(float* x, float* d, float* m, float lr, float clip, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n; i += st) {
    float t = d[i];
    if (t > clip) t = clip;
    if (t < -clip) t = -clip;
    float mm = m[i] + t * t;
    m[i] = mm;
    x[i] -= lr * t / sqrtf(mm + 1e-8f);
    d[i] = 0.f;
  }
}
__global__ void __launch_bounds__(TPB) k_sgd(float* x, float* d, float lr, int64_t n) {
  int64_t n4 = n >> 2;
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (int64_t j = i; j < n4; j += st) {
    float4 X = reinterpret_cast<float4*>(x)[j], D = reinterpret_cast<float4*>(d)[j];
    X.x = X.x * 1.0f + D.x * (-lr); X.y = X.y * 1.0f + D.y * (-lr); X.z = X.z * 1.0f + D.z * (-lr); X.w = X.w * 1.0f + D.w * (-lr);
    reinterpret_cast<float4*>(x)[j] = X; reinterpret_cast<float4*>(d)[j] = make_float4(0.f, 0.f, 0.f, 0.f);
  }
  for (int64_t j = 4 * n4 + i; j < n; j += st) { x[j] = x[j] * 1.0f + d[j] * (-lr); d[j] = 0.f; }
}

// Multi-tensor form: a table of (x, d, v, first chunk) per tensor lives in device memory;
// block b finds its tensor by binary search over chunk starts.  Chunk = 4096 elements.
constexpr int MT_CHUNK = 4096;
struct MtEntry { float* x; float* d; float* v; int64_t n; int64_t chunk0; };
__global__ void __launch_bounds__(TPB) k_multi_update(const MtEntry* tab, int count, int mode, float lr, float mu, float clip, int nesterov) {
  int64_t b = blockIdx.x;
  int lo = 0, hi = count - 1;
  while (lo < hi) { int mid = (lo + hi + 1) >> 1; if (tab[mid].chunk0 <= b) lo = mid; else hi = mid - 1; }
  MtEntry e = tab[lo];
  int64_t start = (b - e.chunk0) * MT_CHUNK, end = start + MT_CHUNK; if (end > e.n) end = e.n;
  for (int64_t j = start + threadIdx.x; j < end; j += TPB) {
    if (mode == 0) { e.x[j] = e.x[j] * 1.0f + e.d[j] * (-lr); e.d[j] = 0.f; }
    else momentum_elem(e.x[j], e.d[j], e.v[j], lr, mu, clip, nesterov);
  }
}
// The device-side table is cached per distinct host table (same pointers => same step plan).  Its memory is reserved by
// lh_setup (MT_TABLE_MAX entries), so no operator call allocates.
constexpr int MT_TABLE_MAX = 65536;
struct MtCache { MtEntry* dev = nullptr; int count = 0; int64_t chunks = 0; uint64_t key = 0; };
static MtCache g_mt;
static uint64_t mt_key(int mode, int count, float* const* hx, float* const* hd, float* const* hv, const int64_t* hn) {
  uint64_t key = 1469598103934665603ULL;
  auto mix = [&key](uint64_t v) { key = (key ^ v) * 1099511628211ULL; };
  for (int t = 0; t < count; t++) { mix((uint64_t)(uintptr_t)hx[t]); mix((uint64_t)(uintptr_t)hd[t]); mix(hv ? (uint64_t)(uintptr_t)hv[t] : 0); mix((uint64_t)hn[t]); }
  mix((uint64_t)mode);
  return key;
}
static void multi_update(int mode, int count, float* const* hx, float* const* hd, float* const* hv, const int64_t* hn,
                         float lr, float mu, float clip, int nesterov) {
  if (count <= 0) return;
  LH_REQUIRE(g_mt.dev != nullptr, "multi-tensor update before lh_setup");
  LH_REQUIRE(count <= MT_TABLE_MAX, "multi-tensor update over %d tensors (at most %d)", count, MT_TABLE_MAX);
  const uint64_t key = mt_key(mode, count, hx, hd, hv, hn);
  if (g_mt.count == 0 || g_mt.key != key || g_mt.count != count) {
    LH_NOT_CAPTURING("the first multi-tensor update of a parameter set (its table is uploaded)");
    MtEntry* host = (MtEntry*)malloc(sizeof(MtEntry) * count);
    LH_REQUIRE(host != nullptr, "multi-tensor table: out of host memory");
    int64_t chunks = 0;
    for (int t = 0; t < count; t++) { host[t] = {hx[t], hd[t], hv ? hv[t] : nullptr, hn[t], chunks}; chunks += cdiv(hn[t] > 0 ? hn[t] : 1, MT_CHUNK); }
    hipError_t e = hipMemcpyAsync(g_mt.dev, host, sizeof(MtEntry) * count, hipMemcpyHostToDevice, g_stream);
    if (e == hipSuccess) e = hipStreamSynchronize(g_stream);
    free(host);
    if (e != hipSuccess) { LH_FAIL("multi-tensor table upload: %s", hipGetErrorString(e)); return; }
    g_mt.key = key; g_mt.count = count; g_mt.chunks = chunks;
  }
  LH_REQUIRE(g_mt.chunks > 0 && g_mt.chunks < 0x7fffffffLL, "multi-tensor update: %lld chunks", (long long)g_mt.chunks);
  hipLaunchKernelGGL(k_multi_update, dim3((unsigned)g_mt.chunks), dim3(TPB), 0, g_stream, (const MtEntry*)g_mt.dev, count, mode, lr, mu, clip, nesterov);
}
// ---- the same update for callers that cannot allocate ----------------------------------------------------------
// The table lives in a fixed device array; it is written by small kernels that receive the entries as launch
// arguments (no host-to-device copy, so nothing waits for the device and nothing is staged).
constexpr int MT_STATIC_MAX = 4096;                 // tensors per call
constexpr int MT_ARGS = 64;                         // table entries one writer launch carries
static __device__ __align__(256) unsigned char scratch[MT_STATIC_MAX * sizeof(MtEntry)];   // 160 KiB per GPU, held until the process ends
struct MtArgs { MtEntry e[MT_ARGS]; };
__global__ void __launch_bounds__(MT_ARGS) k_mt_table_write(MtEntry* tab, const MtArgs a, int first, int n) {
  const int i = threadIdx.x;
  if (i < n) tab[first + i] = a.e[i];
}
constexpr int MT_MAX_DEVICES = 16;
struct MtStatic { MtEntry* ptr = nullptr; };
static MtStatic g_mt_static[MT_MAX_DEVICES];
// The array's address on the current device (looked up once per device: every GPU holds its own copy).
static MtStatic* mt_static_state() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MT_MAX_DEVICES) { LH_FAIL("lh_multi_momentum_static: no current device below %d", MT_MAX_DEVICES); return nullptr; }
  MtStatic* st = &g_mt_static[dev];
  if (st->ptr == nullptr) {
    void* p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) { LH_FAIL("lh_multi_momentum_static: address of the table array: %s", hipGetErrorString(e)); return nullptr; }
    st->ptr = (MtEntry*)p;
  }
  return st;
}
// The table is written on every call: a host-side note of what the array holds would be wrong as soon as a recorded graph
// that contains table writes is replayed (it rewrites the array behind the note's back), and a call recorded into a graph
// must carry its own writes.  At most count / 64 launches of one workgroup each.
static void multi_update_static(int mode, int count, float* const* h_x, float* const* h_d, float* const* h_v, const int64_t* h_n,
                                float lr, float mu, float clip, int nesterov) {
  if (count <= 0) return;
  LH_REQUIRE(count <= MT_STATIC_MAX, "lh_multi_momentum_static: %d tensors, the fixed table holds at most %d (lh_multi_momentum has no such limit)", count, MT_STATIC_MAX);
  LH_REQUIRE(h_x && h_d && h_n, "lh_multi_momentum_static: null pointer table");
  int64_t chunks = 0;
  for (int t = 0; t < count; t++) {
    LH_REQUIRE(h_n[t] >= 0 && (h_n[t] == 0 || (h_x[t] && h_d[t] && (h_v == nullptr || h_v[t]))), "lh_multi_momentum_static: tensor %d has a null pointer or a negative size", t);
    chunks += cdiv(h_n[t] > 0 ? h_n[t] : 1, MT_CHUNK);
  }
  LH_REQUIRE(chunks < 0x7fffffffLL, "lh_multi_momentum_static: %lld chunks of %d elements exceed one launch", (long long)chunks, MT_CHUNK);
  MtStatic* st = mt_static_state();
  if (st == nullptr) return;
  int64_t c0 = 0;
  for (int first = 0; first < count; first += MT_ARGS) {      // entries beyond `count` left by an earlier, larger call are never read
    MtArgs a;
    const int n = count - first < MT_ARGS ? count - first : MT_ARGS;
    for (int i = 0; i < MT_ARGS; i++) {
      if (i < n) { const int t = first + i; a.e[i] = {h_x[t], h_d[t], h_v ? h_v[t] : nullptr, h_n[t], c0}; c0 += cdiv(h_n[t] > 0 ? h_n[t] : 1, MT_CHUNK); }
      else a.e[i] = {nullptr, nullptr, nullptr, 0, 0};
    }
    hipLaunchKernelGGL(k_mt_table_write, dim3(1), dim3(MT_ARGS), 0, g_stream, st->ptr, a, first, n);
  }
  hipLaunchKernelGGL(k_multi_update, dim3((unsigned)chunks), dim3(TPB), 0, g_stream, (const MtEntry*)st->ptr, count, mode, lr, mu, clip, nesterov);
  LH_CHECK_LAUNCH();
}
}  // namespace

namespace lh {
bool multi_tensor_setup() {
  g_mt = MtCache();
  if (hipMalloc((void**)&g_mt.dev, sizeof(MtEntry) * MT_TABLE_MAX) != hipSuccess) { g_mt.dev = nullptr; LH_FAIL("multi-tensor table allocation failed"); return false; }
  for (auto& st : g_mt_static) st = MtStatic();       // a fresh stream after lh_setup: no table written on it yet
  return mt_static_state() != nullptr;                // the fixed table's address on this device
}
void multi_tensor_release() { if (g_mt.dev) (void)hipFree(g_mt.dev); g_mt = MtCache(); }
// what lh_defer.hip launches for work it had put off
void mask_relu(float* dst, const float* src, const float* y, int64_t n) { ProfScope prof_(CAT_ELEMENTWISE);
  ew<2>(dst, src, y, nullptr, n, [] __device__(float d, float yv, float) { return yv > 0.f ? d : 0.f; });
}
void add_plain(const float* a, const float* b, float* out, int64_t n) { ProfScope prof_(CAT_ELEMENTWISE);
  ew<2>(out, a, b, nullptr, n, [] __device__(float x, float y, float) { return x + y; });
}
void relu_grad_inplace_now(const float* y, float* d, int64_t n) { ProfScope prof_(CAT_ELEMENTWISE);
  ew<2>(d, d, y, nullptr, n, [] __device__(float g, float yv, float) { return yv > 0.f ? g : 0.f; });
}
void multi_update_now(int mode, int count, float* const* hx, float* const* hd, float* const* hv, const int64_t* hn, float lr, float mu, float clip, int nesterov) {
  ProfScope prof_(CAT_OPTIM);
  // while a graph is recorded the table cannot be uploaded (a copy that waits): the kernel-written table serves
  if (g_capturing && count <= MT_STATIC_MAX) multi_update_static(mode, count, hx, hd, hv, hn, lr, mu, clip, nesterov);
  else multi_update(mode, count, hx, hd, hv, hn, lr, mu, clip, nesterov);
}
}  // namespace lh

extern "C" {
void lh_sgd(float* x, float* d, float lr, int64_t n) {
  LZ_SCOPE();
  side_join();      // parameter gradients may still be in flight on the side stream
  if (n <= 0) return;
  LH_REQUIRE(al16(x) && al16(d), "lh_sgd: pointers must be 16-byte aligned");
  if (lazy::gather_update(0, x, d, nullptr, lr, 0.f, 0.f, 0, n)) return;     // one launch for a run of these calls
  if (lazy::g_busy && !lazy::g_replay) { lazy::flush_parked(); lazy::forget_forward_records(); lazy::rw_f(x, n); lazy::rw_f(d, n); }
  ProfScope prof_(CAT_OPTIM);
  if (rec_ok(n)) { rec_cmd(CL_SGD, (int)n, 0, 0, lr, 0.f, 0.f, 0.f, x, d, nullptr, nullptr); return; }
  hipLaunchKernelGGL(k_sgd, dim3(stream_grid(n, TPB * 8)), dim3(TPB), 0, g_stream, x, d, lr, n);
  LH_CHECK_LAUNCH();
}
void lh_momentum(float* x, float* d, float* v, float lr, float mu, float clip, int nesterov, int64_t n) {
  LZ_SCOPE();
  side_join();      // parameter gradients may still be in flight on the side stream
  if (n <= 0) return;
  LH_REQUIRE(al16(x) && al16(d) && al16(v), "lh_momentum: pointers must be 16-byte aligned");
  if (lazy::gather_update(1, x, d, v, lr, mu, clip, nesterov, n)) return;    // one launch for a run of these calls (NNModule.scala:296-303 issues one per parameter)
  if (lazy::g_busy && !lazy::g_replay) { lazy::flush_parked(); lazy::forget_forward_records(); lazy::rw_f(x, n); lazy::rw_f(d, n); lazy::rw_f(v, n); }
  ProfScope prof_(CAT_OPTIM);
  hipLaunchKernelGGL(k_momentum, dim3(stream_grid(n, TPB * 8)), dim3(TPB), 0, g_stream, x, d, v, lr, mu, clip, nesterov, n);
  LH_CHECK_LAUNCH();
}
void lh_adagrad(float* x, float* d, float* m, float lr, float clip, int64_t n) {
  LZ_ENTER(); lazy::forget_forward_records(); lazy::rw_f(x, n); lazy::rw_f(d, n); lazy::rw_f(m, n);
  ProfScope prof_(CAT_OPTIM);
  side_join();      // parameter gradients may still be in flight on the side stream
  if (n <= 0) return;
  if (rec_ok(n)) { rec_cmd(CL_ADAGRAD, (int)n, 0, 0, lr, clip, 0.f, 0.f, x, d, m, nullptr); return; }
  hipLaunchKernelGGL(k_adagrad, dim3(stream_grid(n, TPB * 4)), dim3(TPB), 0, g_stream, x, d, m, lr, clip, n);
  LH_CHECK_LAUNCH();
}
void lh_multi_momentum(int count, float* const* h_x, float* const* h_d, float* const* h_v, const int64_t* h_n,
                       float lr, float mu, float clip, int nesterov) {
  LZ_ENTER(); lazy::forget_forward_records();
  for (int t = 0; t < count && lazy::g_busy; t++) { lazy::rw_f(h_x[t], h_n[t]); lazy::rw_f(h_d[t], h_n[t]); lazy::rw_f(h_v[t], h_n[t]); }
  ProfScope prof_(CAT_OPTIM);
  side_join();      // parameter gradients may still be in flight on the side stream
  multi_update(1, count, h_x, h_d, h_v, h_n, lr, mu, clip, nesterov);
  if (!failed()) LH_CHECK_LAUNCH();
}
void lh_multi_momentum_static(int count, float* const* h_x, float* const* h_d, float* const* h_v, const int64_t* h_n,
                              float lr, float mu, float clip, int nesterov) {
  LZ_ENTER(); lazy::forget_forward_records();
  for (int t = 0; t < count && lazy::g_busy && h_x && h_d && h_v && h_n; t++) { lazy::rw_f(h_x[t], h_n[t]); lazy::rw_f(h_d[t], h_n[t]); lazy::rw_f(h_v[t], h_n[t]); }
  ProfScope prof_(CAT_OPTIM);
  side_join();      // parameter gradients may still be in flight on the side stream
  LH_REQUIRE(count <= 0 || h_v != nullptr, "lh_multi_momentum_static: null pointer table");
  multi_update_static(1, count, h_x, h_d, h_v, h_n, lr, mu, clip, nesterov);
}
void lh_multi_sgd(int count, float* const* h_x, float* const* h_d, const int64_t* h_n, float lr) {
  LZ_ENTER(); lazy::forget_forward_records();
  for (int t = 0; t < count && lazy::g_busy; t++) { lazy::rw_f(h_x[t], h_n[t]); lazy::rw_f(h_d[t], h_n[t]); }
  ProfScope prof_(CAT_OPTIM);
  side_join();      // parameter gradients may still be in flight on the side stream
  multi_update(0, count, h_x, h_d, nullptr, h_n, lr, 0.f, 0.f, 0);
  if (!failed()) LH_CHECK_LAUNCH();
}
}  // extern "C"
