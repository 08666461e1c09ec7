// Command list: small operations recorded on the host and executed, in order, by one 1024-thread workgroup.
//
// A model built from 150-element vectors (the sentiment TreeLSTM: ~5000 operator calls per tree) is bound by the
// host's kernel-launch rate (about 3 us per launch), not by the device.  Between lh_cmdlist_begin() and
// lh_cmdlist_end() every entry point whose operands are small appends a 64-byte command to a pinned host buffer
// instead of launching; the buffer is handed to k_cmdlist when it is full, when recording ends, or when any other
// entry point is about to use the stream (lh::ordered_stream), so the program order of all operations is kept.
// One workgroup runs the commands one after the other with a block barrier between them: every command sees the
// global-memory results of the ones before it (same compute unit, same L1), and no other kernel runs in between.
// The arithmetic of each command follows the stand-alone kernel of the same operation.
#include "lh_common.h"
using namespace lh;

namespace lh {
int g_rec_on = 0;
int g_rec_pending = 0;
}

namespace {
constexpr int CL_THREADS = 1024;
constexpr int CL_CHUNK = 256;                 // commands staged in LDS at a time
constexpr int CL_BUF_CMDS = 256;              // commands per host buffer: a full buffer is launched while the host records the next
constexpr int CL_NBUF = 32;

struct Ring {
  LhCmd* host[CL_NBUF]; LhCmd* dev[CL_NBUF]; hipEvent_t done[CL_NBUF]; bool busy[CL_NBUF];
  int cur; bool ready;
  int64_t recorded, launches;
};
static Ring g_ring = {};

__device__ __forceinline__ float cl_bop(int op, float a, float b) {
  switch (op) { case LH_ADD: return a + b; case LH_SUB: return a - b; case LH_MUL: return a * b; default: return a / b; }
}
__device__ __forceinline__ float cl_unary(int op, float v, float lo, float hi) {
  switch (op) {
    case LH_RELU: return v < 0.f ? 0.f : v;
    case LH_TANH: return tanhf(v);
    case LH_SIGMOID: return 1.0f / (expf(-v) + 1.0f);
    case LH_EXP: return expf(v);
    case LH_LOG: return logf(v);
    case LH_SQRT: return sqrtf(v);
    case LH_SQUARE: return v * v;
    default: return v < lo ? lo : (v > hi ? hi : v);        // LH_HARDTANH
  }
}
// dx (+)= g(x | y, dy) exactly as lh_unary_grad's kernels
__device__ __forceinline__ float cl_unary_grad(int op, int inplace, float d, float xv, float yv, float g, float lo, float hi) {
  switch (op) {
    case LH_RELU: return inplace ? (yv > 0.f ? d : 0.f) : d + (xv < 0.f ? 0.f : g);
    case LH_HARDTANH: return inplace ? ((yv > lo && yv < hi) ? d : 0.f) : d + ((xv < lo || xv > hi) ? 0.f : g);
    case LH_TANH: return d + (1.0f - yv * yv) * g;
    case LH_SIGMOID: return d + ((1.0f - yv) * yv) * g;
    case LH_EXP: return d + g * yv;
    case LH_LOG: return d + g / xv;
    case LH_SQRT: return d + g / yv / 2.0f;
    default: return d + g * xv * 2.0f;                         // LH_SQUARE
  }
}
__device__ __forceinline__ float cl_wave_sum_all(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float cl_wave_max_all(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// Data pointers carry no __restrict__ and no const: a command may read what the command before it wrote.
__device__ void cl_run(const LhCmd& c, float* red /* [4][257] */) {
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  constexpr int NT = CL_THREADS, NW = CL_THREADS / 64;
  float* p0 = (float*)c.p0; float* p1 = (float*)c.p1; float* p2 = (float*)c.p2; float* p3 = (float*)c.p3;
  switch (c.op) {
    case CL_ZERO16: { uint4* p = (uint4*)c.p0; const int n = c.i0; for (int i = t; i < n; i += NT) p[i] = make_uint4(0, 0, 0, 0); break; }
    case CL_FILL: { const int n = c.i0; const float v = c.f0; for (int i = t; i < n; i += NT) p0[i] = v; break; }
    case CL_COPY: { const int n = c.i0; for (int i = t; i < n; i += NT) p0[i] = p1[i]; break; }
    case CL_GEAM: { const int n = c.i0; const float al = c.f0, be = c.f1; for (int i = t; i < n; i += NT) p0[i] = p1[i] * al + p2[i] * be; break; }
    case CL_SCALAR: { const int n = c.i0, op = c.i1; const float s = c.f0; for (int i = t; i < n; i += NT) p0[i] = cl_bop(op, p1[i], s); break; }
    case CL_BIN: { const int n = c.i0, op = c.i1; for (int i = t; i < n; i += NT) p0[i] = cl_bop(op, p1[i], p2[i]); break; }
    case CL_ACC: { const int n = c.i0; for (int i = t; i < n; i += NT) p0[i] = p0[i] + p1[i]; break; }
    case CL_ACCNEG: { const int n = c.i0; for (int i = t; i < n; i += NT) p0[i] = p0[i] + (0.0f - p1[i]); break; }
    case CL_ACCMUL: { const int n = c.i0; for (int i = t; i < n; i += NT) p0[i] = p0[i] + p1[i] * p2[i]; break; }
    case CL_UNARY: { const int n = c.i0, op = c.i1; const float lo = c.f0, hi = c.f1; for (int i = t; i < n; i += NT) p0[i] = cl_unary(op, p1[i], lo, hi); break; }
    case CL_UNARY_GRAD: {        // p0 = dx, p1 = x, p2 = y, p3 = dy
      const int n = c.i0, op = c.i1, inplace = c.i2; const float lo = c.f0, hi = c.f1;
      const bool need_x = (op == LH_RELU || op == LH_HARDTANH) ? !inplace : (op == LH_LOG || op == LH_SQUARE);
      const bool need_y = (op == LH_RELU || op == LH_HARDTANH) ? inplace != 0 : !(op == LH_LOG || op == LH_SQUARE);
      const bool need_g = !((op == LH_RELU || op == LH_HARDTANH) && inplace);
      for (int i = t; i < n; i += NT)
        p0[i] = cl_unary_grad(op, inplace, p0[i], need_x ? p1[i] : 0.f, need_y ? p2[i] : 0.f, need_g ? p3[i] : 0.f, lo, hi);
      break;
    }
    case CL_GEMV_N: {            // y[m] = alpha * A[m,n] x[n] + beta * y   (p0 = y, p1 = A, p2 = x; i2 = lda): a wavefront per row,
      // four rows at a time so that their loads are in flight together (a store to y ends a batch, not every row)
      const int m = c.i0, n = c.i1, lda = c.i2; const float al = c.f0, be = c.f1;
      for (int r0 = wave * 4; r0 < m; r0 += NW * 4) {
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        for (int j = lane; j < n; j += 64) {
          const float xv = p2[j];
#pragma unroll
          for (int u = 0; u < 4; u++) acc[u] += (r0 + u < m ? p1[(int64_t)(r0 + u) * lda + j] : 0.f) * xv;
        }
#pragma unroll
        for (int u = 0; u < 4; u++) acc[u] = cl_wave_sum_all(acc[u]);
        if (lane < 4 && r0 + lane < m) {
          const float s = lane == 0 ? acc[0] : (lane == 1 ? acc[1] : (lane == 2 ? acc[2] : acc[3]));
          p0[r0 + lane] = al * s + (be == 0.f ? 0.f : be * p0[r0 + lane]);
        }
      }
      break;
    }
    case CL_GEMV_T: {            // y[n] = alpha * A[m,n]^T x[m] + beta * y  (p0 = y, p1 = A, p2 = x): 256 columns x 4 row groups per pass
      const int m = c.i0, n = c.i1, lda = c.i2; const float al = c.f0, be = c.f1;
      const int col = t & 255, g = t >> 8;
      for (int j0 = 0; j0 < n; j0 += 256) {
        const int j = j0 + col;
        float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
        if (j < n) {
          int i = g;
          for (; i + 12 < m; i += 16) {
            a0 += p1[(int64_t)i * lda + j] * p2[i];
            a1 += p1[(int64_t)(i + 4) * lda + j] * p2[i + 4];
            a2 += p1[(int64_t)(i + 8) * lda + j] * p2[i + 8];
            a3 += p1[(int64_t)(i + 12) * lda + j] * p2[i + 12];
          }
          for (; i < m; i += 4) a0 += p1[(int64_t)i * lda + j] * p2[i];
        }
        red[g * 257 + col] = (a0 + a1) + (a2 + a3);
        __syncthreads();
        if (g == 0 && j < n) {
          const float s = (red[col] + red[257 + col]) + (red[2 * 257 + col] + red[3 * 257 + col]);
          p0[j] = al * s + (be == 0.f ? 0.f : be * p0[j]);
        }
        __syncthreads();
      }
      break;
    }
    case CL_GER: {               // A[m,n] += u[m] (x) v[n]   (p0 = A, p1 = u, p2 = v): four elements per thread and pass, loads first
      const int m = c.i0, n = c.i1, tot = m * n;
      for (int i0 = t; i0 < tot; i0 += 4 * NT) {
        float a[4], w[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
          const int i = i0 + u * NT;
          const bool ok = i < tot;
          const int r = ok ? i / n : 0, cc = ok ? i - r * n : 0;
          a[u] = ok ? p0[i] : 0.f;
          w[u] = p2[cc] * p1[r];
        }
#pragma unroll
        for (int u = 0; u < 4; u++) { const int i = i0 + u * NT; if (i < tot) p0[i] = a[u] + w[u]; }
      }
      break;
    }
    case CL_DOT: {               // out[0] = x . y   (p0 = out, p1 = x, p2 = y)
      const int n = c.i0;
      float acc = 0.f;
      for (int i = t; i < n; i += NT) acc += p1[i] * p2[i];
      acc = cl_wave_sum_all(acc);
      if (lane == 0) red[wave] = acc;
      __syncthreads();
      if (wave == 0) { float v = lane < NW ? red[lane] : 0.f; v = cl_wave_sum_all(v); if (lane == 0) p0[0] = v; }
      break;
    }
    case CL_AXPY_DEV: {          // y += s[0] * x   (p0 = y, p1 = s, p2 = x)
      const int n = c.i0;
      const float a = *(volatile float*)p1;                 // written by an earlier command: a vector load, not the scalar cache
      for (int i = t; i < n; i += NT) p0[i] = p0[i] + a * p2[i];
      break;
    }
    case CL_SOFTMAX: {           // rows of length cc, a wavefront per row   (p0 = y, p1 = x; i2 = log form)
      const int rows = c.i0, cc = c.i1, is_log = c.i2;
      for (int r = wave; r < rows; r += NW) {
        const float* xp = p1 + (int64_t)r * cc; float* yp = p0 + (int64_t)r * cc;
        float mx = -3.402823466e+38f;
        for (int j = lane; j < cc; j += 64) mx = fmaxf(mx, xp[j]);
        mx = cl_wave_max_all(mx);
        float sum = 0.f;
        for (int j = lane; j < cc; j += 64) sum += expf(xp[j] - mx);
        sum = cl_wave_sum_all(sum);
        if (is_log) { const float ls = mx + logf(sum); for (int j = lane; j < cc; j += 64) yp[j] = xp[j] - ls; }
        else { for (int j = lane; j < cc; j += 64) yp[j] = expf(xp[j] - mx) / sum; }
      }
      break;
    }
    case CL_SOFTMAX_GRAD: {      // p0 = dx (accumulates), p1 = y, p2 = dy; rows of length cc
      const int rows = c.i0, cc = c.i1, is_log = c.i2;
      for (int r = wave; r < rows; r += NW) {
        const int64_t base = (int64_t)r * cc;
        float acc = 0.f;
        for (int j = lane; j < cc; j += 64) acc += is_log ? p2[base + j] : p2[base + j] * p1[base + j];
        acc = cl_wave_sum_all(acc);
        for (int j = lane; j < cc; j += 64) {
          const int64_t i = base + j;
          p0[i] += is_log ? p2[i] - expf(p1[i]) * acc : p1[i] * (p2[i] - acc);
        }
      }
      break;
    }
    case CL_NLL: {               // y[b] = -x[b*stride + target[b]]   (p0 = y, p1 = x, p2 = target)
      const int batch = c.i0, stride = c.i1; const int* tg = (const int*)c.p2;
      for (int b = t; b < batch; b += NT) p0[b] = -1.0f * p1[(int64_t)b * stride + tg[b]];
      break;
    }
    case CL_NLL_GRAD: {          // dx[b*stride + target[b]] += -dy[b]   (p0 = dx, p1 = dy, p2 = target)
      const int batch = c.i0, stride = c.i1; const int* tg = (const int*)c.p2;
      for (int b = t; b < batch; b += NT) p0[(int64_t)b * stride + tg[b]] += -1.0f * p1[b];
      break;
    }
    case CL_ADAGRAD: {           // p0 = x, p1 = d, p2 = m
      const int n = c.i0; const float lr = c.f0, clip = c.f1;
      for (int i = t; i < n; i += NT) {
        float g = p1[i];
        if (g > clip) g = clip;
        if (g < -clip) g = -clip;
        const float mm = p2[i] + g * g;
        p2[i] = mm;
        p0[i] -= lr * g / sqrtf(mm + 1e-8f);
        p1[i] = 0.f;
      }
      break;
    }
    case CL_SGD: {               // p0 = x, p1 = d
      const int n = c.i0; const float lr = c.f0;
      for (int i = t; i < n; i += NT) { p0[i] = p0[i] * 1.0f + p1[i] * (-lr); p1[i] = 0.f; }
      break;
    }
    default: break;
  }
}

// cmds: pinned host memory (read over the host link, a chunk at a time, the next chunk fetched while the current one runs).
__global__ void __launch_bounds__(CL_THREADS) k_cmdlist(const LhCmd* cmds, int n) {
  __shared__ uint4 stage[CL_CHUNK * 4];                 // 256 commands of 64 bytes
  __shared__ float red[4 * 257];
  const int t = threadIdx.x;
  const uint4* src = reinterpret_cast<const uint4*>(cmds);
  const int total16 = n * 4;
  uint4 next = make_uint4(0, 0, 0, 0);
  if (t < total16) next = src[t];
  for (int base = 0; base < n; base += CL_CHUNK) {
    stage[t] = next;
    const int nb = base + CL_CHUNK;
    if (nb < n && nb * 4 + t < total16) next = src[nb * 4 + t];
    __syncthreads();
    const int cnt = n - base < CL_CHUNK ? n - base : CL_CHUNK;
    const LhCmd* list = reinterpret_cast<const LhCmd*>(stage);
    for (int i = 0; i < cnt; i++) {
      cl_run(list[i], red);
      __syncthreads();
    }
  }
}

static bool ring_init() {
  if (g_ring.ready) return true;
  for (int i = 0; i < CL_NBUF; i++) {
    if (hipHostMalloc((void**)&g_ring.host[i], sizeof(LhCmd) * CL_BUF_CMDS, hipHostMallocDefault) != hipSuccess) { LH_FAIL("command list: pinned buffer allocation failed"); return false; }
    if (hipHostGetDevicePointer((void**)&g_ring.dev[i], g_ring.host[i], 0) != hipSuccess) { LH_FAIL("command list: pinned buffer has no device address"); return false; }
    if (hipEventCreateWithFlags(&g_ring.done[i], hipEventDisableTiming) != hipSuccess) { LH_FAIL("command list: event creation failed"); return false; }
    g_ring.busy[i] = false;
  }
  g_ring.cur = 0; g_ring.ready = true;
  return true;
}
}  // namespace

namespace lh {
void rec_flush() {
  const int n = g_rec_pending;
  if (n <= 0) return;
  g_rec_pending = 0;                                  // before any use of the stream below
  Ring& r = g_ring;
  ProfScope prof_(CAT_CMDLIST);
  hipLaunchKernelGGL(k_cmdlist, dim3(1), dim3(CL_THREADS), 0, g_stream_raw, (const LhCmd*)r.dev[r.cur], n);
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) e = hipEventRecord(r.done[r.cur], g_stream_raw);
  if (e != hipSuccess) { LH_FAIL("command list launch: %s", hipGetErrorString(e)); return; }
  r.busy[r.cur] = true;
  r.launches++;
  r.cur = (r.cur + 1) % CL_NBUF;
  if (r.busy[r.cur]) {                                // the buffer about to be refilled must have been consumed
    (void)hipEventSynchronize(r.done[r.cur]);
    r.busy[r.cur] = false;
  }
}
LhCmd* rec_next() {
  if (!g_ring.ready) return nullptr;
  if (g_rec_pending == CL_BUF_CMDS) { rec_flush(); if (failed()) return nullptr; }
  g_ring.recorded++;
  return &g_ring.host[g_ring.cur][g_rec_pending++];
}
void cmdlist_release() {
  g_rec_on = 0; g_rec_pending = 0;
  if (!g_ring.ready) return;
  for (int i = 0; i < CL_NBUF; i++) { (void)hipEventDestroy(g_ring.done[i]); (void)hipHostFree(g_ring.host[i]); }
  g_ring = Ring{};
}
}  // namespace lh

extern "C" {
void lh_cmdlist_begin(void) {
  LH_REQUIRE(g_stream_raw != nullptr, "lh_cmdlist_begin before lh_setup");
  LH_REQUIRE(!g_capturing, "lh_cmdlist_begin: a graph is being recorded (the command buffers cannot be replayed)");
  LH_REQUIRE(g_stream_cur == g_stream_raw, "lh_cmdlist_begin on the side stream");
  if (!ring_init()) return;
  g_rec_on = 1;
}
void lh_cmdlist_end(void) {
  rec_flush();
  g_rec_on = 0;
}
void lh_cmdlist_stats(int64_t* recorded, int64_t* launches) {
  if (recorded) *recorded = g_ring.recorded;
  if (launches) *launches = g_ring.launches;
}
}  // extern "C"
