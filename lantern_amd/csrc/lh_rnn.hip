// Elman RNN layer (tanh / relu, optionally bidirectional) forward and backward, and the CTC loss.
// Reference behaviour being replaced: RNNBase (NNModule.scala:332-417) over cudnnRNNForwardTraining /
// cudnnRNNBackwardData / cudnnRNNBackwardWeights (CDN:1638-1893), and cudnnCTCLoss (CDN:1895-1938).
//
//   h_t = act(W_ih x_t + b_ih + W_hh h_{t-1} + b_hh),  h_{-1} = 0,   y[t,b,:] = [h_t forward ; h_t reverse]
//
// The input projection of all time steps and the three weight/input gradients are large GEMMs
// (lh_sgemm, MFMA).  Only the recurrence is sequential: one small kernel per time step, both
// directions in the same launch.  For aligned operands a block produces 16 hidden units for 16 batch rows
// on the matrix pipes (lh_rnn_tile.h); otherwise 4-16 hidden units for the whole batch from W_hh rows held
// in registers (the vector form).  The output y doubles as the saved hidden states.
#include "lh_common.h"
#include "lh_rnn_tile.h"
#include "../../include/lantern_hip.h"
using namespace lh;

namespace {
constexpr int TPB = 256;

__device__ __forceinline__ float act_fwd(int mode, float v) { return mode == 1 ? tanhf(v) : (v < 0.f ? 0.f : v); }

// Shared shape of both step kernels: out[b, j] = sum_k in[b, k] * Wrow[j, k] for the JC rows j0.. of this
// block and every batch row b.  A lane owns NK values of k (V4: groups of four consecutive ones, k = 256 q + 4 lane + r,
// fetched as one 16-byte load; otherwise k = lane + 64 i); the JC x NK weights it needs stay in registers for the
// whole step.  The four wavefronts of a block take every fourth group of batch rows, a few rows at a time, and the
// loads of the next group are issued before the sums of the current one are reduced.
template <int NK, bool V4>
__device__ __forceinline__ void rnn_load_row(const float* __restrict__ row, int H, bool use, float (&r)[NK]) {
  const int lane = threadIdx.x & 63;
  if (V4) {
#pragma unroll
    for (int q = 0; q < NK / 4; q++) {
      const int k = 256 * q + 4 * lane;
      float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
      if (use && k < H) t = *reinterpret_cast<const float4*>(row + k);      // H % 4 == 0: the whole group is inside the row
      r[4 * q] = t.x; r[4 * q + 1] = t.y; r[4 * q + 2] = t.z; r[4 * q + 3] = t.w;
    }
  } else {
#pragma unroll
    for (int i = 0; i < NK; i++) { const int k = lane + 64 * i; r[i] = (use && k < H) ? row[k] : 0.f; }
  }
}
template <int NK, int JC, bool V4>
__device__ __forceinline__ void rnn_load_w(const float* __restrict__ W, int H, int j0, bool use_w, float (&w)[JC][NK]) {
#pragma unroll
  for (int c = 0; c < JC; c++) rnn_load_row<NK, V4>(W + (int64_t)(j0 + c < H ? j0 + c : 0) * H, H, use_w && j0 + c < H, w[c]);
}
// V = (rows per pass) * JC partial sums per lane and pass go through the wavefront's LDS area ([V][65] floats) so that lane L
// adds up value L % V over one group of lanes; the groups are then combined with xor-shuffles and V lanes
// finish V outputs in parallel (bias, activation, store).
//   in, ld, use_in   input vectors: row b starts at in + b * ld (read only when use_in)
//   pre(b, c)        called on a finishing lane before the sums: fetches what done() will need (so that those
//                    loads are in flight during the arithmetic)
//   done(b, c, s, f) called on the same lane with the finished sum of row b, weight row j0 + c
constexpr int RED_LD = 65;
template <int NK, int JC> struct RnnCfg { static constexpr int V = NK >= 32 ? 16 : 32; static constexpr int UBR = V / JC; };
template <int NK, int JC, bool V4, class Pre, class Done>
__device__ __forceinline__ void rnn_rows_w(const float (&w)[JC][NK], const float* __restrict__ in, int ld, bool use_in, int H, int B, int j0, float* red,
                                           Pre pre, Done done) {
  constexpr int V = RnnCfg<NK, JC>::V, UBR = RnnCfg<NK, JC>::UBR;
  static_assert(UBR >= 1 && UBR * JC == V, "rows per pass times weight rows must be V");
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* my = red + wave * (V * RED_LD);
  const int v = lane % V, grp = lane / V;
  const int fu = v / JC, fc = v % JC;                      // the output this lane finishes in every pass
  float h[UBR][NK];
  auto fetch = [&](int b0) {
#pragma unroll
    for (int u = 0; u < UBR; u++) rnn_load_row<NK, V4>(in + (int64_t)(b0 + u < B ? b0 + u : 0) * ld, H, use_in && b0 + u < B, h[u]);
  };
  int b0 = wave * UBR;
  if (b0 < B) fetch(b0);
  for (; b0 < B; b0 += 4 * UBR) {
    const bool fin = grp == 0 && b0 + fu < B && j0 + fc < H;
    RnnPre f = {0.f, 0.f, 0.f};
    if (fin) f = pre(b0 + fu, fc);
    float t[UBR * JC];
#pragma unroll
    for (int u = 0; u < UBR; u++)
#pragma unroll
      for (int c = 0; c < JC; c++) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < NK; i++) acc = fmaf(h[u][i], w[c][i], acc);
        t[u * JC + c] = acc;
      }
    if (b0 + 4 * UBR < B) fetch(b0 + 4 * UBR);            // next group's loads overlap the reduction below
#pragma unroll
    for (int i = 0; i < UBR * JC; i++) my[i * RED_LD + lane] = t[i];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    float tot = 0.f;
#pragma unroll
    for (int i = 0; i < V; i++) tot += my[v * RED_LD + grp * V + i];
#pragma unroll
    for (int m = V; m < 64; m <<= 1) tot += __shfl_xor(tot, m, 64);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();                       // the area is free for the next pass
    if (fin) done(b0 + fu, fc, tot, f);
  }
}
template <int NK, int JC, bool V4, class Pre, class Done>
__device__ __forceinline__ void rnn_rows(const float* __restrict__ W, const float* __restrict__ in, int ld, bool use_in, int H, int B, int j0, float* red,
                                         Pre pre, Done done) {
  float w[JC][NK];
  rnn_load_w<NK, JC, V4>(W, H, j0, use_in, w);
  rnn_rows_w<NK, JC, V4>(w, in, ld, use_in, H, B, j0, red, pre, done);
}

// One time step of both directions.
//   out[b, j] = act(pre[b, j] + bias1[j] + bias2[j] + sum_k prev[b, k] * W_hh[j, k])
// pre/out alias inside y: row stride ld.  dir = blockIdx.y picks the direction's weights and time index.
struct StepArgs {
  float* cur[2];              // y + t*B*ld + d*H        (pre-activation in, hidden state out)
  const float* prev[2];       // y + tp*B*ld + d*H, or nullptr at the first step
  const float* W[2];          // W_hh of the direction, [H, H] rows = output units
  const float* b1[2]; const float* b2[2];
};
template <int NK, int JC, bool V4>
__global__ void __launch_bounds__(TPB) k_rnn_fwd_step(StepArgs a, int B, int H, int ld, int mode) {
  __shared__ float red[4 * RnnCfg<NK, JC>::V * RED_LD];
  const int d = blockIdx.y, j0 = blockIdx.x * JC;
  float* cur = a.cur[d]; const float* prev = a.prev[d]; const float* b1 = a.b1[d]; const float* b2 = a.b2[d];
  rnn_rows<NK, JC, V4>(a.W[d], prev, ld, prev != nullptr, H, B, j0, red,
    [&](int b, int c) { const int j = j0 + c; RnnPre f = {cur[(int64_t)b * ld + j], b1[j], b2[j]}; return f; },
    [&](int b, int c, float s, const RnnPre& f) { cur[(int64_t)b * ld + j0 + c] = act_fwd(mode, f.a + f.b + f.c + s); });
}

// One backward time step of both directions.  With g_t = dpre of time slice t (already complete):
//   dh[b, i]       = sum_j g_t[b, j] * Wt[i, j]                               (Wt = W_hh transposed, rows = i)
//   g_next[b, i]   = (dy_next[b, i] + dh[b, i]) * act'(h_next[b, i])          for the slice the next launch consumes
// A block reads all of g_t and produces its own columns of g_next, so nothing is computed twice.  cur == nullptr
// starts the chain: g_next = dy_next * act'(h_next).
struct BwdArgs {
  const float* cur[2];          // g_t: dpre + t*B*ld + d*H, or nullptr
  const float* dy[2]; const float* h[2]; float* next[2];          // slice of the next step, direction offset applied
  const float* Wt[2];
};
template <int NK, int JC, bool V4>
__global__ void __launch_bounds__(TPB) k_rnn_bwd_step(BwdArgs a, int B, int H, int ld, int mode) {
  __shared__ float red[4 * RnnCfg<NK, JC>::V * RED_LD];
  const int d = blockIdx.y, i0 = blockIdx.x * JC;
  const float* cur = a.cur[d]; const float* dy = a.dy[d]; const float* hh = a.h[d]; float* next = a.next[d];
  rnn_rows<NK, JC, V4>(a.Wt[d], cur, ld, cur != nullptr, H, B, i0, red,
    [&](int b, int c) { const int64_t o = (int64_t)b * ld + i0 + c; RnnPre f = {hh[o], dy[o], 0.f}; return f; },
    [&](int b, int c, float s, const RnnPre& f) {
      const float g = f.b + s;
      next[(int64_t)b * ld + i0 + c] = mode == 1 ? g * (1.0f - f.a * f.a) : (f.a > 0.f ? g : 0.f); });
}

template <int NIT, int BT, int NW>
__global__ void __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(1, 2))) k_rnn_fwd_step_mfma(StepArgs a, int B, int H, int ld, int mode) {
  __shared__ float red[NW * 256 * BT];
  const int d = blockIdx.y, j0 = blockIdx.x * 16, b0 = blockIdx.z * (16 * BT);
  float* cur = a.cur[d]; const float* prev = a.prev[d]; const float* b1 = a.b1[d]; const float* b2 = a.b2[d];
  rnn_tile_mfma<NIT, BT, NW>(a.W[d], H, H, prev, ld, prev != nullptr, H, B, j0, b0, red,
    [&](int b, int c) { const int j = j0 + c; RnnPre f = {cur[(int64_t)b * ld + j], b1[j], b2[j]}; return f; },
    [&](int b, int c, float s, const RnnPre& f) { cur[(int64_t)b * ld + j0 + c] = act_fwd(mode, f.a + f.b + f.c + s); });
}
template <int NIT, int BT, int NW>
__global__ void __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(1, 2))) k_rnn_bwd_step_mfma(BwdArgs a, int B, int H, int ld, int mode) {
  __shared__ float red[NW * 256 * BT];
  const int d = blockIdx.y, i0 = blockIdx.x * 16, b0 = blockIdx.z * (16 * BT);
  const float* cur = a.cur[d]; const float* dy = a.dy[d]; const float* hh = a.h[d]; float* next = a.next[d];
  rnn_tile_mfma<NIT, BT, NW>(a.Wt[d], H, H, cur, ld, cur != nullptr, H, B, i0, b0, red,
    [&](int b, int c) { const int64_t o = (int64_t)b * ld + i0 + c; RnnPre f = {hh[o], dy[o], 0.f}; return f; },
    [&](int b, int c, float s, const RnnPre& f) {
      const float g = f.b + s;
      next[(int64_t)b * ld + i0 + c] = mode == 1 ? g * (1.0f - f.a * f.a) : (f.a > 0.f ? g : 0.f); });
}
// The matrix-pipe form runs for aligned operands (v4) and hidden sizes from 64 to 2048; LH_RNN_MFMA=0 in the environment
// keeps every step on the vector form above.
static bool rnn_use_mfma(bool v4, int H, int B, int ld) {
  return rnn_mfma_enabled() && v4 && H >= 64 && H <= 2048 && ((size_t)(B - 1) * ld + H) * 4 < 0x80000000ull && (size_t)H * H * 4 < 0x80000000ull;
}

// hidden sizes up to 64 * NK, JC weight rows per block (JC * NK <= 128 registers of weights).  v4: every row the
// kernel reads starts on a 16-byte boundary and H is a multiple of 4.
static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }
template <class A>
static void launch_fwd_step(const A& a, int D, int B, int H, int ld, int mode, bool v4) {
  if (rnn_use_mfma(v4, H, B, ld)) {
    const int nit = (int)cdiv(cdiv(H, 16), 4);
    const dim3 grid((unsigned)cdiv(H, 16), D, (unsigned)cdiv(B, 16));
#define GOM(N) hipLaunchKernelGGL((k_rnn_fwd_step_mfma<N, 1, 4>), grid, dim3(256), 0, g_stream, a, B, H, ld, mode)
    if (nit <= 4) GOM(4); else if (nit <= 8) GOM(8); else if (nit <= 13) GOM(13); else if (nit <= 16) GOM(16); else GOM(32);
#undef GOM
    return;
  }
#define GO(NK, JC) do { if (v4) hipLaunchKernelGGL((k_rnn_fwd_step<NK, JC, true>), dim3((unsigned)cdiv(H, JC), D), dim3(TPB), 0, g_stream, a, B, H, ld, mode); \
                        else hipLaunchKernelGGL((k_rnn_fwd_step<NK, JC, false>), dim3((unsigned)cdiv(H, JC), D), dim3(TPB), 0, g_stream, a, B, H, ld, mode); } while (0)
  if (H <= 256) GO(4, 16); else if (H <= 512) GO(8, 16); else if (H <= 1024) GO(16, 8); else GO(32, 4);
#undef GO
}
template <class A>
static void launch_bwd_step(const A& a, int D, int B, int H, int ld, int mode, bool v4) {
  if (rnn_use_mfma(v4, H, B, ld)) {
    const int nit = (int)cdiv(cdiv(H, 16), 4);
    const dim3 grid((unsigned)cdiv(H, 16), D, (unsigned)cdiv(B, 16));
#define GOM(N) hipLaunchKernelGGL((k_rnn_bwd_step_mfma<N, 1, 4>), grid, dim3(256), 0, g_stream, a, B, H, ld, mode)
    if (nit <= 4) GOM(4); else if (nit <= 8) GOM(8); else if (nit <= 13) GOM(13); else if (nit <= 16) GOM(16); else GOM(32);
#undef GOM
    return;
  }
#define GO(NK, JC) do { if (v4) hipLaunchKernelGGL((k_rnn_bwd_step<NK, JC, true>), dim3((unsigned)cdiv(H, JC), D), dim3(TPB), 0, g_stream, a, B, H, ld, mode); \
                        else hipLaunchKernelGGL((k_rnn_bwd_step<NK, JC, false>), dim3((unsigned)cdiv(H, JC), D), dim3(TPB), 0, g_stream, a, B, H, ld, mode); } while (0)
  if (H <= 256) GO(4, 16); else if (H <= 512) GO(8, 16); else if (H <= 1024) GO(16, 8); else GO(32, 4);
#undef GO
}

// db1[j] += colsum[j]; db2[j] += colsum[j]
__global__ void __launch_bounds__(TPB) k_rnn_bias_grad(const float* __restrict__ colsum, float* db1, float* db2, int H) {
  int j = blockIdx.x * TPB + threadIdx.x;
  if (j < H) { float v = colsum[j]; db1[j] += v; db2[j] += v; }
}

static size_t dir_params(int I, int H) { return (size_t)H * I + (size_t)H * H + 2 * (size_t)H; }

// ---- CTC ----------------------------------------------------------------------------------------------
// One block per sample; threads over the 2L+1 states of the blank-extended label string; time is a loop.
// Scaled forward-backward in double precision (the per-step normaliser keeps alpha in range).
constexpr int CTC_TPB = 128;
__device__ __forceinline__ double block_sum_d(double v, double* sm) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  __syncthreads();
  if (lane == 0) sm[wave] = v;
  __syncthreads();
  double t = 0.0;
  for (int i = 0; i < (int)(blockDim.x >> 6); i++) t += sm[i];
  return t;
}
__global__ void __launch_bounds__(CTC_TPB) k_ctc(const float* __restrict__ probs, float* dprobs, const int* __restrict__ labels, const int* __restrict__ label_off,
                                                 const int* __restrict__ label_len, const int* __restrict__ input_len, float* costs,
                                                 double* alpha_all, double* beta_all, double* cn_all, int T, int B, int A, int Smax) {
  __shared__ double sm[4];
  const int b = blockIdx.x;
  const int L = label_len[b], Tb = input_len[b], S = 2 * L + 1;
  const int* lab = labels + label_off[b];
  double* alpha = alpha_all + (size_t)b * T * Smax; double* beta = beta_all + (size_t)b * T * Smax; double* cn = cn_all + (size_t)b * T;
  auto cls = [&](int s) { return (s & 1) ? lab[s >> 1] : 0; };
  auto P = [&](int t, int s) { return (double)probs[((size_t)t * B + b) * A + cls(s)]; };
  double ll = 0.0;
  for (int t = 0; t < Tb; t++) {
    double part = 0.0;
    for (int s = threadIdx.x; s < S; s += CTC_TPB) {
      double a;
      if (t == 0) a = s < 2 ? P(0, s) : 0.0;
      else {
        const double* ap = alpha + (size_t)(t - 1) * Smax;
        a = ap[s];
        if (s >= 1) a += ap[s - 1];
        if (s >= 2 && (s & 1) && lab[s >> 1] != lab[(s >> 1) - 1]) a += ap[s - 2];
        a *= P(t, s);
      }
      alpha[(size_t)t * Smax + s] = a; part += a;
    }
    const double c = block_sum_d(part, sm);
    if (c > 0.0) for (int s = threadIdx.x; s < S; s += CTC_TPB) alpha[(size_t)t * Smax + s] /= c;
    if (threadIdx.x == 0) cn[t] = c;
    ll += log(c);
    __syncthreads();
  }
  for (int s = threadIdx.x; s < S; s += CTC_TPB) beta[(size_t)(Tb - 1) * Smax + s] = (s >= S - 2) ? 1.0 : 0.0;
  __syncthreads();
  for (int t = Tb - 2; t >= 0; t--) {
    const double* bp = beta + (size_t)(t + 1) * Smax; const double c = cn[t + 1];
    for (int s = threadIdx.x; s < S; s += CTC_TPB) {
      double v = bp[s] * P(t + 1, s);
      if (s + 1 < S) v += bp[s + 1] * P(t + 1, s + 1);
      if (s + 2 < S && ((s + 2) & 1) && lab[(s + 2) >> 1] != lab[s >> 1]) v += bp[s + 2] * P(t + 1, s + 2);
      beta[(size_t)t * Smax + s] = v / c;
    }
    __syncthreads();
  }
  const double* al = alpha + (size_t)(Tb - 1) * Smax;
  const double pfin = al[S - 1] + (S > 1 ? al[S - 2] : 0.0);
  if (threadIdx.x == 0) costs[b] = (float)(-(ll + log(pfin)));
  if (dprobs == nullptr) return;
  // d cost / d activation = probs - posterior(class), the gradient cuDNN reports; accumulated
  for (int idx = threadIdx.x; idx < Tb * A; idx += CTC_TPB) {
    const int t = idx / A, k = idx - t * A;
    double acc = 0.0;
    for (int s = (k == 0 ? 0 : 1); s < S; s += 2) if (cls(s) == k) acc += alpha[(size_t)t * Smax + s] * beta[(size_t)t * Smax + s];
    const size_t i = ((size_t)t * B + b) * A + k;
    dprobs[i] += (float)((double)probs[i] - acc / pfin);
  }
}

// Label strings of at most 63 symbols (2L+1 <= 127 states): one wavefront per recursion, lane l holding the blank state
// 2l and the label state 2l+1, so a time step needs no block barrier: neighbours come through one lane shift and the
// normaliser through a wavefront sum.  Wavefront 0 runs the forward recursion while wavefront 1 runs the backward one,
// each with its own per-step normaliser (the posterior alpha*beta / sum_s alpha*beta does not depend on either scale).
// Then both wavefronts turn rows of alpha*beta into class posteriors through a small LDS table.
constexpr int CTC_ROW = 128;                      // doubles per (sample, time) row of alpha and of beta
__device__ __forceinline__ double wave_sum_d(double v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
__global__ void __launch_bounds__(128) k_ctc_wave(const float* __restrict__ probs, float* dprobs, const int* __restrict__ labels, const int* __restrict__ label_off,
                                                  const int* __restrict__ label_len, const int* __restrict__ input_len, float* costs,
                                                  double* alpha_all, double* beta_all, int T, int B, int A) {
  extern __shared__ double hist_all[];             // [2][A]
  __shared__ double s_pfin;
  const int b = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int L = label_len[b], Tb = input_len[b];
  const int* lab = labels + label_off[b];
  const bool has_e = lane <= L, has_o = lane < L;
  const int my = has_o ? lab[lane] : 0;
  double2* arow = reinterpret_cast<double2*>(alpha_all + (size_t)b * T * CTC_ROW) + lane;      // row t: arow[t * 64]
  double2* brow = reinterpret_cast<double2*>(beta_all + (size_t)b * T * CTC_ROW) + lane;
  auto pe_at = [&](int t) { return (double)probs[((size_t)t * B + b) * A]; };
  auto po_at = [&](int t) { return has_o ? (double)probs[((size_t)t * B + b) * A + my] : 0.0; };
  if (wave == 0) {
    const bool skip = has_o && lane >= 1 && lab[lane - 1] != my;        // label state may be entered from the previous label
    double e = 0.0, o = 0.0, ll = 0.0;
    double pe_n = pe_at(0), po_n = po_at(0);
    for (int t = 0; t < Tb; t++) {
      const double pe = pe_n, po = po_n;
      if (t + 1 < Tb) { pe_n = pe_at(t + 1); po_n = po_at(t + 1); }
      if (t == 0) { e = lane == 0 ? pe : 0.0; o = lane == 0 ? po : 0.0; }
      else {
        double up = __shfl_up(o, 1, 64);
        if (lane == 0) up = 0.0;
        const double ne = has_e ? (e + up) * pe : 0.0;
        const double no = has_o ? (o + e + (skip ? up : 0.0)) * po : 0.0;
        e = ne; o = no;
      }
      const double c = wave_sum_d(e + o);
      if (c > 0.0) { const double r = 1.0 / c; e *= r; o *= r; }
      ll += log(c);
      arow[(size_t)t * 64] = make_double2(e, o);
    }
    const double pf = wave_sum_d((lane == L ? e : 0.0) + (lane == L - 1 ? o : 0.0));
    if (lane == 0) { costs[b] = (float)(-(ll + log(pf))); s_pfin = pf; }
  } else {
    const bool skip = lane + 1 < L && lab[lane + 1] != my;               // label state may jump to the next label
    double e = lane == L ? 1.0 : 0.0, o = lane == L - 1 ? 1.0 : 0.0;
    brow[(size_t)(Tb - 1) * 64] = make_double2(e, o);
    double pe_n = Tb >= 2 ? pe_at(Tb - 1) : 0.0, po_n = Tb >= 2 ? po_at(Tb - 1) : 0.0;
    for (int t = Tb - 2; t >= 0; t--) {
      const double pe = pe_n, po = po_n;                                   // emissions of time t + 1
      if (t >= 1) { pe_n = pe_at(t); po_n = po_at(t); }
      const double qe = e * pe, qo = o * po;
      double dn_e = __shfl_down(qe, 1, 64), dn_o = __shfl_down(qo, 1, 64);
      if (lane == 63) { dn_e = 0.0; dn_o = 0.0; }
      const double ne = has_e ? qe + qo : 0.0;
      const double no = has_o ? qo + dn_e + (skip ? dn_o : 0.0) : 0.0;
      const double c = wave_sum_d(ne + no);
      const double r = c > 0.0 ? 1.0 / c : 1.0;
      e = ne * r; o = no * r;
      brow[(size_t)t * 64] = make_double2(e, o);
    }
  }
  __syncthreads();
  if (dprobs == nullptr) return;
  // d cost / d activation = probs - posterior(class), the gradient cuDNN reports; accumulated
  double* hist = hist_all + (size_t)wave * A;
  for (int t = wave; t < Tb; t += 2) {
    const double2 al = arow[(size_t)t * 64], be = brow[(size_t)t * 64];
    const double ge = al.x * be.x, go = al.y * be.y;
    const double z = wave_sum_d(ge + go), blank = wave_sum_d(ge);
    for (int k = lane; k < A; k += 64) hist[k] = 0.0;
    wave_lds_sync();
    if (has_o) atomicAdd(&hist[my], go);
    wave_lds_sync();
    for (int k = lane; k < A; k += 64) {
      const size_t i = ((size_t)t * B + b) * A + k;
      const double post = (k == 0 ? blank : hist[k]) / z;
      dprobs[i] += (float)((double)probs[i] - post);
    }
    wave_lds_sync();
  }
}
}  // namespace

extern "C" {

void lh_rnn_fwd(int mode, const float* x, const float* w, float* y, int T, int B, int I, int H, int bidir) {
  lh_rnn_fwd_init(mode, x, nullptr, w, y, T, B, I, H, bidir);
}
void lh_rnn_bwd(int mode, const float* x, const float* y, const float* dy, const float* w, float* dx, float beta_dx, float* dw,
                int T, int B, int I, int H, int bidir) {
  lh_rnn_bwd_init(mode, x, nullptr, y, dy, w, dx, beta_dx, dw, T, B, I, H, bidir);
}

void lh_rnn_fwd_init(int mode, const float* x, const float* hx, const float* w, float* y, int T, int B, int I, int H, int bidir) {
  LH_REQUIRE(mode == 0 || mode == 1, "lh_rnn_fwd: mode %d (0 = relu, 1 = tanh)", mode);
  LH_REQUIRE(T >= 1 && B >= 1 && I >= 1 && H >= 1, "lh_rnn_fwd: bad shape T%d B%d I%d H%d", T, B, I, H);
  LH_REQUIRE(H <= 2048, "lh_rnn_fwd: hidden size %d above %d", H, 2048);
  LH_REQUIRE(x && w && y, "lh_rnn_fwd: null operand");
  const int D = bidir ? 2 : 1, ld = D * H;
  LZ_ENTER();
  lazy::rd_f(x, (int64_t)T * B * I); lazy::rd_f(w, (int64_t)D * dir_params(I, H)); lazy::rd_f(hx, (int64_t)D * B * H); lazy::wr_f(y, (int64_t)T * B * ld);
  for (int d = 0; d < D; d++) {          // input projection of every step straight into y
    const float* Wih = w + d * dir_params(I, H);
    lh_sgemm(0, 1, T * B, H, I, 1.0f, x, I, Wih, I, 0.0f, y + d * H, ld);
    // an initial state enters the first processed step as one more product added to that step's input projection
    // (the step kernel then sees no previous step, as with a zero state)
    if (hx) lh_sgemm(0, 1, B, H, H, 1.0f, hx + (size_t)d * B * H, H, Wih + (size_t)H * I, H, 1.0f, y + (size_t)(d == 0 ? 0 : T - 1) * B * ld + d * H, ld);
  }
  ProfScope prof_(CAT_RNN);
  for (int step = 0; step < T; step++) {
    StepArgs a;
    for (int d = 0; d < 2; d++) {
      const int dd = d < D ? d : 0;
      const float* Wih = w + dd * dir_params(I, H); const float* Whh = Wih + (size_t)H * I;
      const int t = dd == 0 ? step : T - 1 - step, tp = dd == 0 ? t - 1 : t + 1;
      a.cur[d] = y + (size_t)t * B * ld + dd * H;
      a.prev[d] = step == 0 ? nullptr : y + (size_t)tp * B * ld + dd * H;
      a.W[d] = Whh; a.b1[d] = Whh + (size_t)H * H; a.b2[d] = a.b1[d] + H;
    }
    launch_fwd_step(a, D, B, H, ld, mode, (H & 3) == 0 && aligned16(y) && aligned16(w));
  }
  LH_CHECK_LAUNCH();
}

void lh_rnn_bwd_init(int mode, const float* x, const float* hx, const float* y, const float* dy, const float* w, float* dx, float beta_dx, float* dw,
                     int T, int B, int I, int H, int bidir) {
  LH_REQUIRE(mode == 0 || mode == 1, "lh_rnn_bwd: mode %d (0 = relu, 1 = tanh)", mode);
  LH_REQUIRE(T >= 1 && B >= 1 && I >= 1 && H >= 1, "lh_rnn_bwd: bad shape T%d B%d I%d H%d", T, B, I, H);
  LH_REQUIRE(H <= 2048, "lh_rnn_bwd: hidden size %d above %d", H, 2048);
  LH_REQUIRE(beta_dx == 0.f || beta_dx == 1.f, "lh_rnn_bwd: beta must be 0 or 1");
  LH_REQUIRE(x && y && dy && w && dw, "lh_rnn_bwd: null operand");
  const int D = bidir ? 2 : 1, ld = D * H;
  LZ_ENTER();
  lazy::rd_f(x, (int64_t)T * B * I); lazy::rd_f(y, (int64_t)T * B * ld); lazy::rd_f(dy, (int64_t)T * B * ld); lazy::rd_f(w, (int64_t)D * dir_params(I, H));
  lazy::rd_f(hx, (int64_t)D * B * H); lazy::rw_f(dw, (int64_t)D * dir_params(I, H));
  if (dx) beta_dx = lazy::beta_f(dx, (int64_t)T * B * I, beta_dx);          // an input gradient nobody has touched since lh_malloc is overwritten
  // scratch from the top of the arena: dpre [T*B, D*H], W_hh^T per direction, column sums
  const size_t n_dpre = (size_t)T * B * ld, n_wt = (size_t)D * H * H, n_cs = (size_t)ld;
  const size_t bytes = (n_dpre + n_wt + n_cs) * sizeof(float);
  float* scratch = (float*)lh_malloc_uninit(bytes);
  if (scratch == nullptr) return;
  float* dpre = scratch; float* wt = dpre + n_dpre; float* colsum = wt + n_wt;
  for (int d = 0; d < D; d++) {
    const float* Whh = w + d * dir_params(I, H) + (size_t)H * I;
    lh_trans(Whh, wt + (size_t)d * H * H, H, H);
  }
  {
    ProfScope prof_(CAT_RNN);
    // launch k produces dpre of the k-th slice in processing order (forward direction: t = T-1-k, reverse: t = k)
    for (int k = 0; k < T; k++) {
      BwdArgs a;
      for (int d = 0; d < 2; d++) {
        const int dd = d < D ? d : 0;
        const int tn = dd == 0 ? T - 1 - k : k;                 // slice produced
        const int tc = dd == 0 ? tn + 1 : tn - 1;               // slice consumed (processed just before)
        const size_t on = (size_t)tn * B * ld + dd * H;
        a.cur[d] = k == 0 ? nullptr : dpre + (size_t)tc * B * ld + dd * H;
        a.dy[d] = dy + on; a.h[d] = y + on; a.next[d] = dpre + on;
        a.Wt[d] = wt + (size_t)dd * H * H;
      }
      launch_bwd_step(a, D, B, H, ld, mode, (H & 3) == 0 && aligned16(dpre) && aligned16(wt) && aligned16(dy) && aligned16(y));
    }
  }
  lh_sum_dim(dpre, colsum, 1, T * B, ld);
  for (int d = 0; d < D; d++) {
    const size_t off = d * dir_params(I, H);
    const float* Wih = w + off;
    float* dWih = dw + off; float* dWhh = dWih + (size_t)H * I; float* dbih = dWhh + (size_t)H * H; float* dbhh = dbih + H;
    lh_sgemm(1, 0, H, I, T * B, 1.0f, dpre + d * H, ld, x, I, 1.0f, dWih, I);
    if (T > 1) {
      // dW_hh += sum_t dpre_t^T h_{prev(t)}: forward pairs (t, t-1), reverse pairs (t, t+1)
      const float* A = d == 0 ? dpre + (size_t)B * ld + d * H : dpre + d * H;
      const float* Bm = d == 0 ? y + d * H : y + (size_t)B * ld + d * H;
      lh_sgemm(1, 0, H, H, (T - 1) * B, 1.0f, A, ld, Bm, ld, 1.0f, dWhh, H);
    }
    // the first processed step's pair is (dpre of that step, the initial state)
    if (hx) lh_sgemm(1, 0, H, H, B, 1.0f, dpre + (size_t)(d == 0 ? 0 : T - 1) * B * ld + d * H, ld, hx + (size_t)d * B * H, H, 1.0f, dWhh, H);
    hipLaunchKernelGGL(k_rnn_bias_grad, dim3((unsigned)cdiv(H, TPB)), dim3(TPB), 0, g_stream, colsum + d * H, dbih, dbhh, H);
    if (dx) lh_sgemm(0, 0, T * B, I, H, 1.0f, dpre + d * H, ld, Wih, I, d == 0 ? beta_dx : 1.0f, dx, I);
  }
  lh_free_top(bytes);      // stream order: the kernels above run before anything that reuses the space
  LH_CHECK_LAUNCH();
}

void lh_ctc_loss(const float* probs, float* dprobs, const int* h_labels, const int* h_label_len, const int* h_input_len,
                 float* costs, int T, int B, int A) {
  ProfScope prof_(CAT_REDUCE);
  LH_NOT_CAPTURING("lh_ctc_loss (it uploads its label and length arrays)");
  LH_REQUIRE(T >= 1 && B >= 1 && A >= 2, "lh_ctc_loss: bad shape T%d B%d A%d", T, B, A);
  LH_REQUIRE(probs && costs && h_labels && h_label_len && h_input_len, "lh_ctc_loss: null operand");
  LZ_ENTER();
  lazy::rd_f(probs, (int64_t)T * B * A); lazy::rw_f(dprobs, (int64_t)T * B * A); lazy::wr_f(costs, B);
  int total = 0, Lmax = 0;
  int* host = (int*)malloc(sizeof(int) * (size_t)(3 * B));
  if (!host) { LH_FAIL("lh_ctc_loss: out of host memory"); return; }
  for (int b = 0; b < B; b++) {
    const int L = h_label_len[b], Tb = h_input_len[b];
    if (L < 0 || Tb < 1 || Tb > T || Tb < L) { free(host); LH_FAIL("lh_ctc_loss: sample %d has label length %d and input length %d (T = %d)", b, L, Tb, T); return; }
    host[b] = total; host[B + b] = L; host[2 * B + b] = Tb;
    total += L; if (L > Lmax) Lmax = L;
  }
  for (int i = 0; i < total; i++) if (h_labels[i] < 1 || h_labels[i] >= A) { free(host); LH_FAIL("lh_ctc_loss: label %d outside 1..%d (0 is the blank)", h_labels[i], A - 1); return; }
  const int Smax = 2 * Lmax + 1;
  const bool one_wave = Lmax <= 63 && A <= 2048;       // 2L+1 states fit a wavefront's lane pairs; the class table fits LDS
  const size_t n_int = (size_t)3 * B + (size_t)(total > 0 ? total : 1);
  const size_t int_bytes = ((n_int * sizeof(int)) + 255) & ~(size_t)255;
  const size_t row = one_wave ? (size_t)CTC_ROW : (size_t)Smax;
  const size_t dbl = ((size_t)2 * B * T * row + (size_t)B * T) * sizeof(double);
  char* scratch = (char*)lh_malloc_uninit(int_bytes + dbl);
  if (scratch == nullptr) { free(host); return; }
  int* d_int = (int*)scratch;
  lh_h2d(d_int, host, sizeof(int) * (size_t)(3 * B));
  if (total > 0 && !failed()) lh_h2d(d_int + 3 * B, h_labels, sizeof(int) * (size_t)total);
  free(host);
  if (failed()) { lh_free_top(int_bytes + dbl); return; }       // nothing is launched on lengths and labels that were not uploaded
  double* alpha = (double*)(scratch + int_bytes); double* beta = alpha + (size_t)B * T * row; double* cn = beta + (size_t)B * T * row;
  if (one_wave) hipLaunchKernelGGL(k_ctc_wave, dim3(B), dim3(128), 2 * (size_t)A * sizeof(double), g_stream, probs, dprobs, d_int + 3 * B, d_int, d_int + B, d_int + 2 * B, costs, alpha, beta, T, B, A);
  else hipLaunchKernelGGL(k_ctc, dim3(B), dim3(CTC_TPB), 0, g_stream, probs, dprobs, d_int + 3 * B, d_int, d_int + B, d_int + 2 * B, costs, alpha, beta, cn, T, B, A, Smax);
  lh_free_top(int_bytes + dbl);
  LH_CHECK_LAUNCH();
}

}  // extern "C"
