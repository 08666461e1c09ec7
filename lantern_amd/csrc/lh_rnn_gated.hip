// LSTM and GRU layers (RNNBase with LstmMode / GruMode: src/main/scala/lantern/NNModule.scala:324-417 over
// cudnnRNNForwardTraining / BackwardData / BackwardWeights, src/main/scala/lantern/TensorDslCudnn.scala:1638-1893).
//
// Gate order and formulas are cuDNN's: LSTM i, f, g, o with c' = f*c + i*g, h' = o*tanh(c'); GRU r, z, n with
// n = tanh(W_in x + b_in + r*(W_hn h + b_hn)), h' = (1 - z)*n + z*h.  One layer, optional initial state (values only, no gradient), optionally
// bidirectional (y = forward half, then reverse half).  Parameters per direction: W_ih[G, I], W_hh[G, H], b_ih[G],
// b_hh[G] with G = 4H or 3H (NNModule.scala:378-390).
//
// Everything that is not sequential is one matrix product over all time steps (lh_sgemm on MFMA): the input projection,
// both weight gradients, the input gradient.  A forward time step is one launch (the [B, H] x [H, G] product with the
// previous state on 16 x 16 matrix tiles that hold all gates of four units, the gate arithmetic behind it); a backward
// step, and a forward step on operands the tile kernel does not take, is a product plus one element-wise kernel over
// [B, H].  The forward pass leaves the gate activations and the cell state (GRU: W_hn h + b_hn)
// of every step in `reserve`; the backward pass turns the activations into pre-activation gradients in place.
#include "lh_common.h"
#include "lh_rnn_tile.h"
#include "../../include/lantern_hip.h"
using namespace lh;

namespace {

constexpr int TPB = 256;

__device__ __forceinline__ float sigm(float v) { return 1.0f / (1.0f + expf(-v)); }

// act [B, 4H]: input projection of this step on entry, gate activations on exit.  gh [B, 4H] = h_prev W_hh^T or null.
__global__ void __launch_bounds__(TPB) k_lstm_fwd_point(float* __restrict__ act, const float* __restrict__ gh, const float* __restrict__ b_ih,
                                                        const float* __restrict__ b_hh, const float* __restrict__ c_prev, float* __restrict__ c,
                                                        float* __restrict__ h, int B, int H, int ldh) {
  const int idx = blockIdx.x * TPB + threadIdx.x;
  if (idx >= B * H) return;
  const int b = idx / H, j = idx - b * H;
  float* a = act + (size_t)b * 4 * H + j;
  float p[4];
#pragma unroll
  for (int g = 0; g < 4; g++) p[g] = a[g * H] + b_ih[g * H + j] + b_hh[g * H + j] + (gh ? gh[(size_t)b * 4 * H + g * H + j] : 0.f);
  const float ig = sigm(p[0]), fg = sigm(p[1]), gg = tanhf(p[2]), og = sigm(p[3]);
  const float cn = fg * (c_prev ? c_prev[idx] : 0.f) + ig * gg;
  a[0] = ig; a[H] = fg; a[2 * H] = gg; a[3 * H] = og;
  c[idx] = cn;
  h[(size_t)b * ldh + j] = og * tanhf(cn);
}

// act [B, 4H]: activations on entry, pre-activation gradients on exit.  dh_rec / dc hold what flows in from the step
// processed before (ignored on the first processed step); dh_rec is cleared, dc is rewritten with the cell gradient passed on.
__global__ void __launch_bounds__(TPB) k_lstm_bwd_point(float* __restrict__ act, const float* __restrict__ c, const float* __restrict__ c_prev,
                                                        const float* __restrict__ dy, float* __restrict__ dh_rec, float* __restrict__ dc,
                                                        int first, int B, int H, int ldh) {
  const int idx = blockIdx.x * TPB + threadIdx.x;
  if (idx >= B * H) return;
  const int b = idx / H, j = idx - b * H;
  float* a = act + (size_t)b * 4 * H + j;
  const float ig = a[0], fg = a[H], gg = a[2 * H], og = a[3 * H];
  const float dh = dy[(size_t)b * ldh + j] + (first ? 0.f : dh_rec[idx]);
  dh_rec[idx] = 0.f;                                             // the product that follows adds the next recurrent gradient into it
  const float tc = tanhf(c[idx]);
  const float dcc = dh * og * (1.f - tc * tc) + (first ? 0.f : dc[idx]);
  const float cp = c_prev ? c_prev[idx] : 0.f;
  a[0] = dcc * gg * ig * (1.f - ig);
  a[H] = dcc * cp * fg * (1.f - fg);
  a[2 * H] = dcc * ig * (1.f - gg * gg);
  a[3 * H] = dh * tc * og * (1.f - og);
  dc[idx] = dcc * fg;
}

// act [B, 3H]: input projection on entry, r, z, n on exit.  gh [B, 3H] = h_prev W_hh^T or null.  q [B, H] = W_hn h + b_hn.
// gh is cleared after it is read: the next step's product adds into it (a product with beta = 0 cut over K needs a pass of its own
// that clears the result first, a launch per step).
__global__ void __launch_bounds__(TPB) k_gru_fwd_point(float* __restrict__ act, float* __restrict__ gh, const float* __restrict__ b_ih,
                                                       const float* __restrict__ b_hh, const float* __restrict__ h_prev, int ldp, float* __restrict__ q,
                                                       float* __restrict__ h, int B, int H, int ldh) {
  const int idx = blockIdx.x * TPB + threadIdx.x;
  if (idx >= B * H) return;
  const int b = idx / H, j = idx - b * H;
  float* a = act + (size_t)b * 3 * H + j;
  float* g = gh + (size_t)b * 3 * H + j;
  const float g0 = g[0], g1 = g[H], g2 = g[2 * H];               // zeros when there is no previous state
  g[0] = 0.f; g[H] = 0.f; g[2 * H] = 0.f;
  const float r = sigm(a[0] + b_ih[j] + b_hh[j] + g0);
  const float z = sigm(a[H] + b_ih[H + j] + b_hh[H + j] + g1);
  const float qq = g2 + b_hh[2 * H + j];
  const float n = tanhf(a[2 * H] + b_ih[2 * H + j] + r * qq);
  const float hp = h_prev ? h_prev[(size_t)b * ldp + j] : 0.f;      // ldp: row stride of h_prev (an initial state is [B, H])
  a[0] = r; a[H] = z; a[2 * H] = n;
  q[idx] = qq;
  h[(size_t)b * ldh + j] = (1.f - z) * n + z * hp;
}

// act [B, 3H]: r, z, n on entry, gradients of the input-side pre-activations on exit; dgh [B, 3H] receives those of the
// hidden side (the n column scaled by r).  carry [B, H]: the recurrent gradient on entry (ignored when first), dh * z on
// exit; the caller adds dgh W_hh to it.
__global__ void __launch_bounds__(TPB) k_gru_bwd_point(float* __restrict__ act, float* __restrict__ dgh, const float* __restrict__ q,
                                                       const float* __restrict__ h_prev, int ldp, const float* __restrict__ dy, float* __restrict__ carry,
                                                       int first, int B, int H, int ldh) {
  const int idx = blockIdx.x * TPB + threadIdx.x;
  if (idx >= B * H) return;
  const int b = idx / H, j = idx - b * H;
  float* a = act + (size_t)b * 3 * H + j;
  float* g = dgh + (size_t)b * 3 * H + j;
  const float r = a[0], z = a[H], n = a[2 * H];
  const float dh = dy[(size_t)b * ldh + j] + (first ? 0.f : carry[idx]);
  const float hp = h_prev ? h_prev[(size_t)b * ldp + j] : 0.f;
  const float dn = dh * (1.f - z) * (1.f - n * n);
  const float dz = dh * (hp - n) * z * (1.f - z);
  const float dr = dn * q[idx] * r * (1.f - r);
  a[0] = dr; a[H] = dz; a[2 * H] = dn;
  g[0] = dr; g[H] = dz; g[2 * H] = dn * r;
  carry[idx] = dh * z;
}

__global__ void __launch_bounds__(TPB) k_add_into(float* __restrict__ dst, const float* __restrict__ src, int n) {
  const int i = blockIdx.x * TPB + threadIdx.x;
  if (i < n) dst[i] += src[i];
}

int gates_of(int mode) { return mode == 2 ? 4 : 3; }
size_t dir_params(int mode, int I, int H) { const size_t G = (size_t)gates_of(mode) * H; return G * I + G * H + 2 * G; }
size_t dir_reserve(int mode, int T, int B, int H) { return (size_t)T * B * (gates_of(mode) + 1) * H; }
unsigned point_grid(int B, int H) { return (unsigned)cdiv((int64_t)B * H, TPB); }

bool check_shape(const char* who, int mode, int T, int B, int I, int H) {
  if (mode != 2 && mode != 3) { LH_FAIL("%s: mode %d (2 = LSTM, 3 = GRU)", who, mode); return false; }
  if (T < 1 || B < 1 || I < 1 || H < 1) { LH_FAIL("%s: bad shape T%d B%d I%d H%d", who, T, B, I, H); return false; }
  if ((int64_t)T * B * 4 * H > INT32_MAX || (int64_t)B * 4 * H > (1 << 28)) { LH_FAIL("%s: T%d B%d H%d too large", who, T, B, H); return false; }
  return true;
}

}  // namespace

// ---- the per-step products on the matrix pipes ----------------------------------------------------------------------
//   out[B, NJ] += in[B, K] * W[NJ, K]^T      (rows of both operands contiguous in k)
// with the tile of lh_rnn_tile.h: a block produces 16 outputs for 16 batch rows, the reduction cut over its 4 wavefronts (8 from
// K = 1040 on, so that a wavefront's loads still fit its registers), every load issued before the first matrix instruction.
// The LSTM's forward step at B 32, H 800 ([32, 800] x [800, 3200]): 400 blocks; layer forward + backward 5.74 -> 5.37 ms (GRU
// 5.40 -> 4.95).  Shapes it does not take (unaligned rows, K not a multiple of 4 or above 3200) go to lh_sgemm.  The backward
// step's product (contraction over the 3200 gate rows, on a transposed copy of W_hh) measured slower this way than through
// lh_sgemm's reduction cut over blocks (6.5 against 5.7 ms) and stays there.
namespace {
struct SmallNt { const float* in; const float* W; float* out; int ldi, ldw, ldo, B, NJ, K; };
template <int NIT, int NW>
__global__ void __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(1, 2))) k_small_nt_mfma(SmallNt a) {
  __shared__ float red[NW * 256];
  const int j0 = blockIdx.x * 16, b0 = blockIdx.y * 16;
  rnn_tile_mfma<NIT, 1, NW>(a.W, a.ldw, a.NJ, a.in, a.ldi, true, a.K, a.B, j0, b0, red,
    [&](int b, int c) { RnnPre f = {a.out[(int64_t)b * a.ldo + j0 + c], 0.f, 0.f}; return f; },
    [&](int b, int c, float s, const RnnPre& f) { a.out[(int64_t)b * a.ldo + j0 + c] = f.a + s; });
}
static bool aligned16g(const void* p) { return ((uintptr_t)p & 15) == 0; }

// The LSTM's forward step in one launch: a block owns the four gates of four hidden units (column c of its tile stands for gate
// c / 4 of unit u0 + c % 4, i.e. row (c / 4) * H + u0 + c % 4 of W_hh) for 16 batch rows; after the partial tiles are in LDS,
// thread (batch row, unit) adds up the four gate sums and does what k_lstm_fwd_point does: activations into `act`, the new cell
// and hidden state.  hp == nullptr: no previous state (the sums are zero).
template <int NIT>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 2)))
k_lstm_fwd_step_mfma(const float* __restrict__ hp, int ldp, const float* __restrict__ Whh, float* __restrict__ act, const float* __restrict__ b_ih,
                     const float* __restrict__ b_hh, const float* __restrict__ c_prev, float* __restrict__ c, float* __restrict__ h, int B, int H, int ldh) {
  __shared__ float red[4 * 256];
  const int t = threadIdx.x, u0 = blockIdx.x * 4, b0 = blockIdx.y * 16;
  const int bl = t >> 2, u = t & 3, b = b0 + bl, j = u0 + u;
  const bool fin = t < 64 && b < B && j < H;
  float pa[4], pb[4], cp = 0.f;
  if (fin) {
    // what the output stage needs, requested before the products
#pragma unroll
    for (int g = 0; g < 4; g++) { pa[g] = act[(size_t)b * 4 * H + g * H + j]; pb[g] = b_ih[g * H + j]; }
    cp = c_prev ? c_prev[(size_t)b * H + j] : 0.f;
  }
  if (hp) {
    const int r = t & 15;
    rnn_tile_partials<NIT, 1, 4>(Whh, H, (size_t)4 * H * H * 4, u0 + (r & 3) < H ? (r >> 2) * H + u0 + (r & 3) : -1, hp, ldp, H, B, b0, red);
  }
  if (!fin) return;
  float p[4];
#pragma unroll
  for (int g = 0; g < 4; g++) {
    float s = 0.f;
    if (hp) { const int o = (bl & 3) * 64 + 16 * (bl >> 2) + 4 * g + u; s = (red[o] + red[256 + o]) + (red[512 + o] + red[768 + o]); }
    p[g] = ((pa[g] + s) + pb[g]) + b_hh[g * H + j];
  }
  const float ig = sigm(p[0]), fg = sigm(p[1]), gg = tanhf(p[2]), og = sigm(p[3]);
  const float cn = fg * cp + ig * gg;
  float* a = act + (size_t)b * 4 * H + j;
  a[0] = ig; a[H] = fg; a[2 * H] = gg; a[3 * H] = og;
  c[(size_t)b * H + j] = cn;
  h[(size_t)b * ldh + j] = og * tanhf(cn);
}
// The GRU's forward step the same way: three gates of four units are 12 of the tile's 16 columns (the last four stay idle);
// the hidden-side sums are used where they are, so no buffer holds them between two launches.
template <int NIT>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 2)))
k_gru_fwd_step_mfma(const float* __restrict__ hp, int ldp, const float* __restrict__ Whh, float* __restrict__ act, const float* __restrict__ b_ih,
                    const float* __restrict__ b_hh, float* __restrict__ q, float* __restrict__ h, int B, int H, int ldh) {
  __shared__ float red[4 * 256];
  const int t = threadIdx.x, u0 = blockIdx.x * 4, b0 = blockIdx.y * 16;
  const int bl = t >> 2, u = t & 3, b = b0 + bl, j = u0 + u;
  const bool fin = t < 64 && b < B && j < H;
  float pa[3], pb[3], hprev = 0.f;
  if (fin) {
#pragma unroll
    for (int g = 0; g < 3; g++) { pa[g] = act[(size_t)b * 3 * H + g * H + j]; pb[g] = b_ih[g * H + j]; }
    hprev = hp ? hp[(size_t)b * ldp + j] : 0.f;
  }
  if (hp) {
    const int r = t & 15;
    rnn_tile_partials<NIT, 1, 4>(Whh, H, (size_t)3 * H * H * 4, (r < 12 && u0 + (r & 3) < H) ? (r >> 2) * H + u0 + (r & 3) : -1, hp, ldp, H, B, b0, red);
  }
  if (!fin) return;
  float gs[3];
#pragma unroll
  for (int g = 0; g < 3; g++) {
    gs[g] = 0.f;
    if (hp) { const int o = (bl & 3) * 64 + 16 * (bl >> 2) + 4 * g + u; gs[g] = (red[o] + red[256 + o]) + (red[512 + o] + red[768 + o]); }
  }
  const float r = sigm(pa[0] + pb[0] + b_hh[j] + gs[0]);
  const float z = sigm(pa[1] + pb[1] + b_hh[H + j] + gs[1]);
  const float qq = gs[2] + b_hh[2 * H + j];
  const float n = tanhf(pa[2] + pb[2] + r * qq);
  float* a = act + (size_t)b * 3 * H + j;
  a[0] = r; a[H] = z; a[2 * H] = n;
  q[(size_t)b * H + j] = qq;
  h[(size_t)b * ldh + j] = (1.f - z) * n + z * hprev;
}
// true when the fused step ran; false: the caller runs the product and the element-wise kernel
static bool gated_fused_ok(const float* hp, int ldp, const float* Whh, int ng, int B, int H) {
  const int nit = (int)cdiv(cdiv(H, 16), 4);
  return rnn_mfma_enabled() && (H & 3) == 0 && (ldp & 3) == 0 && (hp == nullptr || aligned16g(hp)) && aligned16g(Whh) && nit <= 16 &&
         ((size_t)(B - 1) * ldp + H) * 4 < 0x80000000ull && (size_t)ng * H * H * 4 < 0x80000000ull;
}
static bool gru_fwd_step_fused(const float* hp, int ldp, const float* Whh, float* act, const float* b_ih, const float* b_hh, float* q, float* h,
                               int B, int H, int ldh) {
  if (!gated_fused_ok(hp, ldp, Whh, 3, B, H)) return false;
  const int nit = (int)cdiv(cdiv(H, 16), 4);
  const dim3 grid((unsigned)cdiv(H, 4), (unsigned)cdiv(B, 16));
#define GOG(N) hipLaunchKernelGGL((k_gru_fwd_step_mfma<N>), grid, dim3(256), 0, g_stream, hp, ldp, Whh, act, b_ih, b_hh, q, h, B, H, ldh)
  if (nit <= 4) GOG(4); else if (nit <= 8) GOG(8); else if (nit <= 13) GOG(13); else GOG(16);
#undef GOG
  return true;
}
static bool lstm_fwd_step_fused(const float* hp, int ldp, const float* Whh, float* act, const float* b_ih, const float* b_hh, const float* c_prev,
                                float* c, float* h, int B, int H, int ldh) {
  if (!gated_fused_ok(hp, ldp, Whh, 4, B, H)) return false;
  const int nit = (int)cdiv(cdiv(H, 16), 4);
  const dim3 grid((unsigned)cdiv(H, 4), (unsigned)cdiv(B, 16));
#define GOL(N) hipLaunchKernelGGL((k_lstm_fwd_step_mfma<N>), grid, dim3(256), 0, g_stream, hp, ldp, Whh, act, b_ih, b_hh, c_prev, c, h, B, H, ldh)
  if (nit <= 4) GOL(4); else if (nit <= 8) GOL(8); else if (nit <= 13) GOL(13); else GOL(16);
#undef GOL
  return true;
}
static void step_product_nt(const float* in, int ldi, const float* W, int ldw, float* out, int ldo, int B, int NJ, int K) {
  const int groups = (int)cdiv(K, 16), nw = groups > 64 ? 8 : 4, nit = (int)cdiv(groups, nw);
  const bool ok = rnn_mfma_enabled() && (K & 3) == 0 && (ldi & 3) == 0 && (ldw & 3) == 0 && aligned16g(in) && aligned16g(W) && nit <= 25 &&
                  ((size_t)(B - 1) * ldi + K) * 4 < 0x80000000ull && ((size_t)(NJ - 1) * ldw + K) * 4 < 0x80000000ull;
  if (!ok) { lh_sgemm(0, 1, B, NJ, K, 1.0f, in, ldi, W, ldw, 1.0f, out, ldo); return; }
  const SmallNt a = {in, W, out, ldi, ldw, ldo, B, NJ, K};
  const dim3 grid((unsigned)cdiv(NJ, 16), (unsigned)cdiv(B, 16));
#define GON(N, W_) hipLaunchKernelGGL((k_small_nt_mfma<N, W_>), grid, dim3(64 * W_), 0, g_stream, a)
  if (nw == 4) { if (nit <= 4) GON(4, 4); else if (nit <= 8) GON(8, 4); else if (nit <= 13) GON(13, 4); else GON(16, 4); }
  else { if (nit <= 13) GON(13, 8); else if (nit <= 19) GON(19, 8); else GON(25, 8); }
#undef GON
}
}  // namespace

extern "C" {

int64_t lh_rnn_gated_reserve_floats(int mode, int T, int B, int H, int bidir) {
  if ((mode != 2 && mode != 3) || T < 1 || B < 1 || H < 1) return 0;
  return (int64_t)((bidir ? 2 : 1) * dir_reserve(mode, T, B, H));
}

void lh_rnn_gated_fwd(int mode, const float* x, const float* w, float* y, float* reserve, int T, int B, int I, int H, int bidir) {
  lh_rnn_gated_fwd_init(mode, x, nullptr, nullptr, w, y, reserve, T, B, I, H, bidir);
}
void lh_rnn_gated_bwd(int mode, const float* x, const float* y, const float* dy, const float* w, float* reserve, float* dx, float beta_dx,
                      float* dw, int T, int B, int I, int H, int bidir) {
  lh_rnn_gated_bwd_init(mode, x, nullptr, nullptr, y, dy, w, reserve, dx, beta_dx, dw, T, B, I, H, bidir);
}

void lh_rnn_gated_fwd_init(int mode, const float* x, const float* hx, const float* cx, const float* w, float* y, float* reserve,
                           int T, int B, int I, int H, int bidir) {
  if (!check_shape("lh_rnn_gated_fwd", mode, T, B, I, H)) return;
  LH_REQUIRE(cx == nullptr || mode == 2, "lh_rnn_gated_fwd: only the LSTM has a cell state");
  LH_REQUIRE(x && w && y && reserve, "lh_rnn_gated_fwd: null operand");
  const int D = bidir ? 2 : 1, ldh = D * H, ng = gates_of(mode), G = ng * H;
  LZ_ENTER();
  lazy::rd_f(x, (int64_t)T * B * I); lazy::rd_f(w, (int64_t)D * dir_params(mode, I, H)); lazy::rd_f(hx, (int64_t)D * B * H); lazy::rd_f(cx, (int64_t)D * B * H);
  lazy::wr_f(y, (int64_t)T * B * ldh); lazy::wr_f(reserve, (int64_t)D * dir_reserve(mode, T, B, H));
  const size_t per_dir = (size_t)B * G;
  const size_t gh_bytes = (size_t)D * per_dir * sizeof(float);
  float* gh_all = (float*)lh_malloc_uninit(gh_bytes);
  if (gh_all == nullptr) return;
  // The two directions of a bidirectional layer share nothing but the input: the reverse one runs on the library's second
  // stream beside the forward one (in line when that stream is off, while a graph is recorded or in deterministic mode).
  auto run_direction = [&](int d) {
    float* gh = gh_all + (size_t)d * per_dir;
    const float* Wih = w + d * dir_params(mode, I, H);
    const float* Whh = Wih + (size_t)G * I; const float* bih = Whh + (size_t)G * H; const float* bhh = bih + G;
    float* act = reserve + d * dir_reserve(mode, T, B, H);
    float* aux = act + (size_t)T * B * G;
    lh_sgemm(0, 1, T * B, G, I, 1.0f, x, I, Wih, I, 0.0f, act, G);          // input projection of every step
    if (mode == 3) lh_fill(gh, 0.0f, (int64_t)B * G);
    for (int step = 0; step < T; step++) {
      const int t = d == 0 ? step : T - 1 - step, tp = d == 0 ? t - 1 : t + 1;
      float* h = y + (size_t)t * B * ldh + d * H;
      // previous state: the step processed before, or the caller's initial state ([B, H] rows), or none (zeros)
      const float* hp = step == 0 ? (hx ? hx + (size_t)d * B * H : nullptr) : y + (size_t)tp * B * ldh + d * H;
      const int ldp = step == 0 ? H : ldh;
      const float* cp = step == 0 ? (cx ? cx + (size_t)d * B * H : nullptr) : aux + (size_t)tp * B * H;
      float* a = act + (size_t)t * B * G;
      // the hidden-side product ADDS into its target (beta = 1): a product cut over K with beta = 0 would first need a launch that
      // clears it.  The LSTM adds straight into the step's input projection; the GRU keeps the hidden side apart (its n gate scales
      // it by r) in gh, which the point kernel clears after reading.
      if (mode == 2) {
        if (!lstm_fwd_step_fused(hp, ldp, Whh, a, bih, bhh, cp, aux + (size_t)t * B * H, h, B, H, ldh)) {
          if (hp) step_product_nt(hp, ldp, Whh, H, a, G, B, G, H);
          hipLaunchKernelGGL(k_lstm_fwd_point, dim3(point_grid(B, H)), dim3(TPB), 0, g_stream, a, nullptr, bih, bhh,
                             cp, aux + (size_t)t * B * H, h, B, H, ldh);
        }
      } else {
        if (!gru_fwd_step_fused(hp, ldp, Whh, a, bih, bhh, aux + (size_t)t * B * H, h, B, H, ldh)) {
          if (hp) step_product_nt(hp, ldp, Whh, H, gh, G, B, G, H);
          hipLaunchKernelGGL(k_gru_fwd_point, dim3(point_grid(B, H)), dim3(TPB), 0, g_stream, a, gh, bih, bhh, hp, ldp,
                             aux + (size_t)t * B * H, h, B, H, ldh);
        }
      }
    }
  };
  const bool fork = D == 2 && g_stream_cur == g_stream_raw;
  if (fork) { lh_side_begin(); run_direction(1); lh_side_end(); run_direction(0); lh_side_join(); }
  else for (int d = 0; d < D; d++) run_direction(d);
  lh_free_top(gh_bytes);       // stream order: the kernels above run before anything that reuses the space
  LH_CHECK_LAUNCH();
}

void lh_rnn_gated_bwd_init(int mode, const float* x, const float* hx, const float* cx, const float* y, const float* dy, const float* w,
                           float* reserve, float* dx, float beta_dx, float* dw, int T, int B, int I, int H, int bidir) {
  if (!check_shape("lh_rnn_gated_bwd", mode, T, B, I, H)) return;
  LH_REQUIRE(cx == nullptr || mode == 2, "lh_rnn_gated_bwd: only the LSTM has a cell state");
  LH_REQUIRE(beta_dx == 0.f || beta_dx == 1.f, "lh_rnn_gated_bwd: beta must be 0 or 1");
  LH_REQUIRE(x && y && dy && w && reserve && dw, "lh_rnn_gated_bwd: null operand");
  const int D = bidir ? 2 : 1, ldh = D * H, ng = gates_of(mode), G = ng * H;
  LZ_ENTER();
  lazy::rd_f(x, (int64_t)T * B * I); lazy::rd_f(y, (int64_t)T * B * ldh); lazy::rd_f(dy, (int64_t)T * B * ldh); lazy::rd_f(w, (int64_t)D * dir_params(mode, I, H));
  lazy::rd_f(hx, (int64_t)D * B * H); lazy::rd_f(cx, (int64_t)D * B * H); lazy::rw_f(reserve, (int64_t)D * dir_reserve(mode, T, B, H));
  lazy::rw_f(dw, (int64_t)D * dir_params(mode, I, H));
  if (dx) beta_dx = lazy::beta_f(dx, (int64_t)T * B * I, beta_dx);
  // scratch from the top of the arena: recurrent gradient [B, H], cell gradient [B, H], column sums [2G],
  // and for the GRU the hidden-side pre-activation gradients of every step [T, B, G]
  const size_t n_bh = (size_t)B * H, n_dgh = mode == 3 ? (size_t)T * B * G : 0;
  const size_t per_dir = 2 * n_bh + 2 * (size_t)G + n_dgh;
  const size_t bytes = (size_t)D * per_dir * sizeof(float);
  float* scratch = (float*)lh_malloc_uninit(bytes);
  if (scratch == nullptr) return;
  // each direction has its own scratch and its own part of dw, and runs on its own stream (see the forward pass); the input
  // gradient, to which both add, is formed afterwards on the caller's stream
  auto run_direction = [&](int d) {
    float* carry = scratch + (size_t)d * per_dir; float* dc = carry + n_bh; float* colsum = dc + n_bh; float* dgh = colsum + 2 * (size_t)G;
    const size_t off = d * dir_params(mode, I, H);
    const float* Wih = w + off; const float* Whh = Wih + (size_t)G * I;
    float* dWih = dw + off; float* dWhh = dWih + (size_t)G * I; float* dbih = dWhh + (size_t)G * H; float* dbhh = dbih + G;
    float* act = reserve + d * dir_reserve(mode, T, B, H);
    const float* aux = act + (size_t)T * B * G;
    for (int k = 0; k < T; k++) {
      const int t = d == 0 ? T - 1 - k : k;                        // reverse of the forward processing order
      const int tp = d == 0 ? t - 1 : t + 1;                       // the step whose state this one consumed
      const bool has_prev = d == 0 ? t > 0 : t < T - 1;
      const float* h0 = hx ? hx + (size_t)d * B * H : nullptr;      // read only by the step the forward pass processed first
      const float* c0 = cx ? cx + (size_t)d * B * H : nullptr;
      float* a = act + (size_t)t * B * G;
      const float* dyt = dy + (size_t)t * B * ldh + d * H;
      if (mode == 2) {
        hipLaunchKernelGGL(k_lstm_bwd_point, dim3(point_grid(B, H)), dim3(TPB), 0, g_stream, a, aux + (size_t)t * B * H,
                           has_prev ? aux + (size_t)tp * B * H : c0, dyt, carry, dc, k == 0 ? 1 : 0, B, H, ldh);
        if (has_prev) lh_sgemm(0, 0, B, H, G, 1.0f, a, G, Whh, H, 1.0f, carry, H);       // into the carry the point kernel has just cleared
      } else {
        float* g = dgh + (size_t)t * B * G;
        hipLaunchKernelGGL(k_gru_bwd_point, dim3(point_grid(B, H)), dim3(TPB), 0, g_stream, a, g, aux + (size_t)t * B * H,
                           has_prev ? y + (size_t)tp * B * ldh + d * H : h0, has_prev ? ldh : H, dyt, carry, k == 0 ? 1 : 0, B, H, ldh);
        if (has_prev) lh_sgemm(0, 0, B, H, G, 1.0f, g, G, Whh, H, 1.0f, carry, H);
      }
    }
    const float* hid = mode == 2 ? act : dgh;                       // gradients of the hidden-side pre-activations
    lh_sgemm(1, 0, G, I, T * B, 1.0f, act, G, x, I, 1.0f, dWih, I);
    if (T > 1) {
      // dW_hh += sum_t hid_t^T h_{prev(t)}: forward pairs (t, t-1), reverse pairs (t, t+1)
      const float* A = d == 0 ? hid + (size_t)B * G : hid;
      const float* Bm = d == 0 ? y + d * H : y + (size_t)B * ldh + d * H;
      lh_sgemm(1, 0, G, H, (T - 1) * B, 1.0f, A, G, Bm, ldh, 1.0f, dWhh, H);
    }
    // the first processed step's pair is (its hidden-side gradients, the initial state)
    if (hx) lh_sgemm(1, 0, G, H, B, 1.0f, hid + (size_t)(d == 0 ? 0 : T - 1) * B * G, G, hx + (size_t)d * B * H, H, 1.0f, dWhh, H);
    lh_sum_dim(act, colsum, 1, T * B, G);
    hipLaunchKernelGGL(k_add_into, dim3((unsigned)cdiv(G, TPB)), dim3(TPB), 0, g_stream, dbih, colsum, G);
    if (mode == 3) lh_sum_dim(dgh, colsum + G, 1, T * B, G);
    hipLaunchKernelGGL(k_add_into, dim3((unsigned)cdiv(G, TPB)), dim3(TPB), 0, g_stream, dbhh, mode == 3 ? colsum + G : colsum, G);
  };
  const bool fork = D == 2 && g_stream_cur == g_stream_raw;
  if (fork) { lh_side_begin(); run_direction(1); lh_side_end(); run_direction(0); lh_side_join(); }
  else for (int d = 0; d < D; d++) run_direction(d);
  if (dx)
    for (int d = 0; d < D; d++)
      lh_sgemm(0, 0, T * B, I, G, 1.0f, reserve + d * dir_reserve(mode, T, B, H), G, w + d * dir_params(mode, I, H), I, d == 0 ? beta_dx : 1.0f, dx, I);
  lh_free_top(bytes);
  LH_CHECK_LAUNCH();
}

}  // extern "C"
