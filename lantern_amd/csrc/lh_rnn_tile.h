// One 16 x 16 (x BT) output tile of  out[b, j] = sum_k in[b, k] * W[j, k]  on the matrix pipes: the shared core of the Elman
// recurrence step (lh_rnn.hip) and of the per-step products of the LSTM / GRU layers (lh_rnn_gated.hip).
#pragma once
#include "lh_common.h"

namespace lh {
struct RnnPre { float a, b, c; };        // what a finishing lane fetched before the arithmetic (pre) for its output stage (done)

// A block produces 16 outputs j (rows of W: hidden units, gate rows) for 16 * BT batch rows: BT 16 x 16 accumulator tiles of v_mfma_f32_16x16x4_f32 that share
// the weight operand.  The reduction over k is cut NW ways: wavefront w takes the groups of 16 consecutive k numbered
// w, w + NW, ...; inside a group lane l reads four consecutive k (one 16-byte load) of weight row j0 + l % 16 and of batch
// row b0 + l % 16 (and b0 + 16 + l % 16), k = 16 * group + 4 * (l / 16) + (0..3), and component c of those loads feeds matrix
// step c (which k a step contracts does not matter as long as both operands agree).  All loads of a wavefront are issued
// before the first matrix instruction (NIT groups of 16-byte registers), so a step pays the memory latency once.
// The partial tiles are added through LDS, and thread t finishes output t (and t + 256) of the block's.
//   W [NJ rows, K], row stride ldw;  in [B rows, K], row stride ld;  pre(b, c) / done(b, c, sum, fetched) with j = j0 + c.
// Needs K % 4 == 0 and 16-byte aligned rows of both operands; both operands below 2 GiB.
// Measured at T 185, B 32, H 800 (200 blocks with BT = 1): 5.0 us per step against 7.9 for the vector form; two batch tiles
// per block (100 blocks) 7.2 us, eight wavefronts per block 5.1 us: BT = 1, NW = 4 is what gets launched.
typedef float rnn_f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned rnn_u32x4 __attribute__((ext_vector_type(4)));
constexpr int RNN_RSRC_FLAGS = 0x00020000;
constexpr unsigned RNN_OOB = 0x80000000u;
// The partial tiles of the block's NW wavefronts: red[w * 256 * BT + (tile * 4 + v) * 64 + lane] = accumulator register v of
// wavefront w (batch row 4 * (lane / 16) + v of the tile, column lane % 16), complete after the __syncthreads() this ends with.
//   wrow: the row of W that column lane % 16 of the tile stands for, or -1 (the caller's mapping: consecutive rows for a plain
//   product, gate-major rows for a layer whose block owns all gates of a few units);  wbytes: size of W.
template <int NIT, int BT, int NW>
__device__ __forceinline__ void rnn_tile_partials(const float* __restrict__ W, int ldw, size_t wbytes, int wrow, const float* __restrict__ in, int ld, int K, int B,
                                                  int b0, float* red) {
  const int t = threadIdx.x, wave = t >> 6, lane = t & 63, r = lane & 15, kg = lane >> 4;
  const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc((void*)W, 0, (int)wbytes, RNN_RSRC_FLAGS);
  const __amdgpu_buffer_rsrc_t rh = __builtin_amdgcn_make_buffer_rsrc((void*)in, 0, (int)(((size_t)(B - 1) * ld + K) * 4), RNN_RSRC_FLAGS);
  const unsigned ow = wrow >= 0 ? (unsigned)wrow * (unsigned)ldw * 4u : RNN_OOB;
  const unsigned oh0 = b0 + r < B ? (unsigned)(b0 + r) * (unsigned)ld * 4u : RNN_OOB;
  const unsigned oh1 = b0 + 16 + r < B ? (unsigned)(b0 + 16 + r) * (unsigned)ld * 4u : RNN_OOB;
  rnn_u32x4 wv[NIT], h0[NIT], h1[NIT];
#pragma unroll
  for (int i = 0; i < NIT; i++) {
    const int k = 16 * (wave + NW * i) + 4 * kg;
    const bool in_k = k < K;                                   // K % 4 == 0: the group of four is inside the row or outside
    wv[i] = __builtin_amdgcn_raw_buffer_load_b128(rw, in_k ? (int)(ow + 4u * k) : (int)RNN_OOB, 0, 0);
    h0[i] = __builtin_amdgcn_raw_buffer_load_b128(rh, in_k ? (int)(oh0 + 4u * k) : (int)RNN_OOB, 0, 0);
    if (BT == 2) h1[i] = __builtin_amdgcn_raw_buffer_load_b128(rh, in_k ? (int)(oh1 + 4u * k) : (int)RNN_OOB, 0, 0);
  }
  __builtin_amdgcn_sched_barrier(0);             // every load is in flight before the first matrix instruction waits for one
  rnn_f32x4 a0 = {0.f, 0.f, 0.f, 0.f}, a1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < NIT; i++) {
#pragma unroll
    for (int c = 0; c < 4; c++) {
      const float wc = __uint_as_float(wv[i][c]);
      a0 = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(h0[i][c]), wc, a0, 0, 0, 0);
      if (BT == 2) a1 = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(h1[i][c]), wc, a1, 0, 0, 0);
    }
  }
  // D layout of a 16 x 16 tile: lane holds column lane % 16, rows (batch) 4 * (lane / 16) + v
  float* my = red + wave * (256 * BT);
#pragma unroll
  for (int v = 0; v < 4; v++) { my[v * 64 + lane] = a0[v]; if (BT == 2) my[(4 + v) * 64 + lane] = a1[v]; }
  __syncthreads();
}

template <int NIT, int BT, int NW, class Pre, class Done>
__device__ __forceinline__ void rnn_tile_mfma(const float* __restrict__ W, int ldw, int NJ, const float* __restrict__ in, int ld, bool use_in, int K, int B,
                                              int j0, int b0, float* red, Pre pre, Done done) {
  const int t = threadIdx.x, r = t & 15;
  // the outputs this thread finishes: index o = slot * 64 + lane' with slot = tile * 4 + v (accumulator register v of
  // tile `tile`), lane' = 16 * (row / 4 within the tile) + column
  int ob[BT], oc[BT]; bool fin[BT]; RnnPre f[BT];
#pragma unroll
  for (int q = 0; q < BT; q++) {
    const int o = (t & 255) + 256 * q, slot = o >> 6, ln = o & 63;
    ob[q] = b0 + 16 * (slot >> 2) + 4 * (ln >> 4) + (slot & 3); oc[q] = ln & 15;
    fin[q] = t < 256 && ob[q] < B && j0 + oc[q] < NJ;
    f[q] = {0.f, 0.f, 0.f};
    if (fin[q]) f[q] = pre(ob[q], oc[q]);
  }
  float tot[BT];
#pragma unroll
  for (int q = 0; q < BT; q++) tot[q] = 0.f;
  if (use_in) {
    rnn_tile_partials<NIT, BT, NW>(W, ldw, (((size_t)NJ - 1) * ldw + K) * 4, j0 + r < NJ ? j0 + r : -1, in, ld, K, B, b0, red);
#pragma unroll
    for (int q = 0; q < BT; q++) {
      const int o = (t & 255) + 256 * q;
#pragma unroll
      for (int w = 0; w < NW; w++) tot[q] += red[w * (256 * BT) + o];
    }
  }
#pragma unroll
  for (int q = 0; q < BT; q++) if (fin[q]) done(ob[q], oc[q], tot[q], f[q]);
}

// LH_RNN_MFMA=0 in the environment keeps the recurrent layers off the kernels built on rnn_tile_mfma.
static inline bool rnn_mfma_enabled() {
  static int on = -1;
  if (on < 0) { const char* e = getenv("LH_RNN_MFMA"); on = (e && e[0] == '0') ? 0 : 1; }
  return on != 0;
}

}  // namespace lh
