// conv2D_batch forward, input gradient and filter gradient (NCHW fp32 cross-correlation) as
// implicit GEMM on fp32 MFMA.  Reference behaviour being replaced: CPU:532-692 (im2col +
// SGEMM per sample) and CDN:515-880 (cuDNN forward / backward-data / backward-filter / bias).
//
//   forward         Y[k, (n,p,q)]   = sum_{(c,r,s)} W[k, (c,r,s)]   * X[(c,r,s), (n,p,q)]
//   input gradient  dX[c, (n,h,w)] += sum_{(k,r,s)} Wt[c, (k,r,s)]  * dY[(k,r,s), (n,h,w)]
//   filter gradient dW[k, (c,r,s)] += sum_{(n,p,q)} dY[k, (n,p,q)]  * X[(n,p,q), (c,r,s)]
//
// Algorithmic work of each: 2*N*K*C*R*S*P*Q flop.
#include "lh_igemm.h"
#include <map>
#include <tuple>
using namespace lh;

namespace {
// Slices of the filter-gradient reduction that measured fastest, per convolution shape (filled on first use).
struct BwdfKey {
  int v[11];
  bool operator<(const BwdfKey& o) const { for (int i = 0; i < 11; i++) if (v[i] != o.v[i]) return v[i] < o.v[i]; return false; }
};
struct BwdfPlan { int bm, bn, split, twopass; };     // twopass: the slices go to scratch blocks and a second kernel adds them up (no atomic adds)
static std::map<BwdfKey, BwdfPlan> g_bwdf_split;

constexpr int TPB = 256;

struct ConvDims { int N, C, H, W, K, R, S, sH, sW, pH, pW, P, Q; };

static bool make_dims(ConvDims& d, int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW) {
  if (N < 1 || C < 1 || H < 1 || W < 1 || K < 1 || R < 1 || S < 1 || sH < 1 || sW < 1 || pH < 0 || pW < 0) return false;
  if (H + 2 * pH < R || W + 2 * pW < S) return false;
  d = {N, C, H, W, K, R, S, sH, sW, pH, pW, (H + 2 * pH - R) / sH + 1, (W + 2 * pW - S) / sW + 1};
  const int64_t lim = 0x20000000LL;   // 2 GiB of fp32 per tensor: byte offsets of the buffer loads stay below 2^31
  if ((int64_t)N * C * H * W >= lim || (int64_t)N * K * d.P * d.Q >= lim || (int64_t)K * C * R * S >= lim) return false;
  return true;
}

// ---- B operand of the forward pass: im2col gather of x --------------------------------------
// column j = (n, p, q) fixed per thread; k = (c, r, s) is uniform across a wavefront.
struct LoadConvFwdB {
  static constexpr bool ALONG_K = false;
  static constexpr bool VEC4 = false;
  static constexpr bool SPLIT = false;
  const float* base; uint32_t nbytes;
  int C, H, W, sH, sW, pH, pW, HW;
  FastDiv dPQ, dQ, dRS, dS;
  struct State { int pix, h0, w0; bool valid; };     // pix = n*C*H*W + h0*W + w0 (may be negative)
  __device__ __forceinline__ void init(State& s, int j, int ncols) const {
    s.valid = j < ncols;
    uint32_t n, pq, p, q;
    dPQ.divmod(s.valid ? j : 0, n, pq); dQ.divmod(pq, p, q);
    s.h0 = (int)p * sH - pH; s.w0 = (int)q * sW - pW;
    s.pix = (int)n * C * HW + s.h0 * W + s.w0;
  }
  __device__ __forceinline__ uint32_t off1(const State& s, int k, int kend, int e) const {
    uint32_t c, rs, r, ss;
    dRS.divmod(k + e, c, rs); dS.divmod(rs, r, ss);
    const int tap = ((int)c * H + (int)r) * W + (int)ss;       // wave-uniform
    const bool ok = s.valid && k + e < kend && (unsigned)(s.h0 + (int)r) < (unsigned)H && (unsigned)(s.w0 + (int)ss) < (unsigned)W;
    return ok ? (uint32_t)(s.pix + tap) * 4u : LH_OOB;
  }
};

// ---- B operand of the input gradient: gather of dy ------------------------------------------------
// column j = (n, h, w) of dx fixed per thread; k = (ko, r, s) uniform across a wavefront.
struct LoadConvBwdDataB {
  static constexpr bool ALONG_K = false;
  static constexpr bool VEC4 = false;
  static constexpr bool SPLIT = false;
  const float* base; uint32_t nbytes;
  int K, P, Q, PQ;
  FastDiv dHW, dW, dRS, dS, dsH, dsW;
  int pH, pW;
  struct State { int nbase, hh, ww; bool valid; };
  __device__ __forceinline__ void init(State& s, int j, int ncols) const {
    s.valid = j < ncols;
    uint32_t n, hw, h, w;
    dHW.divmod(s.valid ? j : 0, n, hw); dW.divmod(hw, h, w);
    s.nbase = (int)n * K * PQ; s.hh = (int)h + pH; s.ww = (int)w + pW;
  }
  __device__ __forceinline__ uint32_t off1(const State& s, int k, int kend, int e) const {
    uint32_t ko, rs, r, ss;
    dRS.divmod(k + e, ko, rs); dS.divmod(rs, r, ss);
    const int th = s.hh - (int)r, tw = s.ww - (int)ss;
    uint32_t p, ph, q, qw;
    dsH.divmod(th < 0 ? 0 : th, p, ph); dsW.divmod(tw < 0 ? 0 : tw, q, qw);
    const bool ok = s.valid && k + e < kend && th >= 0 && tw >= 0 && ph == 0 && qw == 0 && (int)p < P && (int)q < Q;
    return ok ? (uint32_t)(s.nbase + ((int)ko * P + (int)p) * Q + (int)q) * 4u : LH_OOB;
  }
};

// ---- fast B operands for channel counts that are a multiple of the k-slab (16) -------------------------
// The reduction index is ordered tap-major, channel-minor: k = tap*CH + ch.  A 16-wide k-slab
// then lies inside one filter tap, so the tap decode and the bounds check are done once per
// slab on wave-uniform values and each element costs an add and a select.  The filter operand
// is brought into the matching [row][tap][ch] layout by a small transform kernel.
//
// Forward: column j = (n, p, q); element = x[n][ch][p*sH - pH + r][q*sW - pW + s], tap = r*S + s.
struct LoadConvFwdTapB {
  static constexpr bool ALONG_K = false;
  static constexpr bool VEC4 = false;
  static constexpr bool SPLIT = true;
  static constexpr bool STEP = true;
  const float* base; uint32_t nbytes;
  int C, H, W, sH, sW, pH, pW, HW;
  FastDiv dPQ, dQ, dC, dS;
  // inside a tap the next slab is the same pixels, bk channel planes further on
  __device__ __forceinline__ uint32_t step_bytes(int bk) const { return (uint32_t)(bk * HW) * 4u; }
  __device__ __forceinline__ int run_slabs(int k, int bk) const {
    uint32_t tap, ch;
    dC.divmod(k, tap, ch);
    return (C % bk) ? 1 : (C - (int)ch) / bk;
  }
  struct State { int pix, h0, w0; bool valid; };
  __device__ __forceinline__ void init(State& s, int j, int ncols) const {
    s.valid = j < ncols;
    uint32_t n, pq, p, q;
    dPQ.divmod(s.valid ? j : 0, n, pq); dQ.divmod(pq, p, q);
    s.h0 = (int)p * sH - pH; s.w0 = (int)q * sW - pW;
    s.pix = (int)n * C * HW + s.h0 * W + s.w0;
  }
  // per-lane part: the pixel under the tap of this group of four k (same tap for all four), or LH_OOB
  __device__ __forceinline__ uint32_t voff(const State& s, int k, int kend) const {
    uint32_t tap, ch, r, ss;
    dC.divmod(k, tap, ch); dS.divmod(tap, r, ss);                 // wave-uniform
    const bool ok = s.valid && k < kend && (unsigned)(s.h0 + (int)r) < (unsigned)H && (unsigned)(s.w0 + (int)ss) < (unsigned)W;
    return ok ? (uint32_t)(s.pix + (int)r * W + (int)ss) * 4u : LH_OOB;
  }
  // wave-uniform part: the channel plane of element e
  __device__ __forceinline__ uint32_t soff(int k, int e) const {
    uint32_t tap, ch;
    dC.divmod(k, tap, ch);
    return (uint32_t)(((int)ch + e) * HW) * 4u;
  }
};
// Input gradient for one residue class of output pixels (h = aH + sH*h', w = aW + sW*w'): only
// the taps r = r0 + sH*tr, s = s0 + sW*ts reach it, and on the class grid the gather is a
// stride-1 correlation:  dy[n][ko][h' + offH - tr][w' + offW - ts],  k = (tr*Sc + ts)*K + ko.
struct LoadConvBwdDataTapB {
  static constexpr bool ALONG_K = false;
  static constexpr bool VEC4 = false;
  static constexpr bool SPLIT = true;
  static constexpr bool STEP = true;
  const float* base; uint32_t nbytes;
  int K, P, Q, PQ, offH, offW;
  FastDiv dPIX, dWc, dK, dSc;       // class-grid pixels per sample, class-grid width, K, taps per row
  __device__ __forceinline__ uint32_t step_bytes(int bk) const { return (uint32_t)(bk * PQ) * 4u; }
  __device__ __forceinline__ int run_slabs(int k, int bk) const {
    uint32_t tap, ko;
    dK.divmod(k, tap, ko);
    return (K % bk) ? 1 : (K - (int)ko) / bk;
  }
  struct State { int nbase, hq, wq; bool valid; };
  __device__ __forceinline__ void init(State& s, int j, int ncols) const {
    s.valid = j < ncols;
    uint32_t n, pix, h, w;
    dPIX.divmod(s.valid ? j : 0, n, pix); dWc.divmod(pix, h, w);
    s.nbase = (int)n * K * PQ; s.hq = (int)h + offH; s.wq = (int)w + offW;
  }
  __device__ __forceinline__ uint32_t voff(const State& s, int k, int kend) const {
    uint32_t tap, ko, tr, ts;
    dK.divmod(k, tap, ko); dSc.divmod(tap, tr, ts);               // wave-uniform
    const int p = s.hq - (int)tr, q = s.wq - (int)ts;
    const bool ok = s.valid && k < kend && (unsigned)p < (unsigned)P && (unsigned)q < (unsigned)Q;
    return ok ? (uint32_t)(s.nbase + p * Q + q) * 4u : LH_OOB;
  }
  __device__ __forceinline__ uint32_t soff(int k, int e) const {
    uint32_t tap, ko;
    dK.divmod(k, tap, ko);
    return (uint32_t)(((int)ko + e) * PQ) * 4u;
  }
};

// ---- A operand of the filter gradient: dy rows, reduction index (n, p, q) ------------------------------
// VEC: PQ % 4 == 0 and dy 16-byte aligned (one 16-byte load per group of four reduction indices).
// CARRY (PQ >= 4): the group's first index is decoded once and the other three follow by stepping with at most one carry
// into the next sample, instead of one division each.
// PAD (maps whose P*Q is not a multiple of 4): the reduction runs over N * PQP indices, PQP = P*Q rounded up to a multiple of 4,
// so that a group of four never crosses into the next sample and is one 16-byte load (4-byte aligned) again.  The indices
// from P*Q to PQP - 1 of a sample stand for zeros: the last group of a sample, which has P*Q % 4 real elements, is loaded
// from 4 - P*Q % 4 elements further down (inside the row) and moved up by the kernel (keep(), lh_keep_first), so nothing
// outside the row is read.  dPQ divides by PQP; the other operand uses the same numbering.
template <bool VEC, bool CARRY = false, bool PAD = false>
struct LoadConvBwdFilterA {
  static constexpr bool ALONG_K = true;
  static constexpr bool VEC4 = VEC || PAD;
  static constexpr bool SPLIT = false;
  static constexpr bool MASKED = PAD;
  const float* base; uint32_t nbytes;
  int K, PQ;
  FastDiv dPQ;
  static constexpr bool STEP = !PAD;
  // a slab that lies inside one sample is followed, inside that sample, by the same offsets bk elements further on
  __device__ __forceinline__ uint32_t step_bytes(int bk) const { return (uint32_t)bk * 4u; }
  __device__ __forceinline__ int run_slabs(int k, int bk) const {
    uint32_t n, pq;
    dPQ.divmod(k, n, pq);
    return (int)pq + bk > PQ ? 1 : (PQ - (int)pq) / bk;
  }
  struct State { int rowoff; bool valid; };
  __device__ __forceinline__ void init(State& s, int i, int nrows) const { s.valid = i < nrows; s.rowoff = (s.valid ? i : 0) * PQ; }
  static __device__ __forceinline__ float4 fix(const float4 v, uint32_t keep) { return lh_keep_first(v, keep); }
  // PAD: the offset of the group's load and how many of its elements are real (the load starts 4 - keep elements early)
  __device__ __forceinline__ uint32_t off_keep(const State& s, int kk, int kend, uint32_t& keep) const {
    uint32_t n, pq;
    dPQ.divmod(kk, n, pq);
    const int left = PQ - (int)pq;
    keep = (uint32_t)(left < 4 ? left : 4);
    return (s.valid && kk < kend) ? (uint32_t)((int)n * K * PQ + s.rowoff + (int)pq - (4 - (int)keep)) * 4u : LH_OOB;
  }
  __device__ __forceinline__ uint32_t off1(const State& s, int kk, int kend, int e) const {
    // VEC: the reduction length N*PQ is a multiple of 4 too, so the group at e == 0 is all in or all out
    uint32_t n, pq;
    if (CARRY && !VEC) {
      dPQ.divmod(kk, n, pq);
      pq += (uint32_t)e;
      if (pq >= (uint32_t)PQ) { pq -= (uint32_t)PQ; n += 1; }
    } else {
      dPQ.divmod(kk + e, n, pq);
    }
    return (s.valid && kk + e < kend) ? (uint32_t)((int)n * K * PQ + s.rowoff + (int)pq) * 4u : LH_OOB;
  }
};

// ---- B operand of the filter gradient: gather of x, reduction index (n, p, q) ------------------------------
// column j = (c, r, s) fixed per thread.  MODE 1: Q % 4 == 0, the four reduction indices of a group share (n, p).
// MODE 2 (Q >= 4): the group's first index is decoded once, the others step along the row with at most one carry
// into the next row / sample.  MODE 0: one decode per index (maps narrower than 4).  MODE 3: as MODE 2 over the padded
// numbering of LoadConvBwdFilterA<.., PAD> (dPQ divides by PQP; a step past the last row is a padding index: zero).
template <int MODE>
struct LoadConvBwdFilterB {
  static constexpr bool ALONG_K = true;
  static constexpr bool VEC4 = false;
  static constexpr bool SPLIT = false;
  const float* base; uint32_t nbytes;
  int C, H, W, sH, sW, pH, pW, CHW, P, Q;
  FastDiv dPQ, dQ, dRS, dS;
  struct State { int coff, dh, dw; bool valid; };
  __device__ __forceinline__ void init(State& s, int j, int ncols) const {
    s.valid = j < ncols;
    uint32_t c, rs, r, ss;
    dRS.divmod(s.valid ? j : 0, c, rs); dS.divmod(rs, r, ss);
    s.coff = (int)c * H * W; s.dh = (int)r - pH; s.dw = (int)ss - pW;
  }
  __device__ __forceinline__ uint32_t off1(const State& s, int kk, int kend, int e) const {
    uint32_t n, pq, p, q;
    dPQ.divmod(MODE == 0 ? kk + e : kk, n, pq); dQ.divmod(pq, p, q);
    if (MODE != 0) q += (uint32_t)e;
    if ((MODE == 2 || MODE == 3) && q >= (uint32_t)Q) {
      q -= (uint32_t)Q; p += 1;
      if (MODE == 2 && p >= (uint32_t)P) { p = 0; n += 1; }
    }
    const int h = (int)p * sH + s.dh, w = (int)q * sW + s.dw;
    const bool ok = s.valid && kk + e < kend && (MODE != 3 || p < (uint32_t)P) && (unsigned)h < (unsigned)H && (unsigned)w < (unsigned)W;
    return ok ? (uint32_t)((int)n * CHW + s.coff + h * W + w) * 4u : LH_OOB;
  }
};

// ---- B operand of the filter gradient, lanes along the columns: filters without padding whose rows are 5 taps and wider ----
// Column j = (c, r, s) is fixed per lane and contributes c*H*W + r*W + s; the reduction index (n, p, q) is the same in all lanes
// of a wavefront and contributes n*C*H*W + p*sH*W + q*sW, decoded on the scalar unit into the scalar-offset operand of the load:
// no per-lane arithmetic per element at all (LoadConvBwdFilterB decodes and bounds-checks every element in vector registers,
// which is what bounds the filter gradient of a 21x11 filter).  A wavefront's load covers 64 consecutive (c, r, s): runs of S
// consecutive floats.  Without padding every tap of every output pixel lies inside the image, so there is nothing to check.
// PADNUM: the padded numbering of LoadConvBwdFilterA<.., PAD> (dPQ divides by PQP; indices from P*Q on are zeros).
// The elements of a group that lie past the end of the slice or are padding indices are cleared on the way to LDS (keep, fix);
// their scalar offsets are 0, so what is loaded for them is inside the tensor.
template <bool PADNUM>
struct LoadConvBwdFilterSplitB {
  static constexpr bool ALONG_K = false;
  static constexpr bool VEC4 = false;
  static constexpr bool SPLIT = true;
  static constexpr bool STEP = false;
  static constexpr bool MASKED = true;
  const float* base; uint32_t nbytes;
  int C, H, W, sH, sW, pH, pW, CHW, P, Q;
  FastDiv dPQ, dQ, dRS, dS;
  struct State { int off; bool valid; };
  __device__ __forceinline__ void init(State& s, int j, int ncols) const {
    s.valid = j < ncols;
    uint32_t c, rs, r, ss;
    dRS.divmod(s.valid ? j : 0, c, rs); dS.divmod(rs, r, ss);
    s.off = (int)c * H * W + (int)r * W + (int)ss;
  }
  __device__ __forceinline__ uint32_t voff(const State& s, int k, int kend) const { return (s.valid && k < kend) ? (uint32_t)s.off * 4u : LH_OOB; }
  __device__ __forceinline__ uint32_t keep(int k, int kend) const {
    int left = kend - k;
    if (PADNUM) { uint32_t n, pq; dPQ.divmod(k, n, pq); const int real = P * Q - (int)pq; left = left < real ? left : real; }
    return (uint32_t)(left < 0 ? 0 : (left > 4 ? 4 : left));
  }
  // the four scalar offsets of the group at k (all scalar arithmetic): one decode, then steps along the row with the carries
  __device__ __forceinline__ void soff4(int k, int kend, uint32_t (&so)[4]) const {
    uint32_t n, pq, p, q;
    dPQ.divmod(k, n, pq); dQ.divmod(pq, p, q);          // (with PADNUM a group starts on a real index: P*Q is not a multiple of 4)
    int off = (int)n * CHW + (int)p * sH * W + (int)q * sW;
    bool real = true;
    uint32_t r0, r1, r2, r3;
    auto step = [&](uint32_t& out, int e) {
      out = (real && k + e < kend) ? (uint32_t)off * 4u : 0u;
      q += 1; off += sW;
      if ((int)q == Q) {
        q = 0; p += 1; off += sH * W - Q * sW;
        if ((int)p == P) {
          if (PADNUM) real = false;                       // what is left of the group are padding indices
          else { p = 0; n += 1; off = (int)n * CHW; }
        }
      }
    };
    step(r0, 0); step(r1, 1); step(r2, 2); step(r3, 3);
    so[0] = r0; so[1] = r1; so[2] = r2; so[3] = r3;
  }
  static __device__ __forceinline__ float4 fix(const float4 v, uint32_t keep) {
    float4 r;
    r.x = keep > 0 ? v.x : 0.f; r.y = keep > 1 ? v.y : 0.f; r.z = keep > 2 ? v.z : 0.f; r.w = keep > 3 ? v.w : 0.f;
    return r;
  }
};

// ---- epilogue writing an NCHW activation: row i = channel, column j = (n, u, v) on a grid of
//      Wc columns; the element lands at out[n][i][aH + eH*u][aW + eW*v] of an image W wide with PIX pixels.
struct EpiConvOut {
  static constexpr bool STATS = false;
  static constexpr bool SLICED = false;
  float* out; const float* bias; int chan, PIX, W, eH, eW, aH, aW; float beta;
  int relu = 0;             // complete sums are stored as max(v, 0); a launch that adds partial sums leaves that to a pass of its own (conv_fwd_impl)
  int zfill2 = 0;           // the grid is every second pixel of every second row of an image with even sides (a 1x1 filter, stride 2):
                            // the element is stored together with the three zeros of its 2x2 cell, so the output needs no clearing
  FastDiv dPIXc, dWc;
  struct Col { int off; bool valid; };
  __device__ __forceinline__ Col col(int j, int N) const {
    Col c; c.valid = j < N;
    uint32_t n, pix, u, v; dPIXc.divmod(c.valid ? j : 0, n, pix); dWc.divmod(pix, u, v);
    c.off = (int)n * chan * PIX + (aH + eH * (int)u) * W + aW + eW * (int)v;
    return c;
  }
  // lean stores: element (i, j) at lane_bytes(col(j)) + i * row_bytes() from `out` (the tensor is below 2 GiB); the bias of
  // the row and the clamp are applied to the value on its way (lean_fix)
  static constexpr bool LEAN = true;
  static constexpr bool LEAN_FIX = true;
  __device__ __forceinline__ bool lean_ok(int M) const { return (M & 7) == 0; }
  __device__ __forceinline__ float lean_fix(float v, int row) const {
    if (bias) v += bias[row];
    if (relu) v = v < 0.f ? 0.f : v;
    return v;
  }
  __device__ __forceinline__ float* lean_base() const { return out; }
  __device__ __forceinline__ uint32_t lane_bytes(const Col& c) const { return (uint32_t)c.off * 4u; }
  __device__ __forceinline__ uint32_t row_bytes() const { return (uint32_t)PIX * 4u; }
  __device__ __forceinline__ uint32_t cell_row_bytes() const { return (uint32_t)W * 4u; }
  __device__ __forceinline__ int lean_mode() const { return zfill2 ? 2 : (beta == 0.f ? 0 : 1); }
  __device__ __forceinline__ float lean_scale() const { return 1.f; }
  // part: 0 = complete sum; 1 = first partial, 2 = later partial (atomic adds onto a prepared output)
  __device__ __forceinline__ void store(const Col& c, int i, int M, float v, int part) const {
    if (!c.valid || i >= M) return;
    float* p = out + c.off + i * PIX;
    if (bias && part < 2) v += bias[i];
    if (relu && part == 0) v = v < 0.f ? 0.f : v;
    if (zfill2) {             // only set for overwriting, complete sums (host side)
      *reinterpret_cast<float2*>(p) = make_float2(v, 0.f);
      *reinterpret_cast<float2*>(p + W) = make_float2(0.f, 0.f);
      return;
    }
    if (part) atomicAdd(p, v);
    else *p = beta == 0.f ? v : v + beta * *p;
  }
};
// The same epilogue, also leaving per-channel (sum, sum of squares) of every 32- or 64-column piece in `partial`.
struct EpiConvOutStats : EpiConvOut {
  static constexpr bool STATS = true;
  float* partial; int slotBase, slotsTotal;      // partial[channel][slot] = (sum, sum of squares)
};
static EpiConvOut make_epi(float* out, const float* bias, int chan, int Himg, int Wimg, float beta) {   // dense: grid == image
  EpiConvOut ep; ep.out = out; ep.bias = bias; ep.chan = chan; ep.PIX = Himg * Wimg; ep.W = Wimg; ep.eH = 1; ep.eW = 1; ep.aH = 0; ep.aW = 0; ep.beta = beta;
  ep.dPIXc.init(Himg * Wimg); ep.dWc.init(Wimg);
  return ep;
}

// Several filter layouts in one launch (the copies of all of a network's filters, made again after an optimizer step: dozens of
// tensors of a few KB to a few MB each, whose one-launch-per-copy form is bound by the launches).  Job j owns blocks
// [start[j], start[j+1]); its parameters are those of build_filter_layout.
constexpr int LAYOUT_BATCH = 48;
struct LayoutJobs {
  const float* w[LAYOUT_BATCH]; float* dst[LAYOUT_BATCH];
  int kind[LAYOUT_BATCH]; int prm[LAYOUT_BATCH][LAYOUT_PRM];
  int start[LAYOUT_BATCH + 1]; int njobs;
};
static_assert(sizeof(LayoutJobs) <= 4096, "kernel arguments are limited to 4 KB");
__global__ void __launch_bounds__(TPB) k_filter_layouts(const LayoutJobs jobs) {
  int j = 0;
  while (j + 1 < jobs.njobs && (int)blockIdx.x >= jobs.start[j + 1]) j++;
  const float* __restrict__ w = jobs.w[j]; float* __restrict__ wt = jobs.dst[j];
  const int* p = jobs.prm[j];
  const int kind = jobs.kind[j];
  int64_t i = (int64_t)((int)blockIdx.x - jobs.start[j]) * TPB + threadIdx.x;
  const int64_t st = (int64_t)(jobs.start[j + 1] - jobs.start[j]) * TPB;
  if (kind == LAYOUT_KRSC) {
    const int C = p[1], RS = p[2]; const int64_t n = (int64_t)p[0] * C * RS;
    for (; i < n; i += st) {
      int c = (int)(i % C); int64_t t = i / C; int rs = (int)(t % RS); int64_t k = t / RS;
      wt[i] = w[(k * C + c) * RS + rs];
    }
  } else if (kind == LAYOUT_CTK) {
    const int K = p[0], C = p[1], R = p[2], S = p[3], r0 = p[4], s0 = p[5], sH = p[6], sW = p[7], Rc = p[8], Sc = p[9];
    const int64_t n = (int64_t)Rc * Sc * K * C;
    for (; i < n; i += st) {
      int k = (int)(i % K); int64_t t = i / K; int ts = (int)(t % Sc); t /= Sc; int tr = (int)(t % Rc); int c = (int)(t / Rc);
      wt[i] = w[(((int64_t)k * C + c) * R + (r0 + sH * tr)) * S + (s0 + sW * ts)];
    }
  } else {
    const int K = p[0], C = p[1], RS = p[2]; const int64_t n = (int64_t)K * C * RS;
    for (; i < n; i += st) {
      int rs = (int)(i % RS); int64_t t = i / RS; int k = (int)(t % K); int c = (int)(t / K);
      wt[i] = w[((int64_t)k * C + c) * RS + rs];
    }
  }
}
// w[K][C][RS] -> wt[K][RS][C]   (forward, tap-major reduction order)
__global__ void __launch_bounds__(TPB) k_filter_to_krsc(const float* __restrict__ w, float* __restrict__ wt, int C, int RS, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n; i += st) {
    int c = (int)(i % C); int64_t t = i / C; int rs = (int)(t % RS); int64_t k = t / RS;
    wt[i] = w[(k * C + c) * RS + rs];
  }
}
// w[K][C][R][S] -> wt[C][tr][ts][K] for the taps r = r0 + sH*tr (tr < Rc), s = s0 + sW*ts (ts < Sc)
__global__ void __launch_bounds__(TPB) k_filter_to_ctk(const float* __restrict__ w, float* __restrict__ wt, int K, int C, int R, int S,
                                                       int r0, int s0, int sH, int sW, int Rc, int Sc, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n; i += st) {
    int k = (int)(i % K); int64_t t = i / K; int ts = (int)(t % Sc); t /= Sc; int tr = (int)(t % Rc); int c = (int)(t / Rc);
    wt[i] = w[(((int64_t)k * C + c) * R + (r0 + sH * tr)) * S + (s0 + sW * ts)];
  }
}
// w[K][C][RS] -> wt[C][K][RS]
__global__ void __launch_bounds__(TPB) k_filter_transpose(const float* __restrict__ w, float* __restrict__ wt, int K, int C, int RS, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n; i += st) {
    int rs = (int)(i % RS); int64_t t = i / RS; int k = (int)(t % K); int c = (int)(t / K);
    wt[i] = w[((int64_t)k * C + c) * RS + rs];
  }
}
// db[k] += sum over n, p, q of dy: block (k, slice of the batch); slices add their sums atomically.
// MASK: the gradient is one that relu_grad has yet to mask: dy = y > 0 ? dy : 0 is written back on the way.
// VEC: P*Q is a multiple of 4 and the tensors are 16-byte aligned (every channel image then starts on a 16-byte boundary).
// (sample, pixel) pairs are flattened over the threads: small maps (P*Q below the block size) keep every lane busy and the
// loads of one thread do not wait for each other.  Both forms add the same terms in the same order.
template <bool VEC, bool MASK>
__global__ void __launch_bounds__(TPB) k_conv_bwd_bias(const float* __restrict__ y, float* dy, float* db, int N, int K, int PQ, int n_per) {
  __shared__ float sm[17];
  const int k = blockIdx.x, n0 = blockIdx.y * n_per, n1 = min(N, n0 + n_per);
  float acc = 0.f;
  if (VEC) {
    const int PQ4 = PQ >> 2, total = (n1 - n0) * PQ4;
#pragma unroll 2
    for (int i = threadIdx.x; i < total; i += TPB) {
      const int dn = i / PQ4, l = i - dn * PQ4;
      const int64_t o = (((int64_t)(n0 + dn) * K + k) * PQ4 + l) * 4;
      float4 g = *reinterpret_cast<const float4*>(dy + o);
      if (MASK) {
        const float4 a = *reinterpret_cast<const float4*>(y + o);
        g.x = a.x > 0.f ? g.x : 0.f; g.y = a.y > 0.f ? g.y : 0.f; g.z = a.z > 0.f ? g.z : 0.f; g.w = a.w > 0.f ? g.w : 0.f;
        *reinterpret_cast<float4*>(dy + o) = g;
      }
      acc += (g.x + g.y) + (g.z + g.w);
    }
  } else {
    const int total = (n1 - n0) * PQ;
#pragma unroll 4
    for (int i = threadIdx.x; i < total; i += TPB) {
      const int dn = i / PQ, l = i - dn * PQ;
      const int64_t o = ((int64_t)(n0 + dn) * K + k) * PQ + l;
      float g = dy[o];
      if (MASK) { g = y[o] > 0.f ? g : 0.f; dy[o] = g; }
      acc += g;
    }
  }
  acc = lh_block_sum(acc, sm);
  if (threadIdx.x == 0) atomicAdd(db + k, acc);
}
static void bias_grad_launch(const float* y, float* dy, float* db, int N, int K, int PQ) {
  int bslices = g_deterministic ? 1 : (int)cdiv(4 * (int64_t)g_num_cu, K);     // slices of the batch add atomically: one slice when the order must be fixed
  if (bslices > N) bslices = N;
  if (bslices < 1) bslices = 1;
  const int n_per = (int)cdiv(N, bslices);
  const dim3 grid(K, (unsigned)cdiv(N, n_per));
  const bool vec = PQ % 4 == 0 && (((uintptr_t)y | (uintptr_t)dy) & 15) == 0;
  if (y && vec) hipLaunchKernelGGL((k_conv_bwd_bias<true, true>), grid, dim3(TPB), 0, g_stream, y, dy, db, N, K, PQ, n_per);
  else if (y) hipLaunchKernelGGL((k_conv_bwd_bias<false, true>), grid, dim3(TPB), 0, g_stream, y, dy, db, N, K, PQ, n_per);
  else if (vec) hipLaunchKernelGGL((k_conv_bwd_bias<true, false>), grid, dim3(TPB), 0, g_stream, y, dy, db, N, K, PQ, n_per);
  else hipLaunchKernelGGL((k_conv_bwd_bias<false, false>), grid, dim3(TPB), 0, g_stream, y, dy, db, N, K, PQ, n_per);
}

}  // namespace
namespace lh {
// The copy kernel of a filter layout, on the current stream (prm as the convolution entry points fill it in).
void build_filter_layout(int kind, const int* p, const float* w, float* dst) {
  if (kind == LAYOUT_KRSC) {                 // {K, C, RS}
    const int64_t n = (int64_t)p[0] * p[1] * p[2];
    hipLaunchKernelGGL(k_filter_to_krsc, dim3(stream_grid(n, TPB * 4)), dim3(TPB), 0, g_stream, w, dst, p[1], p[2], n);
  } else if (kind == LAYOUT_CTK) {           // {K, C, R, S, r0, s0, sH, sW, Rc, Sc}
    const int64_t n = (int64_t)p[8] * p[9] * p[0] * p[1];
    hipLaunchKernelGGL(k_filter_to_ctk, dim3(stream_grid(n, TPB * 4)), dim3(TPB), 0, g_stream, w, dst, p[0], p[1], p[2], p[3], p[4], p[5], p[6], p[7], p[8], p[9], n);
  } else {                                   // LAYOUT_CKRS {K, C, RS}
    const int64_t n = (int64_t)p[0] * p[1] * p[2];
    hipLaunchKernelGGL(k_filter_transpose, dim3(stream_grid(n, TPB * 4)), dim3(TPB), 0, g_stream, w, dst, p[0], p[1], p[2], n);
  }
}
static int64_t layout_elems(int kind, const int* p) { return kind == LAYOUT_CTK ? (int64_t)p[8] * p[9] * p[0] * p[1] : (int64_t)p[0] * p[1] * p[2]; }
// Several layouts at once, on the current stream: one launch per LAYOUT_BATCH of them.
void build_filter_layouts(int n, const int* kinds, const int* const* prms, const float* const* ws, float* const* dsts) {
  for (int first = 0; first < n; first += LAYOUT_BATCH) {
    const int m = n - first < LAYOUT_BATCH ? n - first : LAYOUT_BATCH;
    if (m == 1) { build_filter_layout(kinds[first], prms[first], ws[first], dsts[first]); continue; }
    LayoutJobs jobs;
    jobs.njobs = m; jobs.start[0] = 0;
    for (int j = 0; j < m; j++) {
      jobs.w[j] = ws[first + j]; jobs.dst[j] = dsts[first + j]; jobs.kind[j] = kinds[first + j];
      for (int q = 0; q < LAYOUT_PRM; q++) jobs.prm[j][q] = prms[first + j][q];
      jobs.start[j + 1] = jobs.start[j] + stream_grid(layout_elems(kinds[first + j], prms[first + j]), TPB * 4);
    }
    for (int j = m; j < LAYOUT_BATCH; j++) { jobs.w[j] = nullptr; jobs.dst[j] = nullptr; jobs.kind[j] = 0; for (int q = 0; q < LAYOUT_PRM; q++) jobs.prm[j][q] = 0; jobs.start[j + 1] = jobs.start[m]; }
    hipLaunchKernelGGL(k_filter_layouts, dim3(jobs.start[m]), dim3(TPB), 0, g_stream, jobs);
  }
}
}  // namespace lh
namespace {
// The filter in the layout a launch reads: the library's kept copy (written now if it is stale), or, where none is kept,
// scratch from the arena top that the caller pops behind the launch (stream order keeps that safe).
struct FilterCopy { float* p = nullptr; size_t scratch = 0; };
static bool filter_copy(FilterCopy& fc, const float* w, size_t wbytes, int kind, const int* prm, size_t bytes) {
  bool build = false;
  fc.scratch = 0;
  fc.p = lazy::layout_lookup(w, wbytes, kind, prm, bytes, build);
  if (fc.p == nullptr) {
    fc.p = (float*)lh_malloc_uninit(bytes);
    if (fc.p == nullptr) return false;
    fc.scratch = bytes; build = true;
  }
  if (build) build_filter_layout(kind, prm, w, fc.p);
  return true;
}

#ifndef LH_CONV_BK
#define LH_CONV_BK 16
#endif
constexpr int CONV_BK = LH_CONV_BK;      // k-slab of the forward / input-gradient kernels
#ifndef LH_BWDF_BK
#define LH_BWDF_BK 32
#endif
constexpr int BWDF_BK = LH_BWDF_BK;      // k-slab of the filter-gradient kernel
// Forward / input-gradient launch.  A grid with few tiles per CU leaves CUs idle in its last wave
// of blocks; such shapes run stream-K instead (largest tile, two workers per CU, every worker the
// same number of k-slabs).  `zero_out`/`zero_n`: the output to clear first when the epilogue
// overwrites (beta = 0), because shared tiles are completed with atomic adds.
// All blocks of a launch that fit on the chip at once form a round; tiles take about the same
// time, so a last round with only a few tiles leaves most CUs idle for a whole tile time.  When the
// tile count is a little above a whole number of rounds, the columns of the surplus tiles are
// computed by a second launch with smaller tiles, which spreads them over four times as many CUs.
// Tile choice of the forward / input-gradient launches.  With a reduction of at most 512 (1x1 filters over up to 512
// channels) a tile is finished after at most 32 slabs, and the fixed cost per tile (pipeline fill, epilogue) and the
// low occupancy of the 128-wide tiles weigh more than their better operand reuse: measured over the ResNet-50 layers,
// 64x64 tiles are 4-17 % faster there and equal or slower for longer reductions.
static inline TilePick pick_tile_conv(int M, int N, int K) {
  if (K <= 512) return {64, 64};
  return pick_tile(M, N);
}
template <int BM, int BN, int SBM, int SBN, class AL, class BL, class EP>
static bool launch_rounds(const AL& al, const BL& bl, const EP& ep, int M, int N, int K) {
  constexpr int rem_div = 3;        // split when the surplus is at most a third of a round
  const int64_t tm = cdiv(M, BM), tn = cdiv(N, BN), tiles = tm * tn;
  const int64_t slots = (int64_t)igemm_blocks_per_cu<BM, BN, CONV_BK, AL, BL, EP>() * g_num_cu;
  const int64_t full = tiles / slots, rem = tiles - full * slots;
  if (rem_div > 0 && full >= 1 && rem > 0 && rem * rem_div <= slots) {
    const int col1 = (int)((full * slots / tm) * BN);
    if (col1 > 0 && col1 < N)
      return igemm_launch<BM, BN, CONV_BK>(al, bl, ep, M, N, K, 1, 0, 0, col1) && igemm_launch<SBM, SBN, CONV_BK>(al, bl, ep, M, N, K, 1, 0, col1, N);
  }
  return igemm_launch<BM, BN, CONV_BK>(al, bl, ep, M, N, K, 1);
}

// The launch plans of a forward / input-gradient product.  0: the built-in rule (stream-K for few tiles over a long
// reduction, else the tile pick_tile_conv names).  1-3: plain tiles 128x128, 64x128, 64x64.  4-7: stream-K over
// 128x128 / 64x128 tiles with two or three workers per CU.  8-9: stream-K over 64x64 tiles with four or eight workers per
// CU, for products so small that even their 64x64 tiles leave most CUs with one block whose loads nothing hides.
// 10: 32x128 tiles (32-deep slabs) for products of at most 32 rows, whose 64-row tiles would be half empty.
// 11-12: stream-K over 64x64 tiles with one worker per 32 or 8 slabs: a handful of tiles under a very long reduction (a filter
// as large as the map: a fully connected layer), where a worker per CU would mean hundreds of atomic adds onto each element.
// 13-15: whole 64x64 / 64x128 / 128x128 tiles, the last ones (what is left over a multiple of the compute units) cut into
// slices along the reduction and finished by whichever slice arrives last (igemm_launch_shared_tail).
constexpr int N_PLANS = 16;
// LH_FORCE_M32 in the environment: products of at most 32 rows always take the 32-row tile (for tests of that tile; the
// measured choice may well be another one).
static inline bool force_m32() { return getenv("LH_FORCE_M32") != nullptr; }
// LH_FORCE_PLAN=n in the environment: forward / input-gradient products take launch plan n where it is valid (for tests that
// compare the plans' results with each other).
// LH_NO_PADDED_REDUCTION=1 (tests): the filter gradient over maps whose pixel count is not a multiple of 4 keeps to 4-byte loads
static inline bool no_padded_reduction() { const char* e = getenv("LH_NO_PADDED_REDUCTION"); return e && e[0] == '1'; }
// LH_NO_SPLIT_GATHER=1 (tests): the filter gradient of unpadded filters with wide rows keeps to the per-element gather of x
static inline bool no_split_gather() { const char* e = getenv("LH_NO_SPLIT_GATHER"); return e && e[0] == '1'; }
static inline int force_plan() { const char* e = getenv("LH_FORCE_PLAN"); return e ? atoi(e) : -1; }
// LH_FORCE_STATS_TILE=f: the same for the forward launches that leave batch-norm statistics behind (f as in conv_fwd_impl's `run`).
static inline int force_stats_tile() { const char* e = getenv("LH_FORCE_STATS_TILE"); return e ? atoi(e) : -1; }
template <class AL, class BL, class EP>
static bool plan_valid(int plan, const EP& ep, int M, int K, bool can_zero) {
  if (plan == 0) return true;
  if (plan == 10) return M <= 32;
  if ((plan == 1 || plan == 4 || plan == 6) && M <= 64) return false;
  if (plan >= 13 && plan <= 15) return !g_deterministic && g_stream_cur == g_stream_raw && cdiv(K, CONV_BK) >= 8 && (plan != 15 || M > 64);   // (same bits in every run, but not those of the whole-tile plans)
  if ((plan >= 4 && plan <= 9) || plan == 11 || plan == 12) {
    if (g_deterministic) return false;        // partial sums meet in atomic adds, in whatever order the blocks arrive
    return (ep.beta == 1.f || can_zero) && cdiv(K, CONV_BK) >= (plan >= 11 ? 64 : 16);
  }
  return true;
}
static bool g_launch_partial = false;     // the last launch_plan combined partial sums with atomic adds (stream-K): its epilogue saw incomplete sums
template <class AL, class BL, class EP>
static bool launch_plan(int plan, const AL& al, const BL& bl, const EP& ep, int M, int N, int K, float* zero_out, int64_t zero_n, bool prezeroed) {
  g_launch_partial = false;
  if (plan == 10) return igemm_launch<32, 128, 32>(al, bl, ep, M, N, K, 1);
  if (plan == 13) return igemm_launch_shared_tail<64, 64, CONV_BK>(al, bl, ep, M, N, K);
  if (plan == 14) return igemm_launch_shared_tail<64, 128, CONV_BK>(al, bl, ep, M, N, K);
  if (plan == 15) return igemm_launch_shared_tail<128, 128, CONV_BK>(al, bl, ep, M, N, K);
  if (plan >= 11) {
    g_launch_partial = true;
    const int64_t units = cdiv(M, 64) * cdiv(N, 64) * cdiv(K, CONV_BK);
    int64_t workers = cdiv(units, plan == 11 ? 32 : 8);
    if (workers > 16 * (int64_t)g_num_cu) workers = 16 * (int64_t)g_num_cu;
    if (ep.beta == 0.f && !prezeroed) lh_fill(zero_out, 0.f, zero_n);
    return igemm_launch<64, 64, CONV_BK>(al, bl, ep, M, N, K, 1, (int)workers);
  }
  if (plan >= 4) {
    g_launch_partial = true;
    const int workers = (plan >= 8 ? (plan == 8 ? 4 : 8) : (plan >= 6 ? 3 : 2)) * g_num_cu;
    if (ep.beta == 0.f && !prezeroed) lh_fill(zero_out, 0.f, zero_n);
    if (plan >= 8) return igemm_launch<64, 64, CONV_BK>(al, bl, ep, M, N, K, 1, workers);
    if (plan == 4 || plan == 6) return igemm_launch<128, 128, CONV_BK>(al, bl, ep, M, N, K, 1, workers);
    return igemm_launch<64, 128, CONV_BK>(al, bl, ep, M, N, K, 1, workers);
  }
  if (plan == 1) return launch_rounds<128, 128, 64, 64>(al, bl, ep, M, N, K);
  if (plan == 2) return launch_rounds<64, 128, 64, 64>(al, bl, ep, M, N, K);
  if (plan == 3) return igemm_launch<64, 64, CONV_BK>(al, bl, ep, M, N, K, 1);
  const int64_t t128 = cdiv(M, 128) * cdiv(N, 128), t64 = cdiv(M, 64) * cdiv(N, 128);
  const int workers = 2 * g_num_cu;
  const bool few = (M > 64 ? t128 : t64) < 6 * (int64_t)g_num_cu;
  const int64_t slabs = cdiv(K, CONV_BK);
  // long reductions only: a worker's share must span many slabs for the per-segment set-up to pay off
  if (!g_deterministic && few && slabs >= 64 && slabs * (M > 64 ? t128 : t64) >= 48 * (int64_t)workers && (ep.beta == 1.f || zero_out != nullptr || prezeroed)) {
    if (ep.beta == 0.f && !prezeroed) lh_fill(zero_out, 0.f, zero_n);
    g_launch_partial = true;
    if (M > 64) return igemm_launch<128, 128, CONV_BK>(al, bl, ep, M, N, K, 1, workers);
    return igemm_launch<64, 128, CONV_BK>(al, bl, ep, M, N, K, 1, workers);
  }
  TilePick tp = pick_tile_conv(M, N, K);
  if (tp.bm == 128) return launch_rounds<128, 128, 64, 64>(al, bl, ep, M, N, K);
  if (tp.bn == 128) return launch_rounds<64, 128, 64, 64>(al, bl, ep, M, N, K);
  return igemm_launch<64, 64, CONV_BK>(al, bl, ep, M, N, K, 1);
}

// Which plan is fastest depends on how the tiles fall onto the chip, on the length of the reduction and on the
// gather; it is measured once per shape, on a call whose epilogue overwrites (so that repeating the launch is
// harmless), and remembered per loader / epilogue combination.
struct PlanKey {
  int v[7];
  bool operator<(const PlanKey& o) const { for (int i = 0; i < 7; i++) if (v[i] != o.v[i]) return v[i] < o.v[i]; return false; }
};
template <class AL, class BL, class EP>
static bool launch_tiles(const AL& al, const BL& bl, const EP& ep, int M, int N, int K, float* zero_out = nullptr, int64_t zero_n = 0, bool prezeroed = false) {
  static std::map<PlanKey, int> chosen;
  const bool can_zero = zero_out != nullptr || prezeroed;
  if (M <= 32 && force_m32()) return launch_plan(10, al, bl, ep, M, N, K, zero_out, zero_n, prezeroed);
  const int forced = force_plan();
  if (forced >= 0 && forced < N_PLANS && plan_valid<AL, BL, EP>(forced, ep, M, K, can_zero)) return launch_plan(forced, al, bl, ep, M, N, K, zero_out, zero_n, prezeroed);
  // Deterministic mode keeps the measured choice among the plans whose tiles are finished by one block each: they add the same
  // terms in the same order whatever the tile shape, so which of them runs changes no bit (tests/test_parity_conv.py compares them).
  if (!g_tune_enabled || 2.0 * M * N * (double)K < g_tune_min_flop) return launch_plan(0, al, bl, ep, M, N, K, zero_out, zero_n, prezeroed);
  const PlanKey key = {{M, N, K, ep.eH | (g_deterministic ? 1 << 16 : 0), ep.eW, ep.W, ep.PIX}};
  auto it = chosen.find(key);
  if (it != chosen.end()) {
    g_plans_remembered++;
    const int plan = plan_valid<AL, BL, EP>(it->second, ep, M, K, can_zero) ? it->second : 0;
    return launch_plan(plan, al, bl, ep, M, N, K, zero_out, zero_n, prezeroed);
  }
  // tuned only on a call that may be repeated: an overwriting epilogue onto an output this launch alone writes
  if (g_capturing || ep.beta != 0.f || prezeroed) return launch_plan(0, al, bl, ep, M, N, K, zero_out, zero_n, prezeroed);
  LaunchTimer timer;
  if (!timer.ok) return launch_plan(0, al, bl, ep, M, N, K, zero_out, zero_n, prezeroed);
  int best = 0; float best_ms = 3.0e38f, base_ms = 0.f;
  for (int plan = 0; plan < N_PLANS; plan++) {
    if (!plan_valid<AL, BL, EP>(plan, ep, M, K, can_zero)) continue;
    const float ms = timer.ms([&]() { return launch_plan(plan, al, bl, ep, M, N, K, zero_out, zero_n, prezeroed); });
    if (ms < 0.f || failed()) return false;
    if (plan == 0) base_ms = ms;
    if (ms < best_ms * 0.98f) { best_ms = ms; best = plan; }      // a later plan must win by 2 % to displace an earlier one
  }
  chosen[key] = best; g_plans_measured++;
  if (getenv("LH_TUNE_VERBOSE")) fprintf(stderr, "conv product M%d N%d K%d (stride %d,%d): plan %d, %.3f ms (built-in rule %.3f ms)\n", M, N, K, ep.eH, ep.eW, best, best_ms, base_ms);
  return true;                                               // the timed launches have produced the result
}

// Where the statistics pieces of a forward launch lie (see bn_finalize_conv_partials).
struct StatLayout { int col1, g_main, slots_main, g_rem, slots_rem; int sliced = 0; };      // sliced: whole tiles and slices of the last ones (igemm_launch_shared_tail)

// The tile plan launch_tiles would choose, for a launch that also leaves statistics pieces.  Returns false (and
// launches nothing) for shapes that take the stream-K path, whose tiles are finished by several blocks.
template <class AL, class BL>
static bool plan_tiles_stats(int M, int N, int K, StatLayout& L, int& bm, int& bn, int force = 0 /* 1-3: the tile of launch plan 1-3; 5-7: 64x64 / 64x128 / 128x128 tiles with the last ones sliced */) {
  const int64_t t128 = cdiv(M, 128) * cdiv(N, 128), t64 = cdiv(M, 64) * cdiv(N, 128);
  const bool few = (M > 64 ? t128 : t64) < 6 * (int64_t)g_num_cu;
  const int64_t slabs = cdiv(K, CONV_BK);
  if (!g_deterministic && few && slabs >= 64 && slabs * (M > 64 ? t128 : t64) >= 48 * (int64_t)(2 * g_num_cu)) return false;
  TilePick tp = pick_tile_conv(M, N, K);
  if ((force == 1 || force == 7) && M > 64) tp = {128, 128}; else if (force == 2 || force == 6) tp = {64, 128}; else if (force == 3 || force == 5) tp = {64, 64};
  L.sliced = (force == 5 || force == 6 || (force == 7 && M > 64)) && !g_deterministic && g_stream_cur == g_stream_raw && cdiv(K, CONV_BK) >= 8;
  bm = tp.bm; bn = tp.bn;
  L.col1 = N; L.g_main = bn / 2; L.g_rem = 32; L.slots_rem = 0;
  if (bn == 128 && !L.sliced) {        // the surplus-tile split of launch_rounds
    const int64_t tm = cdiv(M, bm), tn = cdiv(N, bn), tiles = tm * tn;
    const int64_t slots = (int64_t)(bm == 128 ? igemm_blocks_per_cu<128, 128, CONV_BK, AL, BL, EpiConvOutStats>()
                                              : igemm_blocks_per_cu<64, 128, CONV_BK, AL, BL, EpiConvOutStats>()) * g_num_cu;
    const int64_t full = tiles / slots, rem = tiles - full * slots;
    if (full >= 1 && rem > 0 && rem * 3 <= slots) {
      const int c1 = (int)((full * slots / tm) * bn);
      if (c1 > 0 && c1 < N) L.col1 = c1;
    }
  }
  L.slots_main = (int)cdiv(L.col1, bn) * 2;
  L.slots_rem = L.col1 < N ? (int)cdiv(N - L.col1, 64) * 2 : 0;
  return true;
}
template <class AL, class BL>
static bool launch_tiles_stats(const AL& al, const BL& bl, EpiConvOutStats ep, int M, int N, int K, const StatLayout& L, int bm, int bn) {
  ep.slotBase = 0;
  bool ok;
  if (L.sliced) return bm == 128 ? igemm_launch_shared_tail<128, 128, CONV_BK>(al, bl, ep, M, N, K) : (bn == 128 ? igemm_launch_shared_tail<64, 128, CONV_BK>(al, bl, ep, M, N, K) : igemm_launch_shared_tail<64, 64, CONV_BK>(al, bl, ep, M, N, K));
  if (bm == 128) ok = igemm_launch<128, 128, CONV_BK>(al, bl, ep, M, N, K, 1, 0, 0, L.col1);
  else if (bn == 128) ok = igemm_launch<64, 128, CONV_BK>(al, bl, ep, M, N, K, 1, 0, 0, L.col1);
  else ok = igemm_launch<64, 64, CONV_BK>(al, bl, ep, M, N, K, 1, 0, 0, L.col1);
  if (ok && L.col1 < N) { ep.slotBase = L.slots_main; ok = igemm_launch<64, 64, CONV_BK>(al, bl, ep, M, N, K, 1, 0, L.col1, N); }
  return ok;
}

struct BnStatsOut {
  float* save_mean; float* save_invstd; float* run_mean; float* run_var; float eps, factor;
  // optional: the normalisation itself (out = bn(y) [relu] or relu(bn(y) + shortcut)); when the launch left statistics pieces the
  // apply pass consumes them directly and `applied` is set, otherwise the caller runs it from the saved statistics
  const float* gamma = nullptr; const float* beta = nullptr; const float* shortcut = nullptr; float* out = nullptr; int relu = 0; bool applied = false;
};
}  // namespace

// Forward convolution; with `bn` also the batch-norm statistics of its output channels.
static void conv_fwd_impl(const float* x, const float* w, const float* bias, float* y,
                          int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW, BnStatsOut* bn, int relu = 0) {
  KernelCat kc_(CAT_CONV_FWD);
  ConvDims d;
  LH_REQUIRE(make_dims(d, N, C, H, W, K, R, S, sH, sW, pH, pW), "lh_conv2d_fwd: bad shape N%d C%d H%d W%d K%d R%d S%d s(%d,%d) p(%d,%d)", N, C, H, W, K, R, S, sH, sW, pH, pW);
  const int RS = R * S, CRS = C * RS, PQ = d.P * d.Q;
  const uint32_t wbytes = (uint32_t)((size_t)K * CRS * 4), xbytes = (uint32_t)((size_t)N * C * H * W * 4);
  EpiConvOut ep = make_epi(y, bias, K, d.P, d.Q, 0.f);
  ep.relu = (relu && bn == nullptr) ? 1 : 0;
  g_launch_partial = false;
  bool ok;
  if (C % CONV_BK == 0 && ((uintptr_t)w & 15) == 0) {
    // tap-major reduction order; a 1x1 filter already has that layout
    const float* wk = w;
    size_t scratch = 0;
    if (RS > 1) {
      const int prm[LAYOUT_PRM] = {K, C, RS};
      FilterCopy fc;
      if (!filter_copy(fc, w, wbytes, LAYOUT_KRSC, prm, wbytes)) return;
      wk = fc.p; scratch = fc.scratch;
    }
    LoadPlainK<true> al; al.base = wk; al.nbytes = wbytes; al.ld = CRS;
    LoadConvFwdTapB bl; bl.base = x; bl.nbytes = xbytes; bl.C = C; bl.H = H; bl.W = W; bl.sH = sH; bl.sW = sW; bl.pH = pH; bl.pW = pW; bl.HW = H * W;
    bl.dPQ.init(PQ); bl.dQ.init(d.Q); bl.dC.init(C); bl.dS.init(S);
    StatLayout L; int bm = 0, bn_ = 0;
    if (bn && bias == nullptr && plan_tiles_stats<LoadPlainK<true>, LoadConvFwdTapB>(K, N * PQ, CRS, L, bm, bn_)) {
      // the tile shape of this launch is measured once per shape (the launch overwrites y and its statistics pieces, so
      // repeating it is harmless) and remembered
      static std::map<PlanKey, int> chosen;
      const PlanKey key = {{K, N * PQ, CRS, H, W, sH, R}};
      const bool tunable = g_tune_lookup && 2.0 * K * CRS * (double)N * PQ >= g_tune_min_flop;
      int force = 0;
      auto run = [&](int f) {           // 0: the rule's tile, 1-3: a forced tile, 4: unfused (any launch plan, then a pass over y), 5-7: 64x64 / 64x128 / 128x128 tiles, the last ones sliced
        if (f == 4) {
          if (!launch_tiles(al, bl, ep, K, N * PQ, CRS, y, (int64_t)N * K * PQ)) return false;
          lh_bn_stats(y, bn->save_mean, bn->save_invstd, nullptr, nullptr, N, K, PQ, bn->eps, bn->factor);
          return !failed();
        }
        StatLayout Lf; int bmf = 0, bnf = 0;
        if (!plan_tiles_stats<LoadPlainK<true>, LoadConvFwdTapB>(K, N * PQ, CRS, Lf, bmf, bnf, f)) return false;
        const size_t pbytes = (size_t)(Lf.slots_main + Lf.slots_rem) * K * 2 * sizeof(float);
        float* partial = (float*)lh_malloc_uninit(pbytes);
        if (partial == nullptr) return false;
        EpiConvOutStats es; static_cast<EpiConvOut&>(es) = ep; es.partial = partial; es.slotBase = 0; es.slotsTotal = Lf.slots_main + Lf.slots_rem;
        bool good = launch_tiles_stats(al, bl, es, K, N * PQ, CRS, Lf, bmf, bnf);
        if (good) bn_finalize_conv_partials(partial, K, N * PQ, Lf.col1, Lf.g_main, Lf.slots_main, Lf.g_rem, bn->save_mean, bn->save_invstd, nullptr, nullptr, bn->eps, bn->factor);
        lh_free_top(pbytes);
        return good;
      };
      if (force_stats_tile() >= 0) force = force_stats_tile();
      else if (tunable) {
        auto it = chosen.find(key);
        if (it != chosen.end()) { force = it->second; g_plans_remembered++; }
        else if (g_tune_measure) {
          LaunchTimer timer;
          if (timer.ok) {
            float best_ms = 3.0e38f, base_ms = 0.f; int best = 0;
            for (int f = 0; f <= 7; f++) {
              if ((f == 1 || f == 7) && K <= 64) continue;
              if (f >= 5 && (g_deterministic || CRS < 8 * CONV_BK)) continue;
              const float ms = timer.ms([&]() { return run(f); });
              if (ms < 0.f || failed()) return;
              if (f == 0) base_ms = ms;
              if (ms < best_ms * 0.98f) { best_ms = ms; best = f; }
            }
            chosen[key] = best; force = best; g_plans_measured++;
            if (getenv("LH_TUNE_VERBOSE")) fprintf(stderr, "conv fwd+stats K%d N%d CRS%d H%d: tile plan %d, %.3f ms (built-in rule %.3f ms)\n", K, N * PQ, CRS, H, best, best_ms, base_ms);
          }
        }
      }
      if (force == 4) {           // measured: better without the statistics epilogue (stream-K or another plan, then lh_bn_stats below)
        ok = launch_tiles(al, bl, ep, K, N * PQ, CRS, y, (int64_t)N * K * PQ);
      } else {
        plan_tiles_stats<LoadPlainK<true>, LoadConvFwdTapB>(K, N * PQ, CRS, L, bm, bn_, force);
        const size_t pbytes = (size_t)(L.slots_main + L.slots_rem) * K * 2 * sizeof(float);
        float* partial = (float*)lh_malloc_uninit(pbytes);
        if (partial == nullptr) return;
        EpiConvOutStats es; static_cast<EpiConvOut&>(es) = ep; es.partial = partial; es.slotBase = 0; es.slotsTotal = L.slots_main + L.slots_rem;
        ok = launch_tiles_stats(al, bl, es, K, N * PQ, CRS, L, bm, bn_);
        if (ok && bn->out != nullptr) {
          ConvPieces cp{partial, N * PQ, L.col1, L.g_main, L.slots_main, L.g_rem, L.slots_main + L.slots_rem, bn->eps, bn->factor, bn->save_mean, bn->save_invstd, bn->run_mean, bn->run_var};
          bn_apply_from_pieces(y, cp, bn->gamma, bn->beta, bn->shortcut, bn->out, bn->relu, N, K, PQ);
          bn->applied = true;
        } else if (ok) {
          bn_finalize_conv_partials(partial, K, N * PQ, L.col1, L.g_main, L.slots_main, L.g_rem, bn->save_mean, bn->save_invstd, bn->run_mean, bn->run_var, bn->eps, bn->factor);
        }
        lh_free_top(pbytes);
        bn = nullptr;      // done
      }
    } else {
      ok = launch_tiles(al, bl, ep, K, N * PQ, CRS, y, (int64_t)N * K * PQ);
    }
    if (scratch) lh_free_top(scratch);
  } else {
    const bool avec = (CRS % 4 == 0) && (((uintptr_t)w & 15) == 0);
    LoadConvFwdB bl; bl.base = x; bl.nbytes = xbytes; bl.C = C; bl.H = H; bl.W = W; bl.sH = sH; bl.sW = sW; bl.pH = pH; bl.pW = pW; bl.HW = H * W;
    bl.dPQ.init(PQ); bl.dQ.init(d.Q); bl.dRS.init(RS); bl.dS.init(S);
    if (avec) { LoadPlainK<true> al; al.base = w; al.nbytes = wbytes; al.ld = CRS; ok = launch_tiles(al, bl, ep, K, N * PQ, CRS); }
    else { LoadPlainK<false> al; al.base = w; al.nbytes = wbytes; al.ld = CRS; ok = launch_tiles(al, bl, ep, K, N * PQ, CRS); }
  }
  if (!ok) return;
  LH_CHECK_LAUNCH();
  if (ep.relu && g_launch_partial) {      // elements finished by atomic adds have not been clamped (the others have: clamping twice changes nothing)
    lh_unary(LH_RELU, y, y, (int64_t)N * K * PQ, 0.f, 0.f);
    return;
  }
  // shapes whose launch leaves no statistics pieces: one extra pass over y
  if (bn && bn->out != nullptr && bn->shortcut == nullptr) {       // statistics pass + apply pass that combines the partial sums itself
    if (bn->relu) lh_bn_train_fwd_relu(y, bn->gamma, bn->beta, bn->run_mean, bn->run_var, bn->out, bn->save_mean, bn->save_invstd, N, K, PQ, bn->eps, bn->factor);
    else lh_bn_train_fwd(y, bn->gamma, bn->beta, bn->run_mean, bn->run_var, bn->out, bn->save_mean, bn->save_invstd, N, K, PQ, bn->eps, bn->factor);
    bn->applied = true;
  } else if (bn) {
    lh_bn_stats(y, bn->save_mean, bn->save_invstd, bn->run_mean, bn->run_var, N, K, PQ, bn->eps, bn->factor);
  }
}

extern "C" {

// What a forward convolution reads and writes, stated to the deferred-work bookkeeping; launches whatever is parked.
static void conv_fwd_declare(const float* x, const float* w, const float* bias, float* y, int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW) {
  if (!lazy::g_busy || lazy::g_replay) return;
  lazy::flush_parked();
  ConvDims d;
  if (!make_dims(d, N, C, H, W, K, R, S, sH, sW, pH, pW)) return;
  lazy::rd_f(x, (int64_t)N * C * H * W); lazy::rd_f(w, (int64_t)K * C * R * S); lazy::rd_f(bias, K); lazy::wr_f(y, (int64_t)N * K * d.P * d.Q);
}

void lh_conv2d_fwd(const float* x, const float* w, const float* bias, float* y,
                   int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW) {
  LZ_SCOPE();
  // waits for the call behind it: a batch norm of y takes its statistics from this launch's epilogue
  if (lazy::park_conv_fwd(x, w, bias, y, N, C, H, W, K, R, S, sH, sW, pH, pW)) return;
  conv_fwd_declare(x, w, bias, y, N, C, H, W, K, R, S, sH, sW, pH, pW);
  conv_fwd_impl(x, w, bias, y, N, C, H, W, K, R, S, sH, sW, pH, pW, nullptr);
}

}  // extern "C"
namespace lh {
// relu(conv(x) + bias) written once: the clamp rides in the epilogue.  Called with the operands already stated.
void conv_bwd_bias_mask_now(const float* y, float* dy, float* db, int N, int K, int PQ) {
  KernelCat kc_(CAT_CONV_BWD_FILTER);
  bias_grad_launch(y, dy, db, N, K, PQ);
  LH_CHECK_LAUNCH();
}
void conv2d_fwd_relu_now(const float* x, const float* w, const float* bias, float* y, int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW) {
  conv_fwd_impl(x, w, bias, y, N, C, H, W, K, R, S, sH, sW, pH, pW, nullptr, 1);
}
}  // namespace lh
extern "C" {

void lh_conv2d_fwd_bnstats(const float* x, const float* w, const float* bias, float* y,
                           int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW,
                           float* save_mean, float* save_invstd, float* run_mean, float* run_var, float eps, float factor) {
  LH_REQUIRE(save_mean && save_invstd, "lh_conv2d_fwd_bnstats: save_mean and save_invstd are required");
  LZ_SCOPE();
  conv_fwd_declare(x, w, bias, y, N, C, H, W, K, R, S, sH, sW, pH, pW);
  lazy::wr_f(save_mean, K); lazy::wr_f(save_invstd, K); lazy::rw_f(run_mean, K); lazy::rw_f(run_var, K);
  BnStatsOut bn{save_mean, save_invstd, run_mean, run_var, eps, factor};
  conv_fwd_impl(x, w, bias, y, N, C, H, W, K, R, S, sH, sW, pH, pW, &bn);
}

void lh_conv2d_fwd_bn_apply(const float* x, const float* w, const float* bias, float* y,
                            int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW,
                            const float* gamma, const float* beta, float* save_mean, float* save_invstd, float* run_mean, float* run_var,
                            float eps, float factor, const float* shortcut, float* out, int relu) {
  LH_REQUIRE(save_mean && save_invstd && gamma && beta && out, "lh_conv2d_fwd_bn_apply: gamma, beta, save_mean, save_invstd and out are required");
  LH_REQUIRE(shortcut == nullptr || relu, "lh_conv2d_fwd_bn_apply: the residual join is relu(bn(y) + shortcut)");
  LZ_SCOPE();
  conv_fwd_declare(x, w, bias, y, N, C, H, W, K, R, S, sH, sW, pH, pW);
  if (lazy::g_busy && !lazy::g_replay) {
    ConvDims dd;
    if (make_dims(dd, N, C, H, W, K, R, S, sH, sW, pH, pW)) {
      const int64_t no = (int64_t)N * K * dd.P * dd.Q;
      lazy::rd_f(gamma, K); lazy::rd_f(beta, K); lazy::rd_f(shortcut, no); lazy::wr_f(save_mean, K); lazy::wr_f(save_invstd, K);
      lazy::rw_f(run_mean, K); lazy::rw_f(run_var, K); lazy::wr_f(out, no);
    }
  }
  BnStatsOut bn{save_mean, save_invstd, run_mean, run_var, eps, factor};
  bn.gamma = gamma; bn.beta = beta; bn.shortcut = shortcut; bn.out = out; bn.relu = relu;
  conv_fwd_impl(x, w, bias, y, N, C, H, W, K, R, S, sH, sW, pH, pW, &bn);
  if (failed() || bn.applied) return;
  ConvDims d;
  if (!make_dims(d, N, C, H, W, K, R, S, sH, sW, pH, pW)) return;
  if (shortcut) lh_bn_apply_add_relu(y, gamma, beta, save_mean, save_invstd, shortcut, out, N, K, d.P * d.Q);
  else lh_bn_apply(y, gamma, beta, save_mean, save_invstd, out, N, K, d.P * d.Q, relu);
}

void lh_conv2d_bwd_data(const float* dy, const float* w, float* dx, float beta,
                        int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW) {
  KernelCat kc_(CAT_CONV_BWD_DATA);
  ConvDims d;
  LH_REQUIRE(make_dims(d, N, C, H, W, K, R, S, sH, sW, pH, pW), "lh_conv2d_bwd_data: bad shape");
  LH_REQUIRE(beta == 0.f || beta == 1.f, "lh_conv2d_bwd_data: beta must be 0 or 1");
  LZ_ENTER();
  lazy::rd_f(dy, (int64_t)N * K * d.P * d.Q); lazy::rd_f(w, (int64_t)K * C * R * S);
  beta = lazy::beta_f(dx, (int64_t)N * C * H * W, beta);       // a gradient buffer nobody has touched since lh_malloc is overwritten, not read
  const int RS = R * S, KRS = K * RS, HW = H * W, PQ = d.P * d.Q;
  const uint32_t dybytes = (uint32_t)((size_t)N * K * PQ * 4);
  bool ok = true;
  if (K % CONV_BK == 0) {
    // One implicit GEMM per residue class (aH, aW) of input pixels modulo the stride: no MFMA
    // work is spent on taps that cannot reach a pixel.  Stride 1 is the single class (0, 0).
    bool any_empty = false;
    for (int aH = 0; aH < sH; aH++) for (int aW = 0; aW < sW; aW++) {
      int r0 = (aH + pH) % sH, s0 = (aW + pW) % sW;
      if (r0 >= R || s0 >= S || aH >= H || aW >= W) any_empty = true;
    }
    // Stride > 1 with a filter wider than one tap: the residue classes are independent products with disjoint outputs
    // and different reduction lengths; they run as one grouped launch (longest reduction first), so the chip is
    // filled once instead of up to sH*sW times with a quarter of the columns each.
    if (sH * sW > 1 && RS > 1) {
      struct Cls { int aH, aW, r0, s0, Rc, Sc, Hc, Wc, Kred; };
      Cls cls[IGEMM_MAX_GROUPS]; int ng = 0; bool fits = true;
      for (int aH = 0; aH < sH; aH++) for (int aW = 0; aW < sW; aW++) {
        const int r0 = (aH + pH) % sH, s0 = (aW + pW) % sW;
        if (r0 >= R || s0 >= S || aH >= H || aW >= W) continue;
        if (ng == IGEMM_MAX_GROUPS) { fits = false; continue; }
        Cls c; c.aH = aH; c.aW = aW; c.r0 = r0; c.s0 = s0;
        c.Rc = (R - r0 + sH - 1) / sH; c.Sc = (S - s0 + sW - 1) / sW; c.Hc = (H - aH + sH - 1) / sH; c.Wc = (W - aW + sW - 1) / sW;
        c.Kred = c.Rc * c.Sc * K;
        cls[ng++] = c;
      }
      if (fits && ng >= 2) {
        for (int i = 1; i < ng; i++) for (int j = i; j > 0 && cls[j].Kred > cls[j - 1].Kred; j--) { Cls t = cls[j]; cls[j] = cls[j - 1]; cls[j - 1] = t; }
        if (beta == 0.f && any_empty) lh_fill(dx, 0.f, (int64_t)N * C * HW);       // pixels no class reaches
        FilterCopy fcs[IGEMM_MAX_GROUPS];
        auto release = [&]() { for (int i = ng - 1; i >= 0; i--) if (fcs[i].scratch) { lh_free_top(fcs[i].scratch); fcs[i].scratch = 0; } };
        LoadPlainK<true> al[IGEMM_MAX_GROUPS]; LoadConvBwdDataTapB bl[IGEMM_MAX_GROUPS]; EpiConvOut ep[IGEMM_MAX_GROUPS];
        int Ms[IGEMM_MAX_GROUPS], Ns[IGEMM_MAX_GROUPS], Ks[IGEMM_MAX_GROUPS];
        int64_t ntot = 0; int kmax = 0;
        for (int i = 0; i < ng; i++) {
          const Cls& c = cls[i];
          const size_t wbytes = (size_t)c.Kred * C * sizeof(float);
          const int prm[LAYOUT_PRM] = {K, C, R, S, c.r0, c.s0, sH, sW, c.Rc, c.Sc};
          if (!filter_copy(fcs[i], w, (size_t)K * C * RS * sizeof(float), LAYOUT_CTK, prm, wbytes)) { release(); return; }
          float* wt = fcs[i].p;
          al[i].base = wt; al[i].nbytes = (uint32_t)wbytes; al[i].ld = c.Kred;
          LoadConvBwdDataTapB& b = bl[i];
          b.base = dy; b.nbytes = dybytes; b.K = K; b.P = d.P; b.Q = d.Q; b.PQ = PQ;
          b.offH = (c.aH + pH - c.r0) / sH; b.offW = (c.aW + pW - c.s0) / sW;
          b.dPIX.init(c.Hc * c.Wc); b.dWc.init(c.Wc); b.dK.init(K); b.dSc.init(c.Sc);
          EpiConvOut& e = ep[i];
          e.out = dx; e.bias = nullptr; e.chan = C; e.PIX = HW; e.W = W; e.eH = sH; e.eW = sW; e.aH = c.aH; e.aW = c.aW; e.beta = beta;
          e.dPIXc.init(c.Hc * c.Wc); e.dWc.init(c.Wc);
          Ms[i] = C; Ns[i] = N * c.Hc * c.Wc; Ks[i] = c.Kred;
          ntot += Ns[i]; if (c.Kred > kmax) kmax = c.Kred;
        }
        auto run = [&](int tile) {           // 1: 128x128, 2: 64x128, 3: 64x64, 4: 32x128 (at most 32 input channels)
          if (tile == 4) return igemm_launch_grouped<32, 128, 32>(ng, al, bl, ep, Ms, Ns, Ks);
          if (tile == 1) return igemm_launch_grouped<128, 128, CONV_BK>(ng, al, bl, ep, Ms, Ns, Ks);
          if (tile == 2) return igemm_launch_grouped<64, 128, CONV_BK>(ng, al, bl, ep, Ms, Ns, Ks);
          return igemm_launch_grouped<64, 64, CONV_BK>(ng, al, bl, ep, Ms, Ns, Ks);
        };
        // tile shape: measured once per shape on an overwriting call (every pixel of a class is written by one block, so
        // repeating the launch is harmless), else the remembered one, else by the total tile count
        static std::map<PlanKey, int> chosen;
        const PlanKey key = {{N, C, H, W, K, R * 100 + S, sH * 100 + sW}};
        TilePick tp = pick_tile(C, (int)(ntot < 0x7fffffff ? ntot : 0x7fffffff));
        int tile = tp.bm == 128 ? 1 : (tp.bn == 128 ? 2 : 3);
        auto it = chosen.find(key);
        if (C <= 32 && force_m32()) tile = 4;
        else if (it != chosen.end() && g_tune_lookup) { tile = it->second; g_plans_remembered++; }
        else if (it == chosen.end() && g_tune_measure && beta == 0.f && 2.0 * C * (double)ntot * kmax >= g_tune_min_flop) {
          LaunchTimer timer;
          if (timer.ok) {
            float best_ms = 3.0e38f; int best = tile;
            for (int tcand = 1; tcand <= 4; tcand++) {
              if (tcand == 1 && C <= 64) continue;
              if (tcand == 4 && C > 32) continue;
              const float ms = timer.ms([&]() { return run(tcand); });
              if (ms < 0.f || failed()) { release(); return; }
              if (ms < best_ms * 0.98f) { best_ms = ms; best = tcand; }
            }
            chosen[key] = best; tile = best; g_plans_measured++;
            if (getenv("LH_TUNE_VERBOSE")) fprintf(stderr, "conv input gradient, stride (%d,%d), C%d H%d K%d k%d: %d classes in one launch, tile plan %d, %.3f ms\n", sH, sW, C, H, K, R, ng, best, best_ms);
          }
        }
        ok = run(tile);
        release();
        if (!ok) return;
        LH_CHECK_LAUNCH();
        return;
      }
    }
    // several classes (or an empty one) with beta = 0: clear dx once, then every class may overwrite or add
    const bool strided = sH * sW > 1;
    // 1x1 filter, stride 2, no padding, even image: the one class that has a tap writes whole 2x2 cells
    const bool cells = beta == 0.f && RS == 1 && sH == 2 && sW == 2 && pH == 0 && pW == 0 && (H % 2) == 0 && (W % 2) == 0 && (((uintptr_t)dx & 7) == 0);
    if (beta == 0.f && (any_empty || strided) && !cells) lh_fill(dx, 0.f, (int64_t)N * C * HW);
    float* zo = (beta == 0.f && !strided) ? dx : nullptr;
    const int64_t zn = (int64_t)N * C * HW;
    const bool pz = beta == 0.f && strided && !cells;
    for (int aH = 0; aH < sH && ok; aH++) for (int aW = 0; aW < sW && ok; aW++) {
      const int r0 = (aH + pH) % sH, s0 = (aW + pW) % sW;
      if (r0 >= R || s0 >= S || aH >= H || aW >= W) continue;
      const int Rc = (R - r0 + sH - 1) / sH, Sc = (S - s0 + sW - 1) / sW;
      const int Hc = (H - aH + sH - 1) / sH, Wc = (W - aW + sW - 1) / sW;
      const int Kred = Rc * Sc * K;
      LoadConvBwdDataTapB bl; bl.base = dy; bl.nbytes = dybytes; bl.K = K; bl.P = d.P; bl.Q = d.Q; bl.PQ = PQ;
      bl.offH = (aH + pH - r0) / sH; bl.offW = (aW + pW - s0) / sW;
      bl.dPIX.init(Hc * Wc); bl.dWc.init(Wc); bl.dK.init(K); bl.dSc.init(Sc);
      EpiConvOut ep; ep.out = dx; ep.bias = nullptr; ep.chan = C; ep.PIX = HW; ep.W = W; ep.eH = sH; ep.eW = sW; ep.aH = aH; ep.aW = aW; ep.beta = beta;
      ep.dPIXc.init(Hc * Wc); ep.dWc.init(Wc);
      ep.zfill2 = cells ? 1 : 0;
      if (RS == 1) {
        LoadPlainT al; al.base = w; al.nbytes = (uint32_t)((size_t)K * C * 4); al.ld = C;          // A[c][k] = w[k][c]
        ok = launch_tiles(al, bl, ep, C, N * Hc * Wc, Kred, zo, zn, pz);
      } else {
        size_t bytes = (size_t)Kred * C * sizeof(float);
        const int prm[LAYOUT_PRM] = {K, C, R, S, r0, s0, sH, sW, Rc, Sc};
        FilterCopy fc;
        if (!filter_copy(fc, w, (size_t)K * C * RS * sizeof(float), LAYOUT_CTK, prm, bytes)) return;
        LoadPlainK<true> al; al.base = fc.p; al.nbytes = (uint32_t)bytes; al.ld = Kred;
        ok = launch_tiles(al, bl, ep, C, N * Hc * Wc, Kred, zo, zn, pz);
        if (fc.scratch) lh_free_top(fc.scratch);
      }
    }
  } else {
    LoadConvBwdDataB bl; bl.base = dy; bl.nbytes = dybytes; bl.K = K; bl.P = d.P; bl.Q = d.Q; bl.PQ = PQ; bl.pH = pH; bl.pW = pW;
    bl.dHW.init(HW); bl.dW.init(W); bl.dRS.init(RS); bl.dS.init(S); bl.dsH.init(sH); bl.dsW.init(sW);
    EpiConvOut ep = make_epi(dx, nullptr, C, H, W, beta);
    if (RS == 1) {
      LoadPlainT al; al.base = w; al.nbytes = (uint32_t)((size_t)K * C * 4); al.ld = C;
      ok = launch_tiles(al, bl, ep, C, N * HW, KRS);
    } else {
      size_t bytes = (size_t)KRS * C * sizeof(float);
      const int prm[LAYOUT_PRM] = {K, C, RS};
      FilterCopy fc;
      if (!filter_copy(fc, w, bytes, LAYOUT_CKRS, prm, bytes)) return;
      float* wt = fc.p;
      if (KRS % 4 == 0) { LoadPlainK<true> al; al.base = wt; al.nbytes = (uint32_t)bytes; al.ld = KRS; ok = launch_tiles(al, bl, ep, C, N * HW, KRS); }
      else { LoadPlainK<false> al; al.base = wt; al.nbytes = (uint32_t)bytes; al.ld = KRS; ok = launch_tiles(al, bl, ep, C, N * HW, KRS); }
      if (fc.scratch) lh_free_top(fc.scratch);
    }
  }
  if (!ok) return;
  LH_CHECK_LAUNCH();
}

void lh_conv2d_bwd_filter(const float* x, const float* dy, float* dw, float* db, float beta,
                          int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW) {
  KernelCat kc_(CAT_CONV_BWD_FILTER);
  ConvDims d;
  LH_REQUIRE(make_dims(d, N, C, H, W, K, R, S, sH, sW, pH, pW), "lh_conv2d_bwd_filter: bad shape");
  LH_REQUIRE(beta == 0.f || beta == 1.f, "lh_conv2d_bwd_filter: beta must be 0 or 1");
  LZ_SCOPE();
  // relu_grad(in place) on dy still parked: the bias gradient's pass over dy applies the mask as well
  const bool bias_done = db && lazy::g_busy && !lazy::g_replay && lazy::take_relu_grad_bias(dy, db, N, K, d.P * d.Q);
  if (lazy::g_busy && !lazy::g_replay) lazy::flush_parked();
  lazy::rd_f(x, (int64_t)N * C * H * W); lazy::rd_f(dy, (int64_t)N * K * d.P * d.Q);
  beta = lazy::beta_f(dw, (int64_t)K * C * R * S, beta);
  lazy::rw_f(db, K);
  // A filter gradient issued in line must not overtake one of the same filter that is still on the side stream.
  if (g_stream_cur == g_stream_raw) side_join();
  const int CRS = C * R * S, PQ = d.P * d.Q;
  // Maps whose P*Q is not a multiple of 4 (7x7, 9x9, 81x185 ...): the reduction is numbered with every sample padded to a
  // multiple of 4, which keeps dy (and x under a 1x1 filter) on 16-byte loads (LoadConvBwdFilterA<.., PAD>); for maps of
  // 32 pixels and more, where the padding is at most a tenth of the reduction.
  const int PQP = (PQ + 3) & ~3;
  const bool padded = PQ % 4 != 0 && PQ >= 32 && d.Q >= 4 && !no_padded_reduction();
  const int64_t red = (int64_t)N * (padded ? PQP : PQ);
  LH_REQUIRE(red < 0x7fffffffLL, "lh_conv2d_bwd_filter: reduction length too large");
  const bool avec = (PQ % 4 == 0) && (((uintptr_t)dy & 15) == 0);
  const bool rowvec = (d.Q % 4 == 0);
  // The output is small (K x CRS) and the reduction long (N*P*Q): split it across blocks and
  // combine with fp32 atomic adds.
  TilePick tp = (K >= 128 && CRS >= 128) ? TilePick{128, 128} : (CRS >= 128 ? TilePick{64, 128} : TilePick{64, 64});
  int64_t tiles = cdiv(K, tp.bm) * cdiv(CRS, tp.bn);
  int max_split = (int)cdiv(red, 256); if (max_split < 1) max_split = 1;
  auto clamp_split = [&](int64_t v) { return (int)(v < 1 ? 1 : (v > max_split ? max_split : v)); };
  int split = clamp_split(cdiv(3 * (int64_t)g_num_cu, tiles));
  // How many slices pays best depends on how tiles x slices fall onto the resident block slots and on how short the
  // per-block reduction gets; it is measured once per shape (a few candidates on a scratch output) and remembered.
  const BwdfKey key = {{N, C, H, W, K, R, S, sH | (g_deterministic ? 1 << 16 : 0), sW, pH, pW}};     // deterministic mode measures among fewer forms
  const bool tunable = g_tune_lookup && max_split > 1 && 2.0 * K * CRS * (double)red >= g_tune_min_flop;
  bool tune_now = false;
  // Slices are combined either with atomic adds onto dw (cleared first when beta = 0) or in two passes: every slice writes
  // its own [K, CRS] block of scratch memory and a second kernel adds the blocks onto beta*dw in slice order.  Deterministic
  // mode always takes the second; otherwise it is part of what is measured (large filters over small maps, where a block's
  // reduction is short against the 64 KB of atomic adds it ends in, come out ahead with it).
  bool twopass = g_deterministic;
  if (tunable) {
    auto it = g_bwdf_split.find(key);
    if (it != g_bwdf_split.end()) { g_plans_remembered++; tp = TilePick{it->second.bm, it->second.bn}; tiles = cdiv(K, tp.bm) * cdiv(CRS, tp.bn); split = clamp_split(it->second.split); twopass = it->second.twopass != 0; }
    else tune_now = g_tune_measure;
  }
  if (K <= 32 && force_m32()) { tp = TilePick{32, 128}; tiles = cdiv(K, 32) * cdiv(CRS, 128); split = clamp_split(cdiv(3 * (int64_t)g_num_cu, tiles)); tune_now = false; }
  float* partial = nullptr; size_t partial_bytes = 0; int slices = 1; bool on_side = false;
  // what igemm_launch will make of `split` for the tile in tp
  auto slices_of = [&](int sp) {
    const int bk = tp.bm == 128 ? 16 : (tp.bm == 32 ? 32 : BWDF_BK);
    int64_t kper = cdiv(cdiv(red, sp), bk) * bk; if (kper < bk) kper = bk;
    return (int)cdiv(red, kper);
  };
  EpiRowMajor ep; ep.C = dw; ep.ldc = CRS; ep.alpha = 1.f; ep.beta = 1.f; ep.atomic = split > 1 ? 1 : 0;
  bool ok = false;
  auto go = [&](auto al, auto bl) {
    al.base = dy; al.nbytes = (uint32_t)((size_t)N * K * PQ * 4); al.K = K; al.PQ = PQ; al.dPQ.init(padded ? PQP : PQ);
    bl.base = x; bl.nbytes = (uint32_t)((size_t)N * C * H * W * 4); bl.C = C; bl.H = H; bl.W = W; bl.sH = sH; bl.sW = sW; bl.pH = pH; bl.pW = pW; bl.CHW = C * H * W;
    bl.P = d.P; bl.Q = d.Q; bl.dPQ.init(padded ? PQP : PQ); bl.dQ.init(d.Q); bl.dRS.init(R * S); bl.dS.init(S);
    if (tp.bm == 128) ok = igemm_launch<128, 128, 16>(al, bl, ep, K, CRS, (int)red, split);    // measured: the large tile prefers the short slab
    else if (tp.bm == 32) ok = igemm_launch<32, 128, 32>(al, bl, ep, K, CRS, (int)red, split);
    else if (tp.bn == 128) ok = igemm_launch<64, 128, BWDF_BK>(al, bl, ep, K, CRS, (int)red, split);
    else ok = igemm_launch<64, 64, BWDF_BK>(al, bl, ep, K, CRS, (int)red, split);
  };
  // 1x1, stride 1, no padding: the gather of x is a plain [C][N*PQ] matrix with the same layout as dy
  auto go_plain = [&](auto al, auto bl) {
    al.base = dy; al.nbytes = (uint32_t)((size_t)N * K * PQ * 4); al.K = K; al.PQ = PQ; al.dPQ.init(padded ? PQP : PQ);
    bl.base = x; bl.nbytes = (uint32_t)((size_t)N * C * PQ * 4); bl.K = C; bl.PQ = PQ; bl.dPQ.init(padded ? PQP : PQ);
    if (tp.bm == 128) ok = igemm_launch<128, 128, 16>(al, bl, ep, K, CRS, (int)red, split);
    else if (tp.bm == 32) ok = igemm_launch<32, 128, 32>(al, bl, ep, K, CRS, (int)red, split);
    else if (tp.bn == 128) ok = igemm_launch<64, 128, BWDF_BK>(al, bl, ep, K, CRS, (int)red, split);
    else ok = igemm_launch<64, 64, BWDF_BK>(al, bl, ep, K, CRS, (int)red, split);
  };
  const bool plain = R == 1 && S == 1 && sH == 1 && sW == 1 && pH == 0 && pW == 0;
  const bool xvec = (PQ % 4 == 0) && (((uintptr_t)x & 15) == 0);
  const bool narrow = PQ < 4 || d.Q < 4;        // the stepping loaders assume at most one carry inside a group of four
  // filters without padding whose rows are 5 taps and wider: x is gathered with the lanes along (c, r, s) (LoadConvBwdFilterSplitB)
  const bool wide_rows = pH == 0 && pW == 0 && S >= 5 && !no_split_gather();
  auto dispatch = [&]() {
    ep.atomic = (split > 1 && ep.sliceStride == 0) ? 1 : 0;
    if (wide_rows && padded) go(LoadConvBwdFilterA<false, false, true>(), LoadConvBwdFilterSplitB<true>());
    else if (wide_rows && avec) go(LoadConvBwdFilterA<true>(), LoadConvBwdFilterSplitB<false>());
    else if (padded && plain) go_plain(LoadConvBwdFilterA<false, false, true>(), LoadConvBwdFilterA<false, false, true>());
    else if (padded) go(LoadConvBwdFilterA<false, false, true>(), LoadConvBwdFilterB<3>());
    else if (plain && avec && xvec) go_plain(LoadConvBwdFilterA<true>(), LoadConvBwdFilterA<true>());
    else if (plain && !avec && !xvec && !narrow) go_plain(LoadConvBwdFilterA<false, true>(), LoadConvBwdFilterA<false, true>());
    else if (plain && !avec && !xvec) go_plain(LoadConvBwdFilterA<false>(), LoadConvBwdFilterA<false>());
    else if (narrow) { if (avec) go(LoadConvBwdFilterA<true>(), LoadConvBwdFilterB<0>()); else go(LoadConvBwdFilterA<false>(), LoadConvBwdFilterB<0>()); }
    else if (avec && rowvec) go(LoadConvBwdFilterA<true>(), LoadConvBwdFilterB<1>());
    else if (avec) go(LoadConvBwdFilterA<true>(), LoadConvBwdFilterB<2>());
    else go(LoadConvBwdFilterA<false, true>(), LoadConvBwdFilterB<2>());
  };
  // one launch of the plan in (tp, split) into `out` (accumulating), slices through `pbuf` when it is given
  auto run_plan = [&](float* out, float* pbuf, float out_beta) {
    const int sl = slices_of(split);
    if (pbuf != nullptr && sl > 1) {
      ep.C = pbuf; ep.sliceStride = (long long)K * CRS; ep.beta = 0.f;
      dispatch();
      if (ok) reduce_slices(out, CRS, K, CRS, pbuf, sl, out_beta);
    } else {
      ep.C = out; ep.sliceStride = 0; ep.beta = 1.f;
      dispatch();
    }
  };
  if (tune_now) {
    const size_t sbytes = (size_t)K * CRS * sizeof(float);
    const size_t pcap = (size_t)256 << 20;                    // two-pass candidates whose slices need more scratch than this are not tried
    const double targets[] = {1.0, 1.5, 2.0, 2.5, 3.0, 4.0, 5.0, 6.0};
    const TilePick shapes[4] = {{128, 128}, {64, 128}, {64, 64}, {32, 128}};      // the last for layers of at most 32 output channels
    // candidates first (the scratch for the two-pass ones is one block together with the output: the side stream has one block)
    struct Cand { TilePick tp; int split; };
    Cand cands[40]; int ncand = 0; size_t pmax = 0;
    for (int sh = 0; sh < 4; sh++) {
      if ((shapes[sh].bm == 128 && K < 128) || (shapes[sh].bn == 128 && CRS < 128) || (shapes[sh].bm == 32 && K > 32)) continue;
      tp = shapes[sh];
      tiles = cdiv(K, tp.bm) * cdiv(CRS, tp.bn);
      int cand[10]; int nc = 0;
      auto add = [&](int v) { for (int i = 0; i < nc; i++) if (cand[i] == v) return; cand[nc++] = v; };
      add(clamp_split((3 * (int64_t)g_num_cu) / tiles));
      for (double t : targets) add(clamp_split((int64_t)(t * g_num_cu) / tiles));
      for (int i = 0; i < nc && ncand < 40; i++) {
        cands[ncand++] = Cand{tp, cand[i]};
        const size_t pb = (size_t)slices_of(cand[i]) * sbytes;
        if (slices_of(cand[i]) > 1 && pb <= pcap && pb > pmax) pmax = pb;
      }
    }
    bool tune_side = false;
    float* scratch = (float*)scratch_take(sbytes + pmax, tune_side);
    LaunchTimer timer;
    if (scratch && timer.ok) {
      float* const pbuf = scratch + (size_t)K * CRS;
      BwdfPlan best = {tp.bm, tp.bn, split, 0}; float best_ms = 3.0e38f;
      for (int ci = 0; ci < ncand && !failed(); ci++) {
        tp = cands[ci].tp; split = cands[ci].split;
        tiles = cdiv(K, tp.bm) * cdiv(CRS, tp.bn);
        const int sl = slices_of(split);
        if (!g_deterministic || sl == 1) {
          const float ms_atomic = timer.ms([&]() { run_plan(scratch, nullptr, 1.f); return ok; });
          if (ms_atomic < 0.f) break;
          if (ms_atomic < best_ms) { best_ms = ms_atomic; best = BwdfPlan{tp.bm, tp.bn, split, 0}; }
        }
        if (sl > 1 && (size_t)sl * sbytes <= pmax) {
          const float ms_two = timer.ms([&]() { run_plan(scratch, pbuf, 1.f); return ok; });
          if (ms_two < 0.f) break;
          if (ms_two < best_ms * 0.98f) { best_ms = ms_two; best = BwdfPlan{tp.bm, tp.bn, split, 1}; }
        }
      }
      tp = TilePick{best.bm, best.bn};
      tiles = cdiv(K, tp.bm) * cdiv(CRS, tp.bn);
      split = best.split; twopass = best.twopass != 0;
      g_bwdf_split[key] = best; g_plans_measured++;
      if (getenv("LH_TUNE_VERBOSE")) fprintf(stderr, "bwd_filter N%d C%d H%d K%d k%d s%d: tile %dx%d, %lld tiles, split %d%s (%.3f ms)\n", N, C, H, K, R, sH, tp.bm, tp.bn, (long long)tiles, split, twopass ? ", two passes" : "", best_ms);
    }
    if (scratch) scratch_give(sbytes + pmax, tune_side);
    if (failed()) return;
  }
  slices = slices_of(split);
  if (g_deterministic) twopass = true;
  if (twopass && slices > 1) {
    partial_bytes = (size_t)slices * K * CRS * sizeof(float);
    partial = (float*)scratch_take(partial_bytes, on_side);
    if (partial == nullptr) return;
  }
  if (beta == 0.f && partial == nullptr) lh_fill(dw, 0.f, (int64_t)K * CRS);
  run_plan(dw, partial, beta);
  if (partial) scratch_give(partial_bytes, on_side);
  if (!ok) return;
  if (db && !bias_done) bias_grad_launch(nullptr, const_cast<float*>(dy), db, N, K, PQ);
  LH_CHECK_LAUNCH();
}

}  // extern "C"
