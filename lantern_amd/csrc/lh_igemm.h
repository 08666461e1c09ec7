// Implicit-GEMM core on fp32 MFMA (v_mfma_f32_32x32x2f32) for gfx950.
//
//   C[M,N] (+)= A[M,K] * B[K,N]
//
// A and B are never materialised: "loaders" fetch operand elements straight from the tensors
// (filter, activations, output gradient) with the convolution's index arithmetic, four
// consecutive k at a time, and park them in LDS in a k4-packed layout
//     tile[kq][col][4]          kq = k/4, col = row of A or column of B
// so that one ds_read_b128 hands a lane the operand values of four MFMA steps, and 32
// consecutive lanes read 32 consecutive 16-byte slots (no bank conflicts).
//
// Work decomposition: 256 threads = 4 wavefronts in a 2x2 grid; a wavefront owns a
// (BM/2)x(BN/2) sub-tile as MI x NI blocks of 32x32, accumulators in registers.  Global
// loads for tile t+1 are issued before the MFMAs of tile t and written to the other LDS
// stage afterwards (one barrier per k-slab).  Block ids are remapped so that each of the
// 8 XCDs (own L2 each) works on a contiguous range of tiles, M-tiles of one N-column first.
#pragma once
#include "lh_common.h"
#include <type_traits>

namespace lh {

typedef float f32x16 __attribute__((ext_vector_type(16)));

// ---- division by a run-time constant ------------------------------------------------------
struct FastDiv {
  uint32_t mul, shift, d;
  void init(uint32_t dd) {
    d = dd;
    uint32_t s = 0;
    while ((1ull << s) < dd) s++;
    shift = s;
    mul = (uint32_t)((((1ull << 32) * ((1ull << s) - dd)) / dd) + 1);
  }
  // exact for 0 <= n < 2^31
  __device__ __forceinline__ uint32_t div(uint32_t n) const { return (__umulhi(n, mul) + n) >> shift; }
  __device__ __forceinline__ void divmod(uint32_t n, uint32_t& q, uint32_t& r) const { q = div(n); r = n - q * d; }
};

struct GemmShape {
  int M, N, K;                // N: end of the column range of this launch
  int colBase;                // first column of this launch (tiles are counted from here)
  int tilesM, tilesN, splitK, kPerSplit;
  int total, perXcd;          // work items (tiles x k-splits, or stream-K workers) and items per XCD
  int streamk;                // != 0: `total` workers share tiles*slabsPerTile k-slabs evenly
  int slabsPerTile;
  long long units;            // tiles * slabsPerTile
  // streamk == 2 (whole tiles and slices of the last ones: see igemm_launch_shared_tail): the first fixFull blocks compute
  // one whole tile each; the tiles that are left are cut into fixCmax slices along the reduction (kPerSplit long), one block
  // per slice.  A sliced tile is finished by the LAST of its slices to arrive: each stores its partial sums into fixWs
  // (slot = slice), counts itself in fixCnt[tile], and the one that finds all others counted adds the partial sums up in
  // slice order and runs the epilogue of a whole tile.  Nobody waits for anybody.
  int fixFull, fixCmax, fixPer;       // fixPer: slices per XCD
  float4* fixWs; int* fixCnt;
};

// ---- operand loaders ---------------------------------------------------------------------------
// A loader turns (column, k) into BYTE OFFSETS into its tensor; the kernel fetches them with
// raw buffer loads.  An element outside the matrix (k >= kend, column past the edge, a padding
// tap of the convolution) gets the offset LH_OOB, which lies beyond the buffer's num_records, so
// the hardware returns 0 without touching memory: no branches and no selects in the k-loop.
// Tensors fed through a loader must be at most 2 GiB (checked on the host).
constexpr uint32_t LH_OOB = 0x80000000u;
constexpr int LH_RSRC_FLAGS = 0x00020000;    // raw buffer, 32-bit data format


// Element (col, k) at base[col*ld + k]  (k contiguous).  VEC: rows are 16-byte aligned and
// ld % 4 == 0 and K % 4 == 0, so a group of four k is one aligned 16-byte load, all in or all out.
template <bool VEC>
struct LoadPlainK {
  static constexpr bool ALONG_K = true;
  static constexpr bool VEC4 = VEC;
  static constexpr bool SPLIT = false;
  static constexpr bool STEP = true;
  const float* base; uint32_t nbytes; int ld;
  __device__ __forceinline__ uint32_t step_bytes(int bk) const { return (uint32_t)bk * 4u; }
  __device__ __forceinline__ int run_slabs(int, int) const { return 0x3fffffff; }
  struct State { uint32_t row; bool valid; };
  __device__ __forceinline__ void init(State& s, int col, int ncols) const { s.valid = col < ncols; s.row = (uint32_t)(s.valid ? col : 0) * (uint32_t)ld * 4u; }
  // byte offset of element k + e of the group starting at k (VEC: e == 0 stands for all four)
  __device__ __forceinline__ uint32_t off1(const State& s, int k, int kend, int e) const {
    return (s.valid && k + e < kend) ? s.row + (uint32_t)(k + e) * 4u : LH_OOB;
  }
};
// Element (col, k) at base[k*ld + col]  (col contiguous).
struct LoadPlainT {
  static constexpr bool ALONG_K = false;
  static constexpr bool VEC4 = false;
  static constexpr bool SPLIT = false;
  static constexpr bool STEP = true;
  const float* base; uint32_t nbytes; int ld;
  __device__ __forceinline__ uint32_t step_bytes(int bk) const { return (uint32_t)bk * (uint32_t)ld * 4u; }
  __device__ __forceinline__ int run_slabs(int, int) const { return 0x3fffffff; }
  struct State { uint32_t col; bool valid; };
  __device__ __forceinline__ void init(State& s, int col, int ncols) const { s.valid = col < ncols; s.col = (uint32_t)(s.valid ? col : 0) * 4u; }
  __device__ __forceinline__ uint32_t off1(const State& s, int k, int kend, int e) const {
    return (s.valid && k + e < kend) ? s.col + (uint32_t)(k + e) * (uint32_t)ld * 4u : LH_OOB;
  }
};

// A loader with STEP == true can also be advanced without recomputing anything per lane: inside a run of run_slabs(k, BK)
// consecutive k-slabs (counting the one that starts at k) the per-lane offsets of a slab are those of the slab before it
// plus the wave-uniform step_bytes(BK), which the kernel keeps in the scalar-offset operand of the loads.  (The range
// check of a raw buffer load looks at the per-lane offset only, so LH_OOB lanes stay out of range under any scalar offset.)
template <class L, class = void> struct LhCanStep { static constexpr bool value = false; };
template <class L> struct LhCanStep<L, typename std::enable_if<L::STEP>::type> { static constexpr bool value = true; };

// A MASKED loader says of every group how many of its elements are real (`keep`); the loaded vector passes through the loader's
// fix(v, keep) before it goes to LDS.  VEC4 form (off_keep() gives offset and keep): the group is loaded from 4 - keep elements
// before its place, fix() moves it up and fills with zeros (lh_keep_first).  SPLIT form (voff, keep, soff4): fix() clears the
// elements from `keep` on.
template <class L, class = void> struct LhMasked { static constexpr bool value = false; };
template <class L> struct LhMasked<L, typename std::enable_if<L::MASKED>::type> { static constexpr bool value = true; };
__device__ __forceinline__ float4 lh_keep_first(const float4 v, uint32_t keep) {
  float4 r;
  r.x = keep >= 4 ? v.x : (keep == 3 ? v.y : (keep == 2 ? v.z : v.w));
  r.y = keep >= 4 ? v.y : (keep == 3 ? v.z : (keep == 2 ? v.w : 0.f));
  r.z = keep >= 4 ? v.z : (keep == 3 ? v.w : 0.f);
  r.w = keep >= 4 ? v.w : 0.f;
  return r;
}

template <class L>
__device__ __forceinline__ float4 lh_fix_group(const float4 v, uint32_t keep) {
  if constexpr (LhMasked<L>::value) return L::fix(v, keep);
  else return v;
}

// Offsets of one group of four k (one offset when the loader is VEC4).  A SPLIT loader gives one
// per-lane byte offset for the group (o[0], LH_OOB when the group is out of range for this lane)
// plus four wave-uniform byte offsets s[i] that go into the scalar-offset operand of the load.
template <class L> struct LhOff { uint32_t o[4]; };
struct LhScal { uint32_t s[4]; };      // the wave-uniform parts of a SPLIT loader's group, kept apart from the per-lane ones so that they stay in scalar registers
template <class L>
// `xs`: wave-uniform bytes on top of every offset of the group (the slabs stepped over since the offsets were computed)
__device__ __forceinline__ float4 lh_fetch4(__amdgpu_buffer_rsrc_t rsrc, const LhOff<L>& f, const LhScal& u, int xs = 0) {
  // (the scalar-offset operands are the same in all lanes by construction; said at the use, because inside the segment loop of
  // the stream-K forms the compiler does not see it and wraps every load in a loop over the distinct values of a wavefront)
  xs = __builtin_amdgcn_readfirstlane(xs);
  if (L::SPLIT) {
    float4 r;
    r.x = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)f.o[0], __builtin_amdgcn_readfirstlane((int)u.s[0]) + xs, 0));
    r.y = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)f.o[0], __builtin_amdgcn_readfirstlane((int)u.s[1]) + xs, 0));
    r.z = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)f.o[0], __builtin_amdgcn_readfirstlane((int)u.s[2]) + xs, 0));
    r.w = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)f.o[0], __builtin_amdgcn_readfirstlane((int)u.s[3]) + xs, 0));
    return r;
  }
  if (L::VEC4) {
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)f.o[0], xs, 0);
    return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
  }
  float4 r;
  r.x = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)f.o[0], xs, 0));
  r.y = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)f.o[1], xs, 0));
  r.z = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)f.o[2], xs, 0));
  r.w = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)f.o[3], xs, 0));
  return r;
}

// Does an epilogue offer lean stores (see the store section of igemm_block)?
template <class E, class = void> struct LhHasLean { static constexpr bool value = false; };
template <class E> struct LhHasLean<E, typename std::enable_if<E::LEAN>::type> { static constexpr bool value = true; };

// ---- epilogue for row-major C ------------------------------------------------------------------
// mode 0: C = alpha*acc + beta*C ; mode 1: atomicAdd(C, alpha*acc) (split-K)
struct EpiRowMajor {
  static constexpr bool STATS = false;
  static constexpr bool SLICED = true;
  float* C; int ldc; float alpha, beta; int atomic;
  long long sliceStride = 0;       // != 0: slice sp of a cut reduction writes its own block C + sp*sliceStride (no atomics; added up afterwards)
  __device__ __forceinline__ void slice(int sp) { C += (long long)sp * sliceStride; }
  struct Col { int j; bool valid; };
  __device__ __forceinline__ Col col(int j, int N) const { Col c; c.j = j; c.valid = j < N; return c; }
  // lean stores (see the store section of igemm_block): element (i, j) at j * 4 + i * ldc * 4 bytes from C, for matrices
  // below 2 GiB; not for the atomic combination of partial sums, which measured slower through buffer atomics
  static constexpr bool LEAN = true;
  __device__ __forceinline__ bool lean_ok(int M) const { return !atomic && (M & 7) == 0 && (long long)M * ldc < 0x20000000LL; }
  __device__ __forceinline__ float* lean_base() const { return C; }
  __device__ __forceinline__ uint32_t lane_bytes(const Col& c) const { return (uint32_t)c.j * 4u; }
  __device__ __forceinline__ uint32_t row_bytes() const { return (uint32_t)ldc * 4u; }
  __device__ __forceinline__ uint32_t cell_row_bytes() const { return 0u; }
  __device__ __forceinline__ int lean_mode() const { return beta == 0.f ? 0 : 1; }
  __device__ __forceinline__ float lean_scale() const { return alpha; }
  static constexpr bool LEAN_FIX = false;         // nothing is added to or clamped in a stored element
  __device__ __forceinline__ float lean_fix(float v, int) const { return v; }
  // part: 0 = the whole reduction of this element is in v; 1 = first partial sum, 2 = a later one
  // (partials are combined with atomic adds onto an output the host has prepared)
  __device__ __forceinline__ void store(const Col& c, int i, int M, float v, int part) const {
    if (!c.valid || i >= M) return;
    float* p = C + (int64_t)i * ldc + c.j;
    if (atomic || part) atomicAdd(p, alpha * v);
    else *p = alpha * v + (beta == 0.f ? 0.f : beta * *p);
  }
};

// bytes of LDS of one tile configuration: two stages of both operands, k-packed and padded
template <int BM, int BN, int BK>
constexpr size_t igemm_smem_bytes() { return (size_t)2 * (BK / 4) * ((BM + 8 / (BK / 4)) + (BN + 8 / (BK / 4))) * sizeof(float4); }

// ---- the kernel ------------------------------------------------------------------------------------
// The work of one block; `block` is its index within the launch (or within its group of a grouped launch).
template <int BM, int BN, int BK, class AL, class BL, class EP, int SK>      // SK: 0 one tile (or k-split of a tile) per block, 1 stream-K with atomic adds, 2 rounds + shared tail
__device__ __forceinline__ void igemm_block(const AL& al, const BL& bl, const EP& ep_in, const GemmShape& gs, const int block) {
  typename std::conditional<EP::SLICED, EP, const EP&>::type ep = ep_in;      // a sliced epilogue is a private copy that slice() moves
  constexpr int KQ = BK / 4, PAD = 8 / KQ, LDA = BM + PAD, LDB = BN + PAD;
  // The four wavefronts form a 2 x 2 grid over the tile, or, for a 32-row tile (products with at most 32 rows: layers with
  // few channels), a 1 x 4 grid, so that no matrix instruction is spent on rows beyond the 32.
  constexpr int WM = BM >= 64 ? 2 : 1, WN = 4 / WM;
  constexpr int TM = BM / WM, TN = BN / WN, MI = TM / 32, NI = TN / 32;
  static_assert(WM == 2 || !EP::STATS, "the statistics epilogue assumes two wavefronts along the columns");
  constexpr int GA = BM * KQ / 256, GB = BN * KQ / 256;
  static_assert(GA >= 1 && GB >= 1 && MI >= 1 && NI >= 1, "tile too small for 256 threads");
  extern __shared__ float4 lh_smem[];
  float4* As = lh_smem;
  float4* Bs = lh_smem + 2 * KQ * LDA;

  int logical = (block % 8) * gs.perXcd + block / 8;
  if (SK == 2) {
    // every XCD gets an eighth of the whole tiles (consecutive ones: they share columns in its L2) and, behind them, an
    // eighth of the slices, so that each compute unit is given its whole tiles first and its slices last
    const int x = block % 8, li = block / 8, whole_per = gs.fixFull / 8;
    if (li < whole_per) logical = x * whole_per + li;
    else {
      const int sl = x * gs.fixPer + (li - whole_per);
      if (li - whole_per >= gs.fixPer || sl >= gs.total - gs.fixFull) return;
      logical = gs.fixFull + sl;
    }
  }
  if (logical >= gs.total) return;
  // Work of this block: either one (tile, k-split) item, or -- stream-K -- an equal share of all
  // k-slabs of all tiles, walked tile by tile; a tile whose slabs are shared between two blocks
  // is completed with atomic adds.
  long long u = 0, u_end = 1;
  if (SK == 1) { u = gs.units * logical / gs.total; u_end = gs.units * (logical + 1) / gs.total; }
  // STEPPED: both loaders can be advanced by a wave-uniform step, so inside a run of slabs the offsets of the next slab
  // cost two scalar additions instead of a decode per element; a slab past the end of the reduction is switched off by a
  // buffer descriptor of zero bytes (every lane out of range, the loads return 0 without touching memory).
  // (Not on the 32-row tiles with a tap-major gather: they serve layers of at most 32 channels, where a filter tap is as deep
  // as one 32-deep slab, every slab is decoded anyway and the interleaved decode below is the faster one.)
  constexpr bool STEPPED = LhCanStep<AL>::value && LhCanStep<BL>::value && (BM >= 64 || !(AL::SPLIT || BL::SPLIT));
  const __amdgpu_buffer_rsrc_t rsA = __builtin_amdgcn_make_buffer_rsrc((void*)al.base, 0, (int)al.nbytes, LH_RSRC_FLAGS);
  const __amdgpu_buffer_rsrc_t rsB = __builtin_amdgcn_make_buffer_rsrc((void*)bl.base, 0, (int)bl.nbytes, LH_RSRC_FLAGS);
  const int t = threadIdx.x;
  int a_col[GA], a_kq[GA], b_col[GB], b_kq[GB];
#pragma unroll
  for (int g = 0; g < GA; g++) {
    if (AL::ALONG_K) { a_kq[g] = t % KQ; a_col[g] = t / KQ + g * (256 / KQ); }
    else { a_col[g] = t % BM; a_kq[g] = (BM >= 64 ? __builtin_amdgcn_readfirstlane(t / BM) : t / BM) + g * (256 / BM); }   // uniform per wavefront from 64 rows on
  }
#pragma unroll
  for (int g = 0; g < GB; g++) {
    if (BL::ALONG_K) { b_kq[g] = t % KQ; b_col[g] = t / KQ + g * (256 / KQ); }
    else { b_col[g] = t % BN; b_kq[g] = __builtin_amdgcn_readfirstlane(t / BN) + g * (256 / BN); }
  }
  const int lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6), wm = WM == 2 ? wave >> 1 : 0, wn = WM == 2 ? wave & 1 : wave, half = lane >> 5, l32 = lane & 31;

  while (u < u_end) {
  int tm, tn, kbeg, kend, part = 0;
  int fix_tile = 0, fix_n = 1, fix_slot = 0;       // SK == 2, part != 0: the sliced tile, its number of slices, this block's slice
  if (SK == 2) {
    int tile;
    if (logical < gs.fixFull) { tile = logical; kbeg = 0; kend = gs.K; }
    else {
      const int i = logical - gs.fixFull;
      fix_tile = i / gs.fixCmax; fix_slot = i - fix_tile * gs.fixCmax; fix_n = gs.fixCmax;
      tile = gs.fixFull + fix_tile;
      kbeg = fix_slot * gs.kPerSplit; kend = min(gs.K, kbeg + gs.kPerSplit);
      part = 1;
    }
    tm = tile % gs.tilesM; tn = tile / gs.tilesM;
    u = u_end;
  } else if (SK) {
    const int tile = (int)(u / gs.slabsPerTile), s0 = (int)(u - (long long)tile * gs.slabsPerTile);
    const long long left = u_end - u;
    const int s1 = (int)(left < (long long)(gs.slabsPerTile - s0) ? s0 + left : gs.slabsPerTile);
    tm = tile % gs.tilesM; tn = tile / gs.tilesM;
    kbeg = s0 * BK; kend = min(gs.K, s1 * BK);
    part = (s0 == 0 && s1 == gs.slabsPerTile) ? 0 : (s0 == 0 ? 1 : 2);
    u += s1 - s0;
    __syncthreads();            // LDS of the previous segment is free again
  } else {
    tm = logical % gs.tilesM;
    const int rest = logical / gs.tilesM;
    tn = rest % gs.tilesN;
    const int sp = rest / gs.tilesN;
    kbeg = sp * gs.kPerSplit; kend = min(gs.K, kbeg + gs.kPerSplit);
    if constexpr (EP::SLICED) ep.slice(sp);
    u = u_end;
  }
  if (SK == 1) {       // the segment is the same for all lanes of the block
    tm = __builtin_amdgcn_readfirstlane(tm); tn = __builtin_amdgcn_readfirstlane(tn);
    kbeg = __builtin_amdgcn_readfirstlane(kbeg); kend = __builtin_amdgcn_readfirstlane(kend); part = __builtin_amdgcn_readfirstlane(part);
  }
  const int m0 = tm * BM, n0 = gs.colBase + tn * BN;
  typename AL::State sa[GA];
  typename BL::State sb[GB];
#pragma unroll
  for (int g = 0; g < GA; g++) al.init(sa[g], m0 + a_col[g], gs.M);
#pragma unroll
  for (int g = 0; g < GB; g++) bl.init(sb[g], n0 + b_col[g], gs.N);

  f32x16 acc[MI][NI];
#pragma unroll
  for (int mi = 0; mi < MI; mi++)
#pragma unroll
    for (int ni = 0; ni < NI; ni++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[mi][ni][v] = 0.f;

  const int niter = (kend - kbeg + BK - 1) / BK;
  constexpr int EA = AL::VEC4 ? 1 : 4, EB = BL::VEC4 ? 1 : 4;
  constexpr int NEL = GA * EA + GB * EB;            // offsets to compute per slab and thread
  constexpr int NM_PAIR = 4 * MI * NI, NM = (KQ / 2) * NM_PAIR;
  float4 ra0[GA], rb0[GB], ra1[GA], rb1[GB];
  uint32_t ka0[GA], kb0[GB], ka1[GA], kb1[GB];
  LhOff<AL> oa[GA];
  LhOff<BL> ob[GB];
  LhScal ua[GA], ub[GB];
  // e-th offset of the slab starting at k0
  auto elem = [&](int e, int k0) {
    if (e < GA * EA) {
      const int g = e / EA, i = e % EA, k = k0 + 4 * a_kq[g];
      if constexpr (AL::SPLIT && LhMasked<AL>::value) { if (i == 0) { const int ku = __builtin_amdgcn_readfirstlane(k); oa[g].o[0] = al.voff(sa[g], ku, kend); oa[g].o[1] = al.keep(ku, kend); al.soff4(ku, kend, ua[g].s); } }
      else if constexpr (AL::SPLIT) { const int ku = __builtin_amdgcn_readfirstlane(k); if (i == 0) oa[g].o[0] = al.voff(sa[g], ku, kend); ua[g].s[i] = al.soff(ku, i); }      // (a SPLIT loader's k is the same in all lanes: its groups run along the columns)
      else if constexpr (LhMasked<AL>::value) oa[g].o[0] = al.off_keep(sa[g], k, kend, oa[g].o[1]);
      else oa[g].o[i] = al.off1(sa[g], k, kend, i);
    } else {
      const int f = e - GA * EA, g = f / EB, i = f % EB, k = k0 + 4 * b_kq[g];
      if constexpr (BL::SPLIT && LhMasked<BL>::value) { if (i == 0) { const int ku = __builtin_amdgcn_readfirstlane(k); ob[g].o[0] = bl.voff(sb[g], ku, kend); ob[g].o[1] = bl.keep(ku, kend); bl.soff4(ku, kend, ub[g].s); } }
      else if constexpr (BL::SPLIT) { const int ku = __builtin_amdgcn_readfirstlane(k); if (i == 0) ob[g].o[0] = bl.voff(sb[g], ku, kend); ub[g].s[i] = bl.soff(ku, i); }
      else if constexpr (LhMasked<BL>::value) ob[g].o[0] = bl.off_keep(sb[g], k, kend, ob[g].o[1]);
      else ob[g].o[i] = bl.off1(sb[g], k, kend, i);
    }
  };
  // State of the slab the next fetch loads (STEPPED): bytes stepped since (oa, ob) were computed; how many more slabs can
  // be reached by stepping (whole slabs inside the reduction and inside the loaders' runs); the byte range of the buffer
  // descriptors (0 switches the loads of a slab past the end of the reduction off).
  int xsA = 0, xsB = 0, steps = 0, nrecA = (int)al.nbytes, nrecB = (int)bl.nbytes;
  // (ka, kb: the keep counts of a MASKED loader's groups travel with the loaded registers until stash() applies them)
  auto fetch = [&](float4 (&ra)[GA], float4 (&rb)[GB], uint32_t (&ka)[GA], uint32_t (&kb)[GB]) {
    if constexpr (LhMasked<AL>::value) {
#pragma unroll
      for (int g = 0; g < GA; g++) ka[g] = oa[g].o[1];
    }
    if constexpr (LhMasked<BL>::value) {
#pragma unroll
      for (int g = 0; g < GB; g++) kb[g] = ob[g].o[1];
    }
    if constexpr (STEPPED) {
      // (the byte ranges are the same in all lanes; said here because inside the segment loop of the stream-K forms the
      // compiler no longer sees it and wraps every load in a loop over the distinct descriptors of a wavefront)
      const __amdgpu_buffer_rsrc_t ra_ = __builtin_amdgcn_make_buffer_rsrc((void*)al.base, 0, __builtin_amdgcn_readfirstlane(nrecA), LH_RSRC_FLAGS);
      const __amdgpu_buffer_rsrc_t rb_ = __builtin_amdgcn_make_buffer_rsrc((void*)bl.base, 0, __builtin_amdgcn_readfirstlane(nrecB), LH_RSRC_FLAGS);
#pragma unroll
      for (int g = 0; g < GA; g++) ra[g] = lh_fetch4<AL>(ra_, oa[g], ua[g], xsA);
#pragma unroll
      for (int g = 0; g < GB; g++) rb[g] = lh_fetch4<BL>(rb_, ob[g], ub[g], xsB);
    } else {
#pragma unroll
      for (int g = 0; g < GA; g++) ra[g] = lh_fetch4<AL>(rsA, oa[g], ua[g]);
#pragma unroll
      for (int g = 0; g < GB; g++) rb[g] = lh_fetch4<BL>(rsB, ob[g], ub[g]);
    }
  };
  // all offsets of the slab at kn from scratch
  auto decode = [&](int kn) {
    if constexpr (STEPPED) {
      if (__builtin_amdgcn_readfirstlane((int)(kn >= kend))) { nrecA = 0; nrecB = 0; steps = 0; return; }
#pragma unroll
      for (int e = 0; e < NEL; e++) elem(e, kn);
      xsA = 0; xsB = 0;
      const int whole = (kend - kn) / BK;                       // whole slabs from kn on
      steps = __builtin_amdgcn_readfirstlane(min(min(al.run_slabs(kn, BK), bl.run_slabs(kn, BK)), whole) - 1);
    }
  };
  // (oa, ob, ...) describe the slab at kn - BK and are made to describe the slab at kn
  auto advance = [&](int kn) {
    if constexpr (STEPPED) {
      // (the counters are the same in all lanes; saying so at every update keeps them, and the buffer descriptors and scalar
      // offsets made from them, in scalar registers in every instantiation)
      if (__builtin_expect(__builtin_amdgcn_readfirstlane(steps) > 0, 1)) {
        steps = __builtin_amdgcn_readfirstlane(steps - 1);
        xsA = __builtin_amdgcn_readfirstlane(xsA + (int)al.step_bytes(BK)); xsB = __builtin_amdgcn_readfirstlane(xsB + (int)bl.step_bytes(BK));
      }
      else decode(kn);
    }
  };
  auto stash = [&](const float4 (&ra)[GA], const float4 (&rb)[GB], const uint32_t (&ka)[GA], const uint32_t (&kb)[GB], int stage) {
    const int o = stage * KQ;
#pragma unroll
    for (int g = 0; g < GA; g++) As[(o + a_kq[g]) * LDA + a_col[g]] = lh_fix_group<AL>(ra[g], ka[g]);
#pragma unroll
    for (int g = 0; g < GB; g++) Bs[(o + b_kq[g]) * LDB + b_col[g]] = lh_fix_group<BL>(rb[g], kb[g]);
  };

  // Software pipeline over k-slabs (four slabs in flight):
  //   while the MFMAs of slab t run from LDS, slab t+1 is in registers on its way to LDS (its
  //   loads were issued one iteration earlier), the loads of slab t+2 are issued at the top of the
  //   iteration into the other register set, and the offsets of slab t+3 (VALU/SALU only) are
  //   computed in small pieces placed between the MFMAs, so they issue while the matrix pipe is
  //   busy.  A global load therefore has a whole iteration plus the MFMA time of the next one to
  //   arrive.  Slabs past kend produce LH_OOB offsets (loads return 0) and LDS stages never read.
  if constexpr (STEPPED) {
    nrecA = (int)al.nbytes; nrecB = (int)bl.nbytes;
    decode(kbeg);
    fetch(ra0, rb0, ka0, kb0);
    advance(kbeg + BK);
    fetch(ra1, rb1, ka1, kb1);
    advance(kbeg + 2 * BK);
  } else {
#pragma unroll
    for (int e = 0; e < NEL; e++) elem(e, kbeg);
    fetch(ra0, rb0, ka0, kb0);
#pragma unroll
    for (int e = 0; e < NEL; e++) elem(e, kbeg + BK);
    fetch(ra1, rb1, ka1, kb1);
#pragma unroll
    for (int e = 0; e < NEL; e++) elem(e, kbeg + 2 * BK);
  }
  stash(ra0, rb0, ka0, kb0, 0);
  __syncthreads();

  // one iteration: compute slab `it` from LDS stage st, fetch slab it+2 into (rla, rlb), move slab
  // it+1 from (rsa, rsb) to LDS stage st^1
  auto body = [&](int it, int st, float4 (&rla)[GA], float4 (&rlb)[GB], uint32_t (&kla)[GA], uint32_t (&klb)[GB],
                  const float4 (&rsa)[GA], const float4 (&rsb)[GB], const uint32_t (&ksa)[GA], const uint32_t (&ksb)[GB]) {
    const int k3 = kbeg + (it + 3) * BK;
    fetch(rla, rlb, kla, klb);
    __builtin_amdgcn_sched_barrier(0);
    const float4* Asc = As + st * KQ * LDA + wm * TM + l32;
    const float4* Bsc = Bs + st * KQ * LDB + wn * TN + l32;
    // operands of the next pair of k-quads are read from LDS before the matrix instructions of the current pair are
    // issued, so a wavefront does not stand still for the LDS latency between pairs
    float4 a[2][MI], b[2][NI];
#pragma unroll
    for (int mi = 0; mi < MI; mi++) a[0][mi] = Asc[half * LDA + mi * 32];
#pragma unroll
    for (int ni = 0; ni < NI; ni++) b[0][ni] = Bsc[half * LDB + ni * 32];
#pragma unroll
    for (int pair = 0; pair < KQ / 2; pair++) {
      const int cur = pair & 1, nxt = cur ^ 1;
      if (pair + 1 < KQ / 2) {
        const int kq = 2 * (pair + 1) + half;
#pragma unroll
        for (int mi = 0; mi < MI; mi++) a[nxt][mi] = Asc[kq * LDA + mi * 32];
#pragma unroll
        for (int ni = 0; ni < NI; ni++) b[nxt][ni] = Bsc[kq * LDB + ni * 32];
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < NM_PAIR; m++) {
        const int c = m / (MI * NI), mi = (m / NI) % MI, ni = m % NI;
        const float av = c == 0 ? a[cur][mi].x : c == 1 ? a[cur][mi].y : c == 2 ? a[cur][mi].z : a[cur][mi].w;
        const float bv = c == 0 ? b[cur][ni].x : c == 1 ? b[cur][ni].y : c == 2 ? b[cur][ni].z : b[cur][ni].w;
        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[mi][ni], 0, 0, 0);
        const int gm = pair * NM_PAIR + m;
        if constexpr (STEPPED) {
          if (gm == 1) {
            __builtin_amdgcn_sched_barrier(0);
            advance(k3);
            __builtin_amdgcn_sched_barrier(0);
          }
          continue;
        }
        const int e0 = (gm * NEL) / NM, e1 = ((gm + 1) * NEL) / NM;
        if (e1 > e0) {
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int e = e0; e < e1; e++) elem(e, k3);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    stash(rsa, rsb, ksa, ksb, st ^ 1);
    __syncthreads();
  };
  // the loop runs an even number of iterations: a trailing slab past kend is all zeros
  for (int it = 0; it < niter; it += 2) {
    body(it, 0, ra0, rb0, ka0, kb0, ra1, rb1, ka1, kb1);
    body(it + 1, 1, ra1, rb1, ka1, kb1, ra0, rb0, ka0, kb0);
  }

  if constexpr (SK == 2) {
    if (part) {
      // The partial sums of this segment go to the workspace; the contributor that finds all the others counted adds them
      // up, in slot order (its own included, so the result does not depend on who came last), and goes on as the owner of a
      // whole tile.  Blocks on different XCDs do not share an L2, and a fence that writes a whole L2 back and invalidates it
      // (what __threadfence() costs here: the launch took six times as long) is not needed for 16 KB: the partial sums are
      // stored and loaded with the device-coherent cache policy (sc0 sc1: written through, read past the local L2), every
      // wavefront waits for its stores to be acknowledged before the block counts itself, and the reads come after the count.
      typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
      constexpr int Q = MI * NI * 4;          // 16-byte pieces per thread
      constexpr int COHERENT = 17;            // cache policy bits of the buffer instructions: sc0 | sc1
      const uint32_t slot_bytes = 256u * Q * 16u;
      char* ws = reinterpret_cast<char*>(gs.fixWs) + (size_t)((size_t)fix_tile * gs.fixCmax) * slot_bytes;
      {
        const __amdgpu_buffer_rsrc_t rw_ = __builtin_amdgcn_make_buffer_rsrc((void*)(ws + (size_t)fix_slot * slot_bytes), 0, (int)slot_bytes, LH_RSRC_FLAGS);
#pragma unroll
        for (int mi = 0; mi < MI; mi++)
#pragma unroll
          for (int ni = 0; ni < NI; ni++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
              u32x4 v4;
              v4.x = __float_as_uint(acc[mi][ni][4 * q]); v4.y = __float_as_uint(acc[mi][ni][4 * q + 1]);
              v4.z = __float_as_uint(acc[mi][ni][4 * q + 2]); v4.w = __float_as_uint(acc[mi][ni][4 * q + 3]);
              __builtin_amdgcn_raw_buffer_store_b128(v4, rw_, (int)((t * Q + (mi * NI + ni) * 4 + q) * 16), 0, COHERENT);
            }
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      __shared__ int lh_fix_old;
      if (t == 0) lh_fix_old = atomicAdd(gs.fixCnt + fix_tile, 1);
      __syncthreads();
      const int old = lh_fix_old;
      if (old != fix_n - 1) continue;          // somebody else finishes this tile
      if (t == 0) gs.fixCnt[fix_tile] = 0;     // left as found, for the next launch
#pragma unroll
      for (int mi = 0; mi < MI; mi++)
#pragma unroll
        for (int ni = 0; ni < NI; ni++)
#pragma unroll
          for (int v = 0; v < 16; v++) acc[mi][ni][v] = 0.f;
      // the slices are added in slice order; the loads of up to four of them are in flight at once (each is a round trip to
      // memory past the local L2, and nothing else is left to hide it behind)
      constexpr int AHEAD = Q <= 4 ? 4 : (Q <= 8 ? 2 : 1);
      for (int s0 = 0; s0 < fix_n; s0 += AHEAD) {
        u32x4 w4[AHEAD][Q];
#pragma unroll
        for (int a = 0; a < AHEAD; a++) {
          const int sl = s0 + a < fix_n ? s0 + a : fix_n - 1;          // (a repeat of the last slice is loaded and not added)
          const __amdgpu_buffer_rsrc_t rr_ = __builtin_amdgcn_make_buffer_rsrc((void*)(ws + (size_t)sl * slot_bytes), 0, (int)slot_bytes, LH_RSRC_FLAGS);
#pragma unroll
          for (int j = 0; j < Q; j++) w4[a][j] = __builtin_amdgcn_raw_buffer_load_b128(rr_, (int)((t * Q + j) * 16), 0, COHERENT);
        }
#pragma unroll
        for (int a = 0; a < AHEAD; a++) {
          if (s0 + a >= fix_n) break;
#pragma unroll
          for (int mi = 0; mi < MI; mi++)
#pragma unroll
            for (int ni = 0; ni < NI; ni++)
#pragma unroll
              for (int q = 0; q < 4; q++) {
                const u32x4 v4 = w4[a][(mi * NI + ni) * 4 + q];
                acc[mi][ni][4 * q] += __uint_as_float(v4.x); acc[mi][ni][4 * q + 1] += __uint_as_float(v4.y);
                acc[mi][ni][4 * q + 2] += __uint_as_float(v4.z); acc[mi][ni][4 * q + 3] += __uint_as_float(v4.w);
              }
        }
      }
      part = 0;
    }
  }

  // D layout of a 32x32 block: column = lane % 32, row = 8*(v/4) + 4*(lane/32) + v%4
  // With EP::STATS the same pass also forms per-row sums of the finished tile (the batch-norm statistics of a
  // convolution's output rows = channels): every wavefront reduces its TM x TN piece over the columns and
  // stores (sum, sum of squares) of each row into slot (2*tn + wn) of ep.partial; one writer per slot, no atomics.
  typename EP::Col cs[NI];
#pragma unroll
  for (int ni = 0; ni < NI; ni++) cs[ni] = ep.col(n0 + wn * TN + ni * 32 + l32, gs.N);
  bool want_stats = false;
  if constexpr (EP::STATS && SK != 1) want_stats = ep.partial != nullptr;
  // Lean stores (epilogues that offer them, complete sums only; partial sums added with buffer atomics measured slower
  // and stay on the general path): the element of row i and column j lies at
  // lane_bytes(j) + i * row_bytes(), so a store is one buffer instruction whose per-lane offset is fixed for the tile
  // (LH_OOB for a column past the edge: the store is dropped) and whose row goes into the scalar offset; the two halves of
  // a wavefront hold rows four apart, which the per-lane offset carries, and with M a multiple of 8 both are inside
  // the matrix or both outside.  No address arithmetic per element is left in the vector unit.
  bool lean = false;
  if constexpr (LhHasLean<EP>::value) lean = part == 0 && ep.lean_ok(gs.M);
  if constexpr (LhHasLean<EP>::value) {
    if (lean) {
      const __amdgpu_buffer_rsrc_t rsO = __builtin_amdgcn_make_buffer_rsrc((void*)ep.lean_base(), 0, (int)0x80000000u, LH_RSRC_FLAGS);
      const uint32_t rb = ep.row_bytes();
      uint32_t vo[NI];
#pragma unroll
      for (int ni = 0; ni < NI; ni++) vo[ni] = cs[ni].valid ? ep.lane_bytes(cs[ni]) + (uint32_t)(4 * half) * rb : LH_OOB;
      const int mode = ep.lean_mode();             // 0: overwrite, 1: beta * old + value, 2: value and the three zeros of its 2 x 2 cell
      const float scale = ep.lean_scale();         // alpha of a gemm, 1 for a convolution
      auto pass = [&](auto MODE) {
        constexpr int MD = decltype(MODE)::value;
#pragma unroll
        for (int mi = 0; mi < MI; mi++) {
          const int r0 = m0 + wm * TM + mi * 32;
          // mode 1: all old values of the block are requested before the first of them is used (the compiler cannot move
          // a load across the store in front of it, so element by element every load would wait for a round trip of its own)
          float old[MD == 1 ? 16 : 1][NI];
          if constexpr (MD == 1) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
              const int so = (int)((uint32_t)(r0 + 8 * (v / 4) + (v % 4)) * rb);
              const bool in = r0 + 8 * (v / 4) < gs.M;
#pragma unroll
              for (int ni = 0; ni < NI; ni++)
                old[v][ni] = in ? __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rsO, (int)vo[ni], so, 0)) : 0.f;
            }
          }
#pragma unroll
          for (int v = 0; v < 16; v++) {
            const int row = r0 + 8 * (v / 4) + (v % 4);        // of the lower half; the upper half is four rows further on
            if (r0 + 8 * (v / 4) >= gs.M) continue;
            const int so = (int)((uint32_t)row * rb);
#pragma unroll
            for (int ni = 0; ni < NI; ni++) {
              float val = acc[mi][ni][v] * scale;
              if constexpr (EP::LEAN_FIX) val = ep.lean_fix(val, row + 4 * half);
              if constexpr (MD == 1) val = fmaf(ep.beta, old[v][ni], val);
              if constexpr (MD == 2) {
                typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
                u32x2 a2; a2.x = __float_as_uint(val); a2.y = 0u;
                u32x2 z2; z2.x = 0u; z2.y = 0u;
                __builtin_amdgcn_raw_buffer_store_b64(a2, rsO, (int)vo[ni], so, 0);
                __builtin_amdgcn_raw_buffer_store_b64(z2, rsO, (int)vo[ni], so + (int)ep.cell_row_bytes(), 0);
              } else {
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(val), rsO, (int)vo[ni], so, 0);
              }
            }
          }
        }
      };
      if (mode == 0) pass(std::integral_constant<int, 0>());
      else if (mode == 1) pass(std::integral_constant<int, 1>());
      else pass(std::integral_constant<int, 2>());
    }
  }
  if (!lean) {
#pragma unroll
    for (int mi = 0; mi < MI; mi++) {
      const int ib = m0 + wm * TM + mi * 32 + 4 * half;
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int row = ib + 8 * (v / 4) + (v % 4);
#pragma unroll
        for (int ni = 0; ni < NI; ni++) ep.store(cs[ni], row, gs.M, acc[mi][ni][v], part);
      }
    }
  }
  if constexpr (EP::STATS && SK != 1) {
    if (want_stats) {
      // Row sums of the wavefront's TM x TN piece.  A lane holds 16 rows of one column, and a sum over columns done
      // in registers costs five cross-lane steps per row; instead every 32 x 32 block goes through LDS once, transposed
      // (the operand stages are free by now: the last barrier of the slab loop lies behind every read of them), so that
      // lane l32 of each half reads row l32 of the block, 16 columns per half, and adds them up as it reads.
      // Only this wavefront touches its region, whose LDS operations execute in program order.
      // (sums of the accumulators: the host uses this path only for launches without a bias)
      // Column c of the transposed block is kept rotated by 4c rows, which spreads both the 16-byte writes (lanes =
      // columns) and the reads (lanes = rows) over all banks without padding.
      constexpr int TLD = 32;
      static_assert(4 * 32 * TLD * sizeof(float) <= igemm_smem_bytes<BM, BN, BK>(), "the transposed blocks of the four wavefronts fit the operand stages");
      float* T = reinterpret_cast<float*>(lh_smem) + wave * (32 * TLD);
#pragma unroll
      for (int mi = 0; mi < MI; mi++) {
        float r1 = 0.f, r2 = 0.f;
#pragma unroll
        for (int ni = 0; ni < NI; ni++) {
          const bool cv = cs[ni].valid;
#pragma unroll
          for (int g = 0; g < 4; g++) {
            float4 q;
            q.x = cv ? acc[mi][ni][4 * g + 0] : 0.f; q.y = cv ? acc[mi][ni][4 * g + 1] : 0.f;
            q.z = cv ? acc[mi][ni][4 * g + 2] : 0.f; q.w = cv ? acc[mi][ni][4 * g + 3] : 0.f;
            *reinterpret_cast<float4*>(T + l32 * TLD + ((8 * g + 4 * half + 4 * l32) & 31)) = q;       // rows 8g + 4*half .. +3 of column l32
          }
          __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int c = 0; c < 16; c++) { const int cc = half * 16 + c; const float x = T[cc * TLD + ((l32 + 4 * cc) & 31)]; r1 += x; r2 = fmaf(x, x, r2); }
          __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
          __builtin_amdgcn_wave_barrier();
        }
        r1 += __shfl_xor(r1, 32); r2 += __shfl_xor(r2, 32);
        const int row = m0 + wm * TM + mi * 32 + l32;
        if (half == 0 && row < gs.M) { float2* p = reinterpret_cast<float2*>(ep.partial) + (size_t)row * ep.slotsTotal + (ep.slotBase + tn * 2 + wn); *p = make_float2(r1, r2); }
      }
    }
  }
  }  // segments
}

template <int BM, int BN, int BK, class AL, class BL, class EP, int SK>
__global__ void __launch_bounds__(256) k_igemm(const AL al, const BL bl, const EP ep, const GemmShape gs) {
  igemm_block<BM, BN, BK, AL, BL, EP, SK>(al, bl, ep, gs, (int)blockIdx.x);
}

// Up to four products in one launch (the residue classes of a strided input gradient: same loaders and tile, their own
// operands, reduction lengths and output maps).  Blocks [first[g], first[g+1]) belong to group g; the longest first.
constexpr int IGEMM_MAX_GROUPS = 4;
template <class AL, class BL, class EP>
struct IgemmGroups { AL al[IGEMM_MAX_GROUPS]; BL bl[IGEMM_MAX_GROUPS]; EP ep[IGEMM_MAX_GROUPS]; GemmShape gs[IGEMM_MAX_GROUPS]; int first[IGEMM_MAX_GROUPS + 1]; };
template <int BM, int BN, int BK, class AL, class BL, class EP>
__global__ void __launch_bounds__(256) k_igemm_grouped(const IgemmGroups<AL, BL, EP> g) {
  const int b = (int)blockIdx.x;
  int gi = 0;
#pragma unroll
  for (int i = 1; i < IGEMM_MAX_GROUPS; i++) if (b >= g.first[i]) gi = i;
  igemm_block<BM, BN, BK, AL, BL, EP, 0>(g.al[gi], g.bl[gi], g.ep[gi], g.gs[gi], b - g.first[gi]);
}


// Launch one tile configuration.
//   splitK > 1 : the reduction is cut into splitK pieces per tile (needs an accumulating epilogue).
//   streamk    : `streamk` workers (about two per CU) share all k-slabs of all tiles evenly, which
//                removes the idle tail of a grid with few tiles; tiles shared by two workers are
//                finished with atomic adds, so the caller must have the output hold beta*C.
// Blocks of one tile configuration that fit on a CU at once (registers and LDS), asked of the runtime once.
template <int BM, int BN, int BK, class AL, class BL, class EP>
int igemm_blocks_per_cu() {
  static int occ = 0;
  if (occ == 0) {
    int v = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&v, k_igemm<BM, BN, BK, AL, BL, EP, 0>, 256, igemm_smem_bytes<BM, BN, BK>()) != hipSuccess || v < 1) v = 2;
    occ = v;
  }
  return occ;
}

//   [col0, col1) : the columns this launch covers (col1 < 0: up to N); tiles are laid out from col0.
template <int BM, int BN, int BK, class AL, class BL, class EP>
bool igemm_launch(const AL& al, const BL& bl, const EP& ep, int M, int N, int K, int splitK, int streamk = 0, int col0 = 0, int col1 = -1) {
  GemmShape gs;
  if (col1 < 0 || col1 > N) col1 = N;
  if (col0 >= col1) return true;
  gs.M = M; gs.N = col1; gs.K = K; gs.colBase = col0;
  gs.tilesM = (int)cdiv(M, BM); gs.tilesN = (int)cdiv(col1 - col0, BN);
  if (splitK < 1) splitK = 1;
  int kper = (int)cdiv(cdiv(K, splitK), BK) * BK;
  if (kper < BK) kper = BK;
  gs.kPerSplit = kper;
  gs.splitK = (int)cdiv(K > 0 ? K : 1, kper);
  gs.slabsPerTile = (int)cdiv(K > 0 ? K : 1, BK);
  gs.units = (long long)gs.tilesM * gs.tilesN * gs.slabsPerTile;
  gs.streamk = 0;
  int64_t total = (int64_t)gs.tilesM * gs.tilesN * gs.splitK;
  if (streamk > 0) {
    gs.streamk = 1;
    total = streamk < gs.units ? streamk : gs.units;
  }
  if (total <= 0 || total > 0x3fffffff) { LH_FAIL("igemm: tile count %lld out of range", (long long)total); return false; }
  gs.total = (int)total; gs.perXcd = (int)cdiv(total, 8);
  constexpr size_t smem = igemm_smem_bytes<BM, BN, BK>();
  if (gs.streamk) {
    if constexpr (smem <= 48 * 1024) {   // stream-K is instantiated for the forward / input-gradient tiles only
      ProfScope prof_(g_kernel_cat);
      hipLaunchKernelGGL((k_igemm<BM, BN, BK, AL, BL, EP, 1>), dim3(8 * gs.perXcd), dim3(256), smem, g_stream, al, bl, ep, gs);
      return true;
    } else { LH_FAIL("igemm: stream-K is not built for this tile"); return false; }
  }
  auto kern = k_igemm<BM, BN, BK, AL, BL, EP, 0>;
  static bool attr_done = false;
  if (smem > 48 * 1024 && !attr_done) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
      LH_FAIL("igemm: cannot reserve %zu bytes of LDS", smem); return false;
    }
    attr_done = true;
  }
  ProfScope prof_(g_kernel_cat);
  hipLaunchKernelGGL(kern, dim3(8 * gs.perXcd), dim3(256), smem, g_stream, al, bl, ep, gs);
  return true;
}

// Whole tiles, and slices of the last ones (GemmShape::fixFull ...).  All tiles of these launches are resident at once, so a
// compute unit's time is the number of tiles it was given: with 784 tiles on 256 units some unit has four and the rest wait
// for it (3.06 on average: 76 %).  Here the multiple of the unit count that fits runs as whole tiles, one block each, and the
// tiles that are left are cut along the reduction into 2, 4 or 8 slices, one block each, so that the last blocks placed are
// small and land evenly.  The slices of a tile meet in a workspace; whichever arrives last adds them up in slice order and
// runs the epilogue, so the output needs no clearing, the epilogue sees complete sums (bias, clamp, batch-norm statistics
// work as on whole tiles) and the result does not depend on the order of arrival.  Main stream only: the counters and the
// workspace (arena scratch) have one user at a time.
constexpr int FIX_MAX_TILES = 4096;
template <int BM, int BN, int BK, class AL, class BL, class EP>
bool igemm_launch_shared_tail(const AL& al, const BL& bl, const EP& ep, int M, int N, int K, int col0 = 0, int col1 = -1) {
  constexpr size_t smem = igemm_smem_bytes<BM, BN, BK>();
  if constexpr (smem > 48 * 1024) { LH_FAIL("igemm: sliced tiles are not built for this tile shape"); return false; }
  else {
    if (col1 < 0 || col1 > N) col1 = N;
    if (col0 >= col1) return true;
    GemmShape gs{};
    gs.M = M; gs.N = col1; gs.K = K; gs.colBase = col0;
    gs.tilesM = (int)cdiv(M, BM); gs.tilesN = (int)cdiv(col1 - col0, BN);
    gs.slabsPerTile = (int)cdiv(K > 0 ? K : 1, BK);
    gs.units = (long long)gs.tilesM * gs.tilesN * gs.slabsPerTile;
    gs.streamk = 2; gs.splitK = 1;
    const int64_t tiles = (int64_t)gs.tilesM * gs.tilesN, cus = g_num_cu;
    if (cus % 8 != 0) return igemm_launch<BM, BN, BK>(al, bl, ep, M, N, K, 1, 0, col0, col1);
    const int64_t whole = tiles / cus * cus, tail = tiles - whole;
    // slices per tile of the tail: the count whose last placement round is fullest (what is lost is the idle part of that
    // round, in tiles per unit), at least four slabs per slice; ties go to the smaller count
    // (measured and dropped: preferring more slices at equal loss when there are fewer tiles than units, for the latency
    // more blocks per unit hide: the CIFAR-shaped ResNet-50 step went from 4.18 to 4.33 ms)
    int slices = 1; double best = 1e9;
    for (int sc = 1; sc <= 8; sc *= 2) {
      if (sc > 1 && gs.slabsPerTile / sc < 4) break;
      const double lost = (double)cdiv(tail * sc, cus) / sc - (double)tail / cus;
      if (lost < best - 1e-9) { best = lost; slices = sc; }
    }
    if (tail == 0 || slices == 1 || tail > FIX_MAX_TILES || tiles > 0x3fffffff || g_stream_cur != g_stream_raw)
      return igemm_launch<BM, BN, BK>(al, bl, ep, M, N, K, 1, 0, col0, col1);
    const int per = (int)cdiv(gs.slabsPerTile, slices);
    gs.kPerSplit = per * BK;
    gs.fixCmax = (int)cdiv(gs.slabsPerTile, per);
    gs.fixFull = (int)whole;
    const int64_t total = whole + tail * gs.fixCmax;
    gs.total = (int)total;
    gs.fixPer = (int)cdiv(tail * gs.fixCmax, 8);
    gs.perXcd = (int)(whole / 8) + gs.fixPer;          // (the unit count is a multiple of 8, so are the whole tiles)
    const size_t wsbytes = (size_t)tail * gs.fixCmax * BM * BN * sizeof(float);
    gs.fixWs = (float4*)lh_malloc_uninit(wsbytes);
    gs.fixCnt = fix_counters();
    if (gs.fixWs == nullptr || gs.fixCnt == nullptr) return false;
    if (getenv("LH_TAIL_VERBOSE")) fprintf(stderr, "sliced tail %dx%d: M%d N%d K%d: %lld whole tiles, %lld tiles in %d slices of %d slabs\n", BM, BN, M, col1 - col0, K, (long long)whole, (long long)tail, gs.fixCmax, per);
    {
      ProfScope prof_(g_kernel_cat);
      hipLaunchKernelGGL((k_igemm<BM, BN, BK, AL, BL, EP, 2>), dim3(8 * gs.perXcd), dim3(256), smem, g_stream, al, bl, ep, gs);
    }
    lh_free_top(wsbytes);
    return true;
  }
}

// Times `launch` (a callable returning false on failure) on the library's stream: five repetitions, the first warms
// the caches, the smallest of the other four counts (with two, which of two close plans won changed from run to run).  Returns a negative number when a launch or the timer failed.
struct LaunchTimer {
  hipEvent_t e0 = nullptr, e1 = nullptr;
  bool ok;
  LaunchTimer() { ok = hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess; quiet_other_stream(); }
  ~LaunchTimer() { if (e0) (void)hipEventDestroy(e0); if (e1) (void)hipEventDestroy(e1); }
  template <class F>
  float ms(F launch) {
    float best = 3.0e38f;
    for (int rep = 0; rep < 5; rep++) {
      (void)hipEventRecord(e0, g_stream);
      if (!launch()) return -1.f;
      (void)hipEventRecord(e1, g_stream);
      if (hipEventSynchronize(e1) != hipSuccess) return -1.f;
      float t = 0.f;
      if (hipEventElapsedTime(&t, e0, e1) != hipSuccess) return -1.f;
      if (rep > 0 && t < best) best = t;
    }
    return best;
  }
};

// One launch for up to IGEMM_MAX_GROUPS products that share loaders and tile shape (plain tiles: no k-split, no stream-K).
template <int BM, int BN, int BK, class AL, class BL, class EP>
bool igemm_launch_grouped(int ngroups, const AL* al, const BL* bl, const EP* ep, const int* M, const int* N, const int* K) {
  if (ngroups < 1 || ngroups > IGEMM_MAX_GROUPS) { LH_FAIL("igemm: %d groups", ngroups); return false; }
  IgemmGroups<AL, BL, EP> g;
  int64_t first = 0;
  for (int i = 0; i < IGEMM_MAX_GROUPS; i++) {
    const int j = i < ngroups ? i : 0;                      // unused slots repeat group 0 behind the last block
    g.al[i] = al[j]; g.bl[i] = bl[j]; g.ep[i] = ep[j];
    GemmShape& gs = g.gs[i];
    gs.M = M[j]; gs.N = N[j]; gs.K = K[j]; gs.colBase = 0;
    gs.tilesM = (int)cdiv(M[j], BM); gs.tilesN = (int)cdiv(N[j], BN);
    int kper = (int)cdiv(K[j] > 0 ? K[j] : 1, BK) * BK;
    gs.kPerSplit = kper; gs.splitK = 1;
    gs.slabsPerTile = (int)cdiv(K[j] > 0 ? K[j] : 1, BK);
    gs.units = (long long)gs.tilesM * gs.tilesN * gs.slabsPerTile;
    gs.streamk = 0;
    const int64_t total = (int64_t)gs.tilesM * gs.tilesN;
    gs.total = (int)total; gs.perXcd = (int)cdiv(total, 8);
    g.first[i] = (int)first;
    if (i < ngroups) first += 8 * (int64_t)gs.perXcd;
    if (first <= 0 || first > 0x3fffffff) { LH_FAIL("igemm: grouped tile count %lld out of range", (long long)first); return false; }
  }
  g.first[IGEMM_MAX_GROUPS] = (int)first;
  constexpr size_t smem = igemm_smem_bytes<BM, BN, BK>();
  auto kern = k_igemm_grouped<BM, BN, BK, AL, BL, EP>;
  static bool attr_done = false;
  if (smem > 48 * 1024 && !attr_done) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
      LH_FAIL("igemm: cannot reserve %zu bytes of LDS", smem); return false;
    }
    attr_done = true;
  }
  ProfScope prof_(g_kernel_cat);
  hipLaunchKernelGGL(kern, dim3((unsigned)first), dim3(256), smem, g_stream, g);
  return true;
}

// Tile choice: largest tile that still yields about two blocks per CU.
struct TilePick { int bm, bn; };
static inline TilePick pick_tile(int M, int N) {
  const int64_t want = 2 * (int64_t)g_num_cu;
  if (M > 64 && cdiv(M, 128) * cdiv(N, 128) >= want) return {128, 128};
  if (cdiv(M, 64) * cdiv(N, 128) >= want || N >= 8 * M) return {64, 128};
  return {64, 64};
}

}  // namespace lh
