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
  int M, N, K;
  int tilesM, tilesN, splitK, kPerSplit;
  int total, perXcd;
};

// ---- plain matrix loaders -------------------------------------------------------------------
// Element (col, k) at base[col*ld + k]  (k contiguous).
struct LoadPlainK {
  static constexpr bool ALONG_K = true;
  const float* base; int ld; int vec;   // vec: rows are 16-byte aligned and ld % 4 == 0
  struct State { const float* row; bool valid; };
  __device__ __forceinline__ void init(State& s, int col, int ncols) const { s.valid = col < ncols; s.row = base + (int64_t)(s.valid ? col : 0) * ld; }
  __device__ __forceinline__ float4 load4(const State& s, int k, int kend) const {
    float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
    if (!s.valid) return r;
    if (vec && k + 3 < kend) return *reinterpret_cast<const float4*>(s.row + k);
    if (k < kend) r.x = s.row[k];
    if (k + 1 < kend) r.y = s.row[k + 1];
    if (k + 2 < kend) r.z = s.row[k + 2];
    if (k + 3 < kend) r.w = s.row[k + 3];
    return r;
  }
};
// Element (col, k) at base[k*ld + col]  (col contiguous).
struct LoadPlainT {
  static constexpr bool ALONG_K = false;
  const float* base; int ld;
  struct State { const float* colp; bool valid; };
  __device__ __forceinline__ void init(State& s, int col, int ncols) const { s.valid = col < ncols; s.colp = base + (s.valid ? col : 0); }
  __device__ __forceinline__ float4 load4(const State& s, int k, int kend) const {
    float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
    if (!s.valid) return r;
    if (k < kend) r.x = s.colp[(int64_t)k * ld];
    if (k + 1 < kend) r.y = s.colp[(int64_t)(k + 1) * ld];
    if (k + 2 < kend) r.z = s.colp[(int64_t)(k + 2) * ld];
    if (k + 3 < kend) r.w = s.colp[(int64_t)(k + 3) * ld];
    return r;
  }
};

// ---- epilogue for row-major C ------------------------------------------------------------------
// mode 0: C = alpha*acc + beta*C ; mode 1: atomicAdd(C, alpha*acc) (split-K)
struct EpiRowMajor {
  float* C; int ldc; float alpha, beta; int atomic;
  struct Col { int j; bool valid; };
  __device__ __forceinline__ Col col(int j, int N) const { Col c; c.j = j; c.valid = j < N; return c; }
  __device__ __forceinline__ void store(const Col& c, int i, int M, float v) const {
    if (!c.valid || i >= M) return;
    float* p = C + (int64_t)i * ldc + c.j;
    if (atomic) atomicAdd(p, alpha * v);
    else *p = alpha * v + (beta == 0.f ? 0.f : beta * *p);
  }
};

// ---- the kernel ------------------------------------------------------------------------------------
template <int BM, int BN, int BK, class AL, class BL, class EP>
__global__ void __launch_bounds__(256) k_igemm(const AL al, const BL bl, const EP ep, const GemmShape gs) {
  constexpr int KQ = BK / 4, PAD = 8 / KQ, LDA = BM + PAD, LDB = BN + PAD;
  constexpr int TM = BM / 2, TN = BN / 2, MI = TM / 32, NI = TN / 32;
  constexpr int GA = BM * KQ / 256, GB = BN * KQ / 256;
  static_assert(GA >= 1 && GB >= 1 && MI >= 1 && NI >= 1, "tile too small for 256 threads");
  extern __shared__ float4 lh_smem[];
  float4* As = lh_smem;
  float4* Bs = lh_smem + 2 * KQ * LDA;

  const int logical = (blockIdx.x % 8) * gs.perXcd + blockIdx.x / 8;
  if (logical >= gs.total) return;
  const int tm = logical % gs.tilesM;
  const int rest = logical / gs.tilesM;
  const int tn = rest % gs.tilesN, sp = rest / gs.tilesN;
  const int m0 = tm * BM, n0 = tn * BN;
  const int kbeg = sp * gs.kPerSplit, kend = min(gs.K, kbeg + gs.kPerSplit);

  const int t = threadIdx.x;
  typename AL::State sa[GA];
  typename BL::State sb[GB];
  int a_col[GA], a_kq[GA], b_col[GB], b_kq[GB];
#pragma unroll
  for (int g = 0; g < GA; g++) {
    if (AL::ALONG_K) { a_kq[g] = t % KQ; a_col[g] = t / KQ + g * (256 / KQ); }
    else { a_col[g] = t % BM; a_kq[g] = __builtin_amdgcn_readfirstlane(t / BM) + g * (256 / BM); }
    al.init(sa[g], m0 + a_col[g], gs.M);
  }
#pragma unroll
  for (int g = 0; g < GB; g++) {
    if (BL::ALONG_K) { b_kq[g] = t % KQ; b_col[g] = t / KQ + g * (256 / KQ); }
    else { b_col[g] = t % BN; b_kq[g] = __builtin_amdgcn_readfirstlane(t / BN) + g * (256 / BN); }
    bl.init(sb[g], n0 + b_col[g], gs.N);
  }

  f32x16 acc[MI][NI];
#pragma unroll
  for (int mi = 0; mi < MI; mi++)
#pragma unroll
    for (int ni = 0; ni < NI; ni++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[mi][ni][v] = 0.f;

  const int lane = t & 63, wave = t >> 6, wm = wave >> 1, wn = wave & 1, half = lane >> 5, l32 = lane & 31;
  const int niter = (kend - kbeg + BK - 1) / BK;
  float4 ra[GA], rb[GB];

  if (niter > 0) {
#pragma unroll
    for (int g = 0; g < GA; g++) ra[g] = al.load4(sa[g], kbeg + 4 * a_kq[g], kend);
#pragma unroll
    for (int g = 0; g < GB; g++) rb[g] = bl.load4(sb[g], kbeg + 4 * b_kq[g], kend);
#pragma unroll
    for (int g = 0; g < GA; g++) As[a_kq[g] * LDA + a_col[g]] = ra[g];
#pragma unroll
    for (int g = 0; g < GB; g++) Bs[b_kq[g] * LDB + b_col[g]] = rb[g];
  }
  __syncthreads();

  for (int it = 0; it < niter; it++) {
    const int st = it & 1;
    const bool more = it + 1 < niter;
    if (more) {
      const int k0 = kbeg + (it + 1) * BK;
#pragma unroll
      for (int g = 0; g < GA; g++) ra[g] = al.load4(sa[g], k0 + 4 * a_kq[g], kend);
#pragma unroll
      for (int g = 0; g < GB; g++) rb[g] = bl.load4(sb[g], k0 + 4 * b_kq[g], kend);
    }
    const float4* Asc = As + st * KQ * LDA + wm * TM + l32;
    const float4* Bsc = Bs + st * KQ * LDB + wn * TN + l32;
#pragma unroll
    for (int pair = 0; pair < KQ / 2; pair++) {
      const int kq = 2 * pair + half;
      float4 a[MI], b[NI];
#pragma unroll
      for (int mi = 0; mi < MI; mi++) a[mi] = Asc[kq * LDA + mi * 32];
#pragma unroll
      for (int ni = 0; ni < NI; ni++) b[ni] = Bsc[kq * LDB + ni * 32];
#pragma unroll
      for (int mi = 0; mi < MI; mi++)
#pragma unroll
        for (int ni = 0; ni < NI; ni++) {
          acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[mi].x, b[ni].x, acc[mi][ni], 0, 0, 0);
          acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[mi].y, b[ni].y, acc[mi][ni], 0, 0, 0);
          acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[mi].z, b[ni].z, acc[mi][ni], 0, 0, 0);
          acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[mi].w, b[ni].w, acc[mi][ni], 0, 0, 0);
        }
    }
    if (more) {
      const int o = (st ^ 1) * KQ;
#pragma unroll
      for (int g = 0; g < GA; g++) As[(o + a_kq[g]) * LDA + a_col[g]] = ra[g];
#pragma unroll
      for (int g = 0; g < GB; g++) Bs[(o + b_kq[g]) * LDB + b_col[g]] = rb[g];
    }
    __syncthreads();
  }

  // D layout of a 32x32 block: column = lane % 32, row = 8*(v/4) + 4*(lane/32) + v%4
#pragma unroll
  for (int ni = 0; ni < NI; ni++) {
    const typename EP::Col cs = ep.col(n0 + wn * TN + ni * 32 + l32, gs.N);
#pragma unroll
    for (int mi = 0; mi < MI; mi++) {
      const int ib = m0 + wm * TM + mi * 32 + 4 * half;
#pragma unroll
      for (int v = 0; v < 16; v++) ep.store(cs, ib + 8 * (v / 4) + (v % 4), gs.M, acc[mi][ni][v]);
    }
  }
}

template <int BM, int BN, int BK>
constexpr size_t igemm_smem_bytes() { return (size_t)2 * (BK / 4) * ((BM + 8 / (BK / 4)) + (BN + 8 / (BK / 4))) * sizeof(float4); }

// Launch one tile configuration.  splitK > 1 requires an accumulating (atomic) epilogue.
template <int BM, int BN, int BK, class AL, class BL, class EP>
bool igemm_launch(const AL& al, const BL& bl, const EP& ep, int M, int N, int K, int splitK) {
  GemmShape gs;
  gs.M = M; gs.N = N; gs.K = K;
  gs.tilesM = (int)cdiv(M, BM); gs.tilesN = (int)cdiv(N, BN);
  if (splitK < 1) splitK = 1;
  int kper = (int)cdiv(cdiv(K, splitK), BK) * BK;
  if (kper < BK) kper = BK;
  gs.kPerSplit = kper;
  gs.splitK = (int)cdiv(K > 0 ? K : 1, kper);
  int64_t total = (int64_t)gs.tilesM * gs.tilesN * gs.splitK;
  if (total <= 0 || total > 0x3fffffff) { LH_FAIL("igemm: tile count %lld out of range", (long long)total); return false; }
  gs.total = (int)total; gs.perXcd = (int)cdiv(total, 8);
  constexpr size_t smem = igemm_smem_bytes<BM, BN, BK>();
  auto kern = k_igemm<BM, BN, BK, AL, BL, EP>;
  static bool attr_done = false;
  if (smem > 48 * 1024 && !attr_done) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
      LH_FAIL("igemm: cannot reserve %zu bytes of LDS", smem); return false;
    }
    attr_done = true;
  }
  hipLaunchKernelGGL(kern, dim3(8 * gs.perXcd), dim3(256), smem, g_stream, al, bl, ep, gs);
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
