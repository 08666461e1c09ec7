// Dense linear algebra outside convolution: sgemm (all four transpose cases), sgemv, rank-1
// update and vector dot.  Row-major, fp32.
#include "lh_igemm.h"
#include <array>
#include <map>
using namespace lh;

namespace {
constexpr int TPB = 256;

// Small products (below the MFMA path's sizes): 64x64 output tile per block, 64-deep k slabs through LDS, 4x4 register tile
// per thread.  These launches are latency-bound (one or a few blocks), so a slab is deep: all of a thread's 32 loads of
// a slab are independent and in flight together, and k = 100 takes two round trips to memory instead of seven.
constexpr int SMALL_KS = 64;
template <bool TA, bool TB>
__global__ void __launch_bounds__(TPB) k_sgemm_tile(int m, int n, int k, float alpha, const float* __restrict__ A, int lda,
                                                    const float* __restrict__ B, int ldb, float beta, float* __restrict__ C, int ldc, int kper) {
  // kper < k: blockIdx.z takes the slice [z * kper, (z + 1) * kper) of the reduction and adds its part to C atomically (C holds beta*C)
  __shared__ float As[SMALL_KS][64 + 4];
  __shared__ float Bs[SMALL_KS][64 + 4];
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int i0 = blockIdx.y * 64, j0 = blockIdx.x * 64;
  float acc[4][4] = {};
  const bool sliced = kper < k;
  const int kbeg = sliced ? (int)blockIdx.z * kper : 0, kend = sliced ? min(k, kbeg + kper) : k;
  for (int k0 = kbeg; k0 < kend; k0 += SMALL_KS) {
    const int kn = kend - k0 < SMALL_KS ? kend - k0 : SMALL_KS;
    float ra[SMALL_KS * 64 / TPB], rb[SMALL_KS * 64 / TPB];
#pragma unroll
    for (int r = 0; r < SMALL_KS * 64 / TPB; r++) {
      const int e = threadIdx.x + r * TPB;
      int kk, ii;
      if (TA) { ii = e & 63; kk = e >> 6; } else { kk = e & (SMALL_KS - 1); ii = e / SMALL_KS; }
      const int gi = i0 + ii, gk = k0 + kk;
      ra[r] = (gi < m && kk < kn) ? (TA ? A[(int64_t)gk * lda + gi] : A[(int64_t)gi * lda + gk]) : 0.f;
      int jj;
      if (TB) { kk = e & (SMALL_KS - 1); jj = e / SMALL_KS; } else { jj = e & 63; kk = e >> 6; }
      const int gj = j0 + jj; const int gk2 = k0 + kk;
      rb[r] = (gj < n && kk < kn) ? (TB ? B[(int64_t)gj * ldb + gk2] : B[(int64_t)gk2 * ldb + gj]) : 0.f;
    }
#pragma unroll
    for (int r = 0; r < SMALL_KS * 64 / TPB; r++) {
      const int e = threadIdx.x + r * TPB;
      if (TA) As[e >> 6][e & 63] = ra[r]; else As[e & (SMALL_KS - 1)][e / SMALL_KS] = ra[r];
      if (TB) Bs[e & (SMALL_KS - 1)][e / SMALL_KS] = rb[r]; else Bs[e >> 6][e & 63] = rb[r];
    }
    __syncthreads();
    const int kn8 = (kn + 7) & ~7;          // rows kn.. of the slab hold zeros
#pragma unroll 8
    for (int kk = 0; kk < kn8; kk++) {
      float a[4], b[4];
#pragma unroll
      for (int u = 0; u < 4; u++) { a[u] = As[kk][ty * 4 + u]; b[u] = Bs[kk][tx * 4 + u]; }
#pragma unroll
      for (int u = 0; u < 4; u++)
#pragma unroll
        for (int v = 0; v < 4; v++) acc[u][v] += a[u] * b[v];
    }
    __syncthreads();
  }
  for (int u = 0; u < 4; u++) {
    int gi = i0 + ty * 4 + u;
    if (gi >= m) continue;
    for (int v = 0; v < 4; v++) {
      int gj = j0 + tx * 4 + v;
      if (gj >= n) continue;
      float* c = C + (int64_t)gi * ldc + gj;
      if (sliced) atomicAdd(c, alpha * acc[u][v]);
      else *c = alpha * acc[u][v] + (beta == 0.f ? 0.f : beta * *c);
    }
  }
}

// y[m] = alpha * A[m,n] x[n] + beta*y : one wave per row.
__global__ void __launch_bounds__(TPB) k_sgemv_n(int m, int n, float alpha, const float* __restrict__ A, int lda, const float* __restrict__ x, float beta, float* y) {
  const int lane = threadIdx.x & 63;
  int64_t w = ((int64_t)blockIdx.x * TPB + threadIdx.x) >> 6, nw = ((int64_t)gridDim.x * TPB) >> 6;
  for (; w < m; w += nw) {
    const float* row = A + w * lda;
    float acc = 0.f;
    for (int j = lane; j < n; j += 64) acc += row[j] * x[j];
    acc = lh_wave_sum(acc);
    if (lane == 0) y[w] = alpha * acc + (beta == 0.f ? 0.f : beta * y[w]);
  }
}
// y[n] = alpha * A[m,n]^T x[m] + beta*y : a block owns 32 columns; its 8 row groups each sum every 8th row
// (independent, coalesced loads), and LDS combines the groups.
__global__ void __launch_bounds__(TPB) k_sgemv_t(int m, int n, float alpha, const float* __restrict__ A, int lda, const float* __restrict__ x, float beta, float* y) {
  __shared__ float sm[8][33];
  const int c = threadIdx.x & 31, g = threadIdx.x >> 5;
  const int j = blockIdx.x * 32 + c;
  float acc0 = 0.f, acc1 = 0.f, acc2 = 0.f, acc3 = 0.f;
  if (j < n) {
    const float* a = A + j;
    int i = g;
    for (; i + 24 < m; i += 32) {
      acc0 += a[(int64_t)i * lda] * x[i];
      acc1 += a[(int64_t)(i + 8) * lda] * x[i + 8];
      acc2 += a[(int64_t)(i + 16) * lda] * x[i + 16];
      acc3 += a[(int64_t)(i + 24) * lda] * x[i + 24];
    }
    for (; i < m; i += 8) acc0 += a[(int64_t)i * lda] * x[i];
  }
  sm[g][c] = (acc0 + acc1) + (acc2 + acc3);
  __syncthreads();
  if (g == 0 && j < n) {
    float acc = ((sm[0][c] + sm[1][c]) + (sm[2][c] + sm[3][c])) + ((sm[4][c] + sm[5][c]) + (sm[6][c] + sm[7][c]));
    y[j] = alpha * acc + (beta == 0.f ? 0.f : beta * y[j]);
  }
}
__global__ void __launch_bounds__(TPB) k_ger(int m, int n, const float* __restrict__ u, const float* __restrict__ v, float* A) {
  int64_t tot = (int64_t)m * n;
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < tot; i += st) { int r = (int)(i / n), c = (int)(i - (int64_t)r * n); A[i] = A[i] + v[c] * u[r]; }
}
__global__ void __launch_bounds__(TPB) k_dot(const float* x, const float* y, float* out, int n) {
  __shared__ float sm[17];
  float acc = 0.f;
  for (int i = threadIdx.x; i < n; i += TPB) acc += x[i] * y[i];
  acc = lh_block_sum(acc, sm);
  if (threadIdx.x == 0) out[0] = acc;
}
__global__ void __launch_bounds__(TPB) k_axpy_dev(float* y, const float* s, const float* x, int64_t n) {
  float a = s[0];
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < n; i += st) y[i] = y[i] + a * x[i];
}
}  // namespace

extern "C" {

}  // extern "C"
// MFMA path for all but tiny products; the 64x64 register-tiled kernel covers those.
struct SgemmPlan { TilePick tp; int split; };
// Few output tiles and a long reduction (weight gradients over many rows): the reduction is cut into `split`
// slices whose blocks add into C with fp32 atomics; C is scaled by beta beforehand.
static SgemmPlan sgemm_plan(int m, int n, int k) {
  SgemmPlan p; p.tp = pick_tile(m, n); p.split = 1;
  const int64_t tiles = cdiv(m, p.tp.bm) * cdiv(n, p.tp.bn);
  if (k >= 1024 && 2 * tiles <= 3 * (int64_t)g_num_cu) {
    TilePick big = (m >= 128 && n >= 128) ? TilePick{128, 128} : (n >= 128 ? TilePick{64, 128} : TilePick{64, 64});
    const int64_t bt = cdiv(m, big.bm) * cdiv(n, big.bn);
    int split = (int)cdiv(3 * (int64_t)g_num_cu, bt);
    const int max_split = k / 256;
    if (split > max_split) split = max_split;
    if (split > 1) { p.tp = big; p.split = split; }
  }
  return p;
}
__global__ void __launch_bounds__(TPB) k_scale_rows(float* C, int ldc, int m, int n, float beta) {
  const int64_t tot = (int64_t)m * n;
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < tot; i += st) { const int r = (int)(i / n), c = (int)(i - (int64_t)r * n); float* p = C + (int64_t)r * ldc + c; *p = beta == 0.f ? 0.f : beta * *p; }
}
// C = beta*C + sum of the slices' partial products, in slice order (the deterministic stand-in for atomic adds).
// VEC: n and ldc are multiples of 4 and both pointers 16-byte aligned: four neighbours per lane, the loads of eight slices in flight.
template <bool VEC>
__global__ void __launch_bounds__(TPB) k_reduce_slices(float* C, int ldc, int m, int n, const float* __restrict__ partial, int slices, float beta) {
  if (VEC) {
    const int n4 = n >> 2;
    const int64_t tot4 = (int64_t)m * n4;
    const float4* __restrict__ P = reinterpret_cast<const float4*>(partial);
    int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
    for (; i < tot4; i += st) {
      const int r = (int)(i / n4), c = (int)(i - (int64_t)r * n4);
      float4* p = reinterpret_cast<float4*>(C + (int64_t)r * ldc) + c;
      float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
      if (beta != 0.f) { const float4 o = *p; acc = make_float4(beta * o.x, beta * o.y, beta * o.z, beta * o.w); }
      int s = 0;
      for (; s + 8 <= slices; s += 8) {
        float4 v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = P[(int64_t)(s + u) * tot4 + i];
#pragma unroll
        for (int u = 0; u < 8; u++) { acc.x += v[u].x; acc.y += v[u].y; acc.z += v[u].z; acc.w += v[u].w; }
      }
      for (; s < slices; s++) { const float4 v = P[(int64_t)s * tot4 + i]; acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w; }
      *p = acc;
    }
    return;
  }
  const int64_t tot = (int64_t)m * n;
  int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x, st = (int64_t)gridDim.x * TPB;
  for (; i < tot; i += st) {
    const int r = (int)(i / n), c = (int)(i - (int64_t)r * n);
    float* p = C + (int64_t)r * ldc + c;
    float acc = beta == 0.f ? 0.f : beta * *p;
    for (int s = 0; s < slices; s++) acc += partial[(int64_t)s * tot + i];
    *p = acc;
  }
}
template <class AL, class BL>
static bool sgemm_mfma(const AL& al, const BL& bl, const EpiRowMajor& ep, int m, int n, int k, const SgemmPlan& pl) {
  if (pl.tp.bm == 128) return igemm_launch<128, 128, 16>(al, bl, ep, m, n, k, pl.split);
  if (pl.tp.bn == 128) return igemm_launch<64, 128, 16>(al, bl, ep, m, n, k, pl.split);
  return igemm_launch<64, 64, 16>(al, bl, ep, m, n, k, pl.split);
}

namespace lh {
void reduce_slices(float* C, int ldc, int m, int n, const float* partial, int slices, float beta) {
  const bool vec = (n % 4 == 0) && (ldc % 4 == 0) && ((((uintptr_t)C | (uintptr_t)partial) & 15) == 0);
  if (vec) hipLaunchKernelGGL((k_reduce_slices<true>), dim3(stream_grid((int64_t)m * (n / 4), TPB)), dim3(TPB), 0, g_stream, C, ldc, m, n, partial, slices, beta);
  else hipLaunchKernelGGL((k_reduce_slices<false>), dim3(stream_grid((int64_t)m * n, TPB * 2)), dim3(TPB), 0, g_stream, C, ldc, m, n, partial, slices, beta);
}
}  // namespace lh

void lh_sgemm(int ta, int tb, int m, int n, int k, float alpha, const float* A, int lda,
              const float* B, int ldb, float beta, float* C, int ldc) {
  KernelCat kc_(CAT_GEMM);
  if (m <= 0 || n <= 0) return;
  LH_REQUIRE(k >= 0, "lh_sgemm: negative k");
  LH_REQUIRE(lda >= (ta ? m : k) && ldb >= (tb ? k : n) && ldc >= n, "lh_sgemm: leading dimensions (%d,%d,%d) too small for m%d n%d k%d ta%d tb%d", lda, ldb, ldc, m, n, k, ta, tb);
  LH_REQUIRE(A && B && C, "lh_sgemm: null operand");
  LZ_ENTER();
  if (lazy::g_busy && !lazy::g_replay) {
    lazy::rd_f(A, (int64_t)((ta ? k : m) - 1) * lda + (ta ? m : k)); lazy::rd_f(B, (int64_t)((tb ? n : k) - 1) * ldb + (tb ? k : n));
    if (ldc == n && (beta == 0.f || beta == 1.f)) beta = lazy::beta_f(C, (int64_t)m * n, beta);     // a product added into a block nobody has touched overwrites it
    else lazy::rw_f(C, (int64_t)(m - 1) * ldc + n);
  }
  if ((int64_t)m * n * k >= (1 << 18) && m >= 16 && n >= 16) {
    const bool av = (lda % 4 == 0) && (((uintptr_t)A & 15) == 0) && (k % 4 == 0);
    const bool bv = (ldb % 4 == 0) && (((uintptr_t)B & 15) == 0) && (k % 4 == 0);
    const size_t abytes = (size_t)(ta ? k : m) * lda * 4, bbytes = (size_t)(tb ? n : k) * ldb * 4;
    LH_REQUIRE(abytes <= 0x80000000ull && bbytes <= 0x80000000ull, "lh_sgemm: operands above 2 GiB are not supported");
    LoadPlainK<true> akv; akv.base = A; akv.nbytes = (uint32_t)abytes; akv.ld = lda;
    LoadPlainK<false> aks; aks.base = A; aks.nbytes = (uint32_t)abytes; aks.ld = lda;
    LoadPlainT at; at.base = A; at.nbytes = (uint32_t)abytes; at.ld = lda;
    LoadPlainK<true> bkv; bkv.base = B; bkv.nbytes = (uint32_t)bbytes; bkv.ld = ldb;
    LoadPlainK<false> bks; bks.base = B; bks.nbytes = (uint32_t)bbytes; bks.ld = ldb;
    LoadPlainT bt; bt.base = B; bt.nbytes = (uint32_t)bbytes; bt.ld = ldb;
    // one product under plan `pl` into Cout (row stride ldo) with the given beta
    auto run = [&](const SgemmPlan& pl, float* Cout, int ldo, float be) -> bool {
      EpiRowMajor e; e.C = Cout; e.ldc = ldo; e.alpha = alpha; e.beta = be; e.atomic = 0;
      float* partial = nullptr; size_t pbytes = 0; int slices = 1; bool pside = false;
      if (pl.split > 1 && g_deterministic) {            // slices into scratch blocks, added in order afterwards
        int64_t kper = cdiv(cdiv(k, pl.split), 16) * 16; if (kper < 16) kper = 16;
        slices = (int)cdiv(k, kper);
        pbytes = (size_t)slices * m * n * sizeof(float);
        partial = (float*)scratch_take(pbytes, pside);
        if (partial == nullptr) return false;
        e.C = partial; e.ldc = n; e.beta = 0.f; e.sliceStride = (long long)m * n;
      } else if (pl.split > 1) {
        if (be != 1.f) { hipLaunchKernelGGL(k_scale_rows, dim3(stream_grid((int64_t)m * n, TPB * 4)), dim3(TPB), 0, g_stream, Cout, ldo, m, n, be); }
        e.atomic = 1; e.beta = 1.f;
      }
      bool good;
      if (!ta && !tb) good = av ? sgemm_mfma(akv, bt, e, m, n, k, pl) : sgemm_mfma(aks, bt, e, m, n, k, pl);
      else if (!ta && tb) good = av ? (bv ? sgemm_mfma(akv, bkv, e, m, n, k, pl) : sgemm_mfma(akv, bks, e, m, n, k, pl))
                                    : (bv ? sgemm_mfma(aks, bkv, e, m, n, k, pl) : sgemm_mfma(aks, bks, e, m, n, k, pl));
      else if (ta && !tb) good = sgemm_mfma(at, bt, e, m, n, k, pl);
      else good = bv ? sgemm_mfma(at, bkv, e, m, n, k, pl) : sgemm_mfma(at, bks, e, m, n, k, pl);
      if (partial) {
        if (good) reduce_slices(Cout, ldo, m, n, partial, slices, be);
        scratch_give(pbytes, pside);
      }
      return good;
    };
    SgemmPlan pl = sgemm_plan(m, n, k);
    // Tile shape and reduction slices are measured once per (transposes, m, n, k) on a scratch output and remembered.
    static std::map<std::array<int, 7>, SgemmPlan> chosen;
    if (g_tune_lookup && 2.0 * m * n * (double)k >= g_tune_min_flop) {
      const std::array<int, 7> key = {ta, tb, m, n, k, (int)av, (int)bv};
      auto it = chosen.find(key);
      if (it != chosen.end()) { pl = it->second; g_plans_remembered++; }
      else if (g_tune_measure) {
        const size_t sbytes = (size_t)m * n * sizeof(float);
        bool sside = false;
        float* scratch = (float*)scratch_take(sbytes, sside);
        LaunchTimer timer;
        if (scratch && timer.ok) {
          const TilePick shapes[3] = {{128, 128}, {64, 128}, {64, 64}};
          const double targets[] = {1.5, 3.0, 4.5};
          float best_ms = timer.ms([&]() { return run(pl, scratch, n, 0.f); });
          SgemmPlan best = pl;
          for (int sh = 0; sh < 3 && best_ms >= 0.f && !failed(); sh++) {
            if ((shapes[sh].bm == 128 && m <= 64) || (shapes[sh].bn == 128 && n <= 64)) continue;
            const int64_t tiles = cdiv(m, shapes[sh].bm) * cdiv(n, shapes[sh].bn);
            int cand[4] = {1, 0, 0, 0}; int nc = 1;
            for (double tg : targets) {
              int sp = (int)((int64_t)(tg * g_num_cu) / tiles);
              if (sp > k / 256) sp = k / 256;
              bool dup = sp <= 1;
              for (int i = 0; i < nc; i++) dup = dup || cand[i] == sp;
              if (!dup) cand[nc++] = sp;
            }
            for (int i = 0; i < nc; i++) {
              SgemmPlan c; c.tp = shapes[sh]; c.split = cand[i];
              const float ms = timer.ms([&]() { return run(c, scratch, n, 0.f); });
              if (ms < 0.f) { best_ms = -1.f; break; }
              if (ms < best_ms * 0.98f) { best_ms = ms; best = c; }
            }
          }
          if (best_ms >= 0.f && !failed()) { chosen[key] = best; pl = best; g_plans_measured++; }
          if (getenv("LH_TUNE_VERBOSE")) fprintf(stderr, "sgemm ta%d tb%d %dx%dx%d: tile %dx%d, %d slice(s), %.3f ms\n", ta, tb, m, n, k, best.tp.bm, best.tp.bn, best.split, best_ms);
        }
        if (scratch) scratch_give(sbytes, sside);
        if (failed()) return;
      }
    }
    const bool ok = run(pl, C, ldc, beta);
    if (!ok) return;
    LH_CHECK_LAUNCH();
    return;
  }
  ProfScope prof_(CAT_GEMM);
  dim3 grid((unsigned)cdiv(n, 64), (unsigned)cdiv(m, 64));
  // A few tiles over a long reduction (a classifier with ten outputs behind 2048 features: one block walking 32 slabs took
  // 194 us): the reduction is cut into slices of at least 128 that add into beta*C.
  int kper = k;
  if (k >= 512 && (int64_t)grid.x * grid.y <= 64 && !g_deterministic) {
    int slices = k / 128; if (slices > 32) slices = 32;
    kper = (int)cdiv(cdiv(k, slices), SMALL_KS) * SMALL_KS;
    grid.z = (unsigned)cdiv(k, kper);
    if (grid.z > 1 && beta != 1.f) hipLaunchKernelGGL(k_scale_rows, dim3(stream_grid((int64_t)m * n, TPB * 4)), dim3(TPB), 0, g_stream, C, ldc, m, n, beta);
    if (grid.z <= 1) kper = k;
  }
  if (!ta && !tb) hipLaunchKernelGGL((k_sgemm_tile<false, false>), grid, dim3(TPB), 0, g_stream, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, kper);
  else if (!ta && tb) hipLaunchKernelGGL((k_sgemm_tile<false, true>), grid, dim3(TPB), 0, g_stream, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, kper);
  else if (ta && !tb) hipLaunchKernelGGL((k_sgemm_tile<true, false>), grid, dim3(TPB), 0, g_stream, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, kper);
  else hipLaunchKernelGGL((k_sgemm_tile<true, true>), grid, dim3(TPB), 0, g_stream, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, kper);
  LH_CHECK_LAUNCH();
}
extern "C" {
void lh_sgemv(int trans, int m, int n, float alpha, const float* A, int lda, const float* x, float beta, float* y) {
  if (m <= 0 || n <= 0) return;
  LZ_ENTER(); lazy::rd_f(A, (int64_t)(m - 1) * lda + n); lazy::rd_f(x, trans ? m : n); lazy::rw_f(y, trans ? n : m);
  ProfScope prof_(CAT_GEMM);
  if (rec_ok((int64_t)m * n, REC_MAX_MATRIX)) { rec_cmd(trans ? CL_GEMV_T : CL_GEMV_N, m, n, lda, alpha, beta, 0.f, 0.f, y, A, x, nullptr); return; }
  if (!trans) hipLaunchKernelGGL(k_sgemv_n, dim3(stream_grid((int64_t)m * 64, TPB)), dim3(TPB), 0, g_stream, m, n, alpha, A, lda, x, beta, y);
  else hipLaunchKernelGGL(k_sgemv_t, dim3((unsigned)cdiv(n, 32)), dim3(TPB), 0, g_stream, m, n, alpha, A, lda, x, beta, y);
  LH_CHECK_LAUNCH();
}
void lh_ger(int m, int n, const float* u, const float* v, float* A) {
  if (m <= 0 || n <= 0) return;
  LZ_ENTER(); lazy::rd_f(u, m); lazy::rd_f(v, n); lazy::rw_f(A, (int64_t)m * n);
  ProfScope prof_(CAT_GEMM);
  if (rec_ok((int64_t)m * n, REC_MAX_MATRIX)) { rec_cmd(CL_GER, m, n, 0, 0.f, 0.f, 0.f, 0.f, A, u, v, nullptr); return; }
  hipLaunchKernelGGL(k_ger, dim3(stream_grid((int64_t)m * n, TPB * 4)), dim3(TPB), 0, g_stream, m, n, u, v, A);
  LH_CHECK_LAUNCH();
}
void lh_dot_vv(const float* x, const float* y, float* out, int n) {
  LZ_ENTER(); lazy::rd_f(x, n); lazy::rd_f(y, n); lazy::wr_f(out, 1);
  if (rec_ok(n)) { rec_cmd(CL_DOT, n, 0, 0, 0.f, 0.f, 0.f, 0.f, out, x, y, nullptr); return; }
  hipLaunchKernelGGL(k_dot, dim3(1), dim3(TPB), 0, g_stream, x, y, out, n);
  LH_CHECK_LAUNCH();
}
void lh_axpy_dev(float* y, const float* s, const float* x, int64_t n) {
  if (n <= 0) return;
  LZ_ENTER(); lazy::rd_f(s, 1); lazy::rd_f(x, n); lazy::rw_f(y, n);
  if (rec_ok(n)) { rec_cmd(CL_AXPY_DEV, (int)n, 0, 0, 0.f, 0.f, 0.f, 0.f, y, s, x, nullptr); return; }
  hipLaunchKernelGGL(k_axpy_dev, dim3(stream_grid(n, TPB * 4)), dim3(TPB), 0, g_stream, y, s, x, n);
  LH_CHECK_LAUNCH();
}

}  // extern "C"
