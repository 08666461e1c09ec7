/*
 * TEST INFRASTRUCTURE, NOT PRODUCT: CPU restatement of Lantern's BackendCPU.
 * See lantern_cpu.h for the conventions, the reference files followed and the
 * pinning status.  Loops are written the way the reference's emitted C runs
 * them (single pass, float accumulators unless the reference widens), so
 * results follow BackendCPU's arithmetic; the one place that cannot be line
 * faithful is SGEMM/SGEMV, which the reference hands to OpenBLAS (not
 * vendored): lc_sgemm is an own packed kernel with float accumulation.
 */
#include "lantern_cpu.h"
#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 1;
void lc_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int lc_get_threads(void) { return g_threads; }

/* ------------------------------------------------------------------ fill */
void lc_fill(float* x, float v, long n) { for (long i = 0; i < n; i++) x[i] = v; }

void lc_fill_with_bias(float* y, const float* bias, long outer, long c, long inner) {
  long off = 0;
  for (long hd = 0; hd < outer; hd++)
    for (long cd = 0; cd < c; cd++)
      for (long ld = 0; ld < inner; ld++) y[off++] = bias[cd];
}

void lc_srand(unsigned seed) { srand(seed); }
/* ref emits "(float)rand()/RAND_MAX" (TD:66-69) */
static inline float ref_rand(void) { return (float)rand() / RAND_MAX; }
void lc_rand_uniform(float* x, long n) { for (long i = 0; i < n; i++) x[i] = (ref_rand() - 0.5f) * 1.0f; }

void lc_clip(float* x, float bound, long n) {
  for (long i = 0; i < n; i++) {
    float t = x[i];
    if (t > bound) x[i] = bound;
    if (t < -1.0f * bound) x[i] = -1.0f * bound;
  }
}

/* ----------------------------------------------------------------- sgemm */
/* Row-major C = alpha*op(A)*op(B) + beta*C.  Packed 6x16 register tile, float
 * accumulators, k in increasing order inside a KC block, blocks added in
 * increasing k order. */
typedef float v8f __attribute__((vector_size(32), aligned(4)));
#define MR 6
#define NR 16
#define KC 256
#define MC 96
#define NC 2048

static void pack_a(int ta, const float* A, int lda, int i0, int mb, int k0, int kb, float* dst) {
  for (int i = 0; i < mb; i += MR) {
    int ib = mb - i < MR ? mb - i : MR;
    for (int k = 0; k < kb; k++) {
      for (int ii = 0; ii < MR; ii++) {
        float v = 0.0f;
        if (ii < ib) v = ta ? A[(size_t)(k0 + k) * lda + (i0 + i + ii)] : A[(size_t)(i0 + i + ii) * lda + (k0 + k)];
        *dst++ = v;
      }
    }
  }
}
static void pack_b(int tb, const float* B, int ldb, int k0, int kb, int j0, int nb, float* dst) {
  for (int j = 0; j < nb; j += NR) {
    int jb = nb - j < NR ? nb - j : NR;
    for (int k = 0; k < kb; k++) {
      if (!tb && jb == NR) {
        memcpy(dst, B + (size_t)(k0 + k) * ldb + (j0 + j), NR * sizeof(float));
        dst += NR;
      } else {
        for (int jj = 0; jj < NR; jj++) {
          float v = 0.0f;
          if (jj < jb) v = tb ? B[(size_t)(j0 + j + jj) * ldb + (k0 + k)] : B[(size_t)(k0 + k) * ldb + (j0 + j + jj)];
          *dst++ = v;
        }
      }
    }
  }
}
static inline void micro(int kb, const float* a, const float* b, float* acc /* MR*NR */) {
  v8f c[MR][2];
  for (int i = 0; i < MR; i++) { c[i][0] = (v8f){0}; c[i][1] = (v8f){0}; }
  for (int k = 0; k < kb; k++) {
    v8f b0 = *(const v8f*)(b + k * NR), b1 = *(const v8f*)(b + k * NR + 8);
    for (int i = 0; i < MR; i++) {
      float av = a[k * MR + i];
      v8f avv = {av, av, av, av, av, av, av, av};
      c[i][0] += avv * b0;
      c[i][1] += avv * b1;
    }
  }
  for (int i = 0; i < MR; i++) { *(v8f*)(acc + i * NR) = c[i][0]; *(v8f*)(acc + i * NR + 8) = c[i][1]; }
}

void lc_sgemm(int ta, int tb, int m, int n, int k, float alpha, const float* A, int lda,
              const float* B, int ldb, float beta, float* C, int ldc) {
  if (m <= 0 || n <= 0) return;
  if (beta != 1.0f) {
    for (int i = 0; i < m; i++)
      for (int j = 0; j < n; j++) C[(size_t)i * ldc + j] = beta == 0.0f ? 0.0f : beta * C[(size_t)i * ldc + j];
  }
  if (k <= 0 || alpha == 0.0f) return;
  int nth = g_threads;
  for (int j0 = 0; j0 < n; j0 += NC) {
    int nb = n - j0 < NC ? n - j0 : NC;
    int nbp = (nb + NR - 1) / NR * NR;
    for (int k0 = 0; k0 < k; k0 += KC) {
      int kb = k - k0 < KC ? k - k0 : KC;
      float* pb = (float*)aligned_alloc(64, (size_t)nbp * kb * sizeof(float));
      pack_b(tb, B, ldb, k0, kb, j0, nb, pb);
      int nblk = (m + MC - 1) / MC;
#pragma omp parallel for schedule(dynamic) num_threads(nth) if (nth > 1 && nblk > 1)
      for (int ib = 0; ib < nblk; ib++) {
        int i0 = ib * MC;
        int mb = m - i0 < MC ? m - i0 : MC;
        int mbp = (mb + MR - 1) / MR * MR;
        float pa[MC * KC] __attribute__((aligned(64)));
        float acc[MR * NR] __attribute__((aligned(64)));
        pack_a(ta, A, lda, i0, mb, k0, kb, pa);
        for (int j = 0; j < nb; j += NR) {
          int jb = nb - j < NR ? nb - j : NR;
          for (int i = 0; i < mbp; i += MR) {
            int ibb = mb - i < MR ? mb - i : MR;
            micro(kb, pa + (size_t)i * kb, pb + (size_t)j * kb, acc);
            for (int ii = 0; ii < ibb; ii++) {
              float* crow = C + (size_t)(i0 + i + ii) * ldc + j0 + j;
              for (int jj = 0; jj < jb; jj++) crow[jj] += alpha * acc[ii * NR + jj];
            }
          }
        }
      }
      free(pb);
    }
  }
}

void lc_sgemv(int trans, int m, int n, float alpha, const float* A, int lda, const float* x, float beta, float* y) {
  if (!trans) {
    for (int i = 0; i < m; i++) {
      float s = 0.0f;
      for (int j = 0; j < n; j++) s += A[(size_t)i * lda + j] * x[j];
      y[i] = alpha * s + (beta == 0.0f ? 0.0f : beta * y[i]);
    }
  } else {
    for (int j = 0; j < n; j++) y[j] = beta == 0.0f ? 0.0f : beta * y[j];
    for (int i = 0; i < m; i++) {
      float xv = alpha * x[i];
      for (int j = 0; j < n; j++) y[j] += A[(size_t)i * lda + j] * xv;
    }
  }
}

/* ------------------------------------------------------------ dot family */
void lc_dot_vv(const float* x, const float* y, float* out, int n) { /* CPU:135-144 */
  float v = 0.0f;
  for (int i = 0; i < n; i++) v += x[i] * y[i];
  out[0] = v;
}
void lc_dot_mv(const float* A, const float* v, float* out, int m, int n) { /* CPU:146-156 */
  lc_sgemv(0, m, n, 1.0f, A, n, v, 0.0f, out);
}
void lc_dot_mm(const float* A, const float* B, float* out, int m, int k, int n) { /* CPU:158-169 */
  lc_sgemm(0, 0, m, n, k, 1.0f, A, k, B, n, 0.0f, out, n);
}
void lc_add_cartesian(float* xd, const float* y, const float* outd, int m, int n) { /* CPU:186-196 */
  for (int i = 0; i < m; i++)
    for (int j = 0; j < n; j++) xd[(size_t)i * n + j] = xd[(size_t)i * n + j] + y[j] * outd[i];
}
void lc_add_composition(float* xd, const float* Y, const float* outd, int m, int n) { /* CPU:198-206 */
  lc_sgemv(1, m, n, 1.0f, Y, n, outd, 1.0f, xd);
}
void lc_add_dottrans1(float* xd, const float* Y, const float* outd, int d1, int d2, int d3) { /* CPU:208-215 */
  lc_sgemm(1, 0, d2, d3, d1, 1.0f, Y, d2, outd, d3, 1.0f, xd, d3);
}
void lc_add_dottrans2(float* xd, const float* Y, const float* outd, int d1, int d2, int d3) { /* CPU:217-225 */
  lc_sgemm(0, 1, d1, d2, d3, 1.0f, Y, d3, outd, d3, 1.0f, xd, d2);
}
void lc_addmul_scalar(float* xd, const float* s, const float* y, long n) { /* TD addMul, CPU:174-175 */
  for (long i = 0; i < n; i++) xd[i] = xd[i] + s[0] * y[i];
}

/* ------------------------------------------------------------------ gemm */
/* d1,d2,d3 as the reference names them: result [d1,d3], contraction d2. */
void lc_gemm(int tx, int ty, int d1, int d2, int d3, float alpha, const float* x, const float* y, float* out) {
  lc_sgemm(tx, ty, d1, d3, d2, alpha, x, tx ? d1 : d2, y, ty ? d2 : d3, 0.0f, out, d3);
}
void lc_gemm_grad(int tx, int ty, int d1, int d2, int d3, float alpha, const float* x, float* xd, int x_is_input,
                  const float* y, float* yd, int y_is_input, const float* od) {
  /* CPU:428-472, case by case */
  if (!tx && !ty) {
    if (!x_is_input) lc_sgemm(0, 1, d1, d2, d3, alpha, od, d3, y, d3, 1.0f, xd, d2);
    if (!y_is_input) lc_sgemm(1, 0, d2, d3, d1, alpha, x, d2, od, d3, 1.0f, yd, d3);
  } else if (!tx && ty) {
    if (!x_is_input) lc_sgemm(0, 0, d1, d2, d3, alpha, od, d3, y, d2, 1.0f, xd, d2);
    if (!y_is_input) lc_sgemm(1, 0, d3, d2, d1, alpha, od, d3, x, d2, 1.0f, yd, d2);
  } else if (tx && !ty) {
    if (!x_is_input) lc_sgemm(0, 1, d2, d1, d3, alpha, y, d3, od, d3, 1.0f, xd, d1);
    if (!y_is_input) lc_sgemm(0, 0, d2, d3, d1, alpha, x, d1, od, d3, 1.0f, yd, d3);
  } else {
    if (!x_is_input) lc_sgemm(1, 1, d2, d1, d3, alpha, y, d2, od, d3, 1.0f, xd, d1);
    if (!y_is_input) lc_sgemm(1, 1, d3, d2, d1, alpha, od, d3, x, d1, 1.0f, yd, d2);
  }
}

/* ------------------------------------------------------------- broadcast */
static inline float bop(int op, float a, float b) {
  switch (op) { case LC_ADD: return a + b; case LC_SUB: return a - b; case LC_MUL: return a * b; default: return a / b; }
}
static void shadow_strides(const int* dims, int rank, long* st) { /* CPU:233-234: stride 0 where dim==1 */
  long s = 1;
  for (int i = rank - 1; i >= 0; i--) { st[i] = dims[i] == 1 ? 0 : s; s *= dims[i]; }
}
void lc_bcast_op(int op, const float* a, const int* adims, const float* b, const int* bdims, float* out, const int* odims, int rank) {
  long sa[8], sb[8]; int idx[8] = {0};
  shadow_strides(adims, rank, sa); shadow_strides(bdims, rank, sb);
  long total = 1; for (int i = 0; i < rank; i++) total *= odims[i];
  for (long r = 0; r < total; r++) {
    long ia = 0, ib = 0;
    for (int i = 0; i < rank; i++) { ia += sa[i] * idx[i]; ib += sb[i] * idx[i]; }
    out[r] = bop(op, a[ia], b[ib]);
    for (int i = rank - 1; i >= 0; i--) { if (++idx[i] < odims[i]) break; idx[i] = 0; }
  }
}
void lc_bcast_op_grad(int op, const float* a, float* ad, const int* adims, int a_in,
                      const float* b, float* bd, const int* bdims, int b_in,
                      const float* od, const int* odims, int rank) {
  /* CPU:246-263 with the op pairs of CPU:300-337 */
  long sa[8], sb[8]; int idx[8] = {0};
  shadow_strides(adims, rank, sa); shadow_strides(bdims, rank, sb);
  long total = 1; for (int i = 0; i < rank; i++) total *= odims[i];
  for (long r = 0; r < total; r++) {
    long ia = 0, ib = 0;
    for (int i = 0; i < rank; i++) { ia += sa[i] * idx[i]; ib += sb[i] * idx[i]; }
    float c = od[r], g1, g2;
    switch (op) {
      case LC_ADD: g1 = c; g2 = c; break;
      case LC_SUB: g1 = c; g2 = 0.0f - c; break;
      case LC_MUL: g1 = c * b[ib]; g2 = c * a[ia]; break;
      default:     g1 = c / b[ib]; g2 = -1.0f * a[ia] * c / (b[ib] * b[ib]); break;
    }
    if (!a_in) ad[ia] += g1;
    if (!b_in) bd[ib] += g2;
    for (int i = rank - 1; i >= 0; i--) { if (++idx[i] < odims[i]) break; idx[i] = 0; }
  }
}
void lc_bcast_update(int op, float* a, const int* adims, const float* b, const int* bdims, int rank) {
  /* CPU:265-279: x(idxX) = op(x(idxX), y(idxY)) over the broadcast result shape;
     a dimension of size 1 in `a` under a larger one in `b` reduces. */
  long sa[8], sb[8]; int idx[8] = {0}; int od[8];
  shadow_strides(adims, rank, sa); shadow_strides(bdims, rank, sb);
  long total = 1;
  for (int i = 0; i < rank; i++) { od[i] = adims[i] > bdims[i] ? adims[i] : bdims[i]; total *= od[i]; }
  for (long r = 0; r < total; r++) {
    long ia = 0, ib = 0;
    for (int i = 0; i < rank; i++) { ia += sa[i] * idx[i]; ib += sb[i] * idx[i]; }
    a[ia] = bop(op, a[ia], b[ib]);
    for (int i = rank - 1; i >= 0; i--) { if (++idx[i] < od[i]) break; idx[i] = 0; }
  }
}
void lc_scalar_op(int op, const float* x, float* y, float s, long n) { for (long i = 0; i < n; i++) y[i] = bop(op, x[i], s); }
void lc_geam(const float* x, float alpha, const float* y, float beta, float* out, long n) {
  for (long i = 0; i < n; i++) out[i] = x[i] * alpha + y[i] * beta;
}
void lc_trans(const float* x, float* y, int rows, int cols) {
  for (int i = 0; i < cols; i++) for (int j = 0; j < rows; j++) y[(size_t)i * rows + j] = x[(size_t)j * cols + i];
}
void lc_trans_grad(float* xd, const float* yd, int rows, int cols) {
  for (int i = 0; i < cols; i++) for (int j = 0; j < rows; j++) xd[(size_t)j * cols + i] += yd[(size_t)i * rows + j];
}
/* y.shape[i] = x.shape[perm[i]];  y[idx permuted] = x[idx]  (CUB:524-587 semantics; CPU has ???) */
static void permute_impl(const float* src, float* dst, const int* dims, const int* perm, int rank, int grad) {
  long sx[8], sy[8]; int ydims[8], idx[8] = {0};
  long s = 1; for (int i = rank - 1; i >= 0; i--) { sx[i] = s; s *= dims[i]; }
  for (int i = 0; i < rank; i++) ydims[i] = dims[perm[i]];
  s = 1; for (int i = rank - 1; i >= 0; i--) { sy[i] = s; s *= ydims[i]; }
  long total = s;
  for (long r = 0; r < total; r++) { /* idx iterates y's index space */
    long ix = 0; for (int i = 0; i < rank; i++) ix += sx[perm[i]] * idx[i];
    if (!grad) dst[r] = src[ix]; else dst[ix] += src[r];
    for (int i = rank - 1; i >= 0; i--) { if (++idx[i] < ydims[i]) break; idx[i] = 0; }
  }
  (void)sy;
}
void lc_permute(const float* x, float* y, const int* dims, const int* perm, int rank) { permute_impl(x, y, dims, perm, rank, 0); }
void lc_permute_grad(float* xd, const float* yd, const int* dims, const int* perm, int rank) { permute_impl(yd, xd, dims, perm, rank, 1); }

/* ------------------------------------------------------------------ conv */
/* CPU:484-530.  The reference offsets the kw block by outputWidth*outputWidth
 * (CPU:491), which equals outputHeight*outputWidth only for square outputs;
 * this follows the mathematical im2col (what unfoldedAcc CPU:652 uses). */
static void unfolded_copy(float* finput, const float* input, int kW, int kH, int dW, int dH, int padW, int padH,
                          int nIn, int iW, int iH, int oW, int oH) {
  for (int k = 0; k < nIn * kH * kW; k++) {
    int nip = k / (kH * kW), rest = k % (kH * kW), kh = rest / kW, kw = rest % kW;
    float* dst = finput + (size_t)nip * kH * kW * oH * oW + (size_t)kh * kW * oH * oW + (size_t)kw * oH * oW;
    const float* src = input + (size_t)nip * iH * iW;
    for (int y = 0; y < oH; y++) {
      int iy = y * dH - padH + kh;
      if (iy < 0 || iy >= iH) { memset(dst + (size_t)y * oW, 0, sizeof(float) * oW); continue; }
      for (int x = 0; x < oW; x++) {
        int ix = x * dW - padW + kw;
        dst[(size_t)y * oW + x] = (ix < 0 || ix >= iW) ? 0.0f : src[(size_t)iy * iW + ix];
      }
    }
  }
}
static void unfolded_acc(const float* finput, float* input, int kW, int kH, int dW, int dH, int padW, int padH,
                         int nIn, int iW, int iH, int oW, int oH) { /* CPU:647-692 */
  for (int nip = 0; nip < nIn; nip++)
    for (int kh = 0; kh < kH; kh++)
      for (int kw = 0; kw < kW; kw++) {
        const float* src = finput + (size_t)nip * kH * kW * oH * oW + (size_t)kh * kW * oH * oW + (size_t)kw * oH * oW;
        float* dst = input + (size_t)nip * iH * iW;
        for (int y = 0; y < oH; y++) {
          int iy = y * dH - padH + kh;
          if (iy < 0 || iy >= iH) continue;
          for (int x = 0; x < oW; x++) {
            int ix = x * dW - padW + kw;
            if (ix < 0 || ix >= iW) continue;
            dst[(size_t)iy * iW + ix] += src[(size_t)y * oW + x];
          }
        }
      }
}
void lc_conv2d_fwd(const float* x, const float* w, const float* bias, float* y, float* finput,
                   int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW) {
  /* CPU:532-571: output prefilled with bias (or zero), per-sample im2col, sgemm beta=1 */
  int oH = (H + 2 * pH - R) / sH + 1, oW = (W + 2 * pW - S) / sW + 1;
  size_t fsz = (size_t)C * R * S * oH * oW;
  int par = g_threads > 1 && N > 1;
  int save = g_threads;
  if (par) g_threads = 1; /* batch-parallel outside, serial sgemm inside */
#pragma omp parallel for schedule(dynamic) num_threads(save) if (par)
  for (int t = 0; t < N; t++) {
    float* yt = y + (size_t)t * K * oH * oW;
    float* ft = finput + (size_t)t * fsz;
    if (bias) lc_fill_with_bias(yt, bias, 1, K, (long)oH * oW); else memset(yt, 0, sizeof(float) * (size_t)K * oH * oW);
    unfolded_copy(ft, x + (size_t)t * C * H * W, S, R, sW, sH, pW, pH, C, W, H, oW, oH);
    lc_sgemm(0, 0, K, oH * oW, C * R * S, 1.0f, w, C * R * S, ft, oH * oW, 1.0f, yt, oH * oW);
  }
  g_threads = save;
}
void lc_conv2d_bwd(const float* finput, const float* w, const float* dy, float* dx, float* dw, float* db,
                   float* fgrad, int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW) {
  int oH = (H + 2 * pH - R) / sH + 1, oW = (W + 2 * pW - S) / sW + 1;
  int crs = C * R * S, pq = oH * oW;
  size_t fsz = (size_t)crs * pq;
  if (dx) { /* ConvGradInput CPU:622-645; dx NULL <=> input.isInput (CPU:584) */
    int par = g_threads > 1 && N > 1, save = g_threads;
    if (par) g_threads = 1;
#pragma omp parallel for schedule(dynamic) num_threads(save) if (par)
    for (int t = 0; t < N; t++) {
      float* fg = fgrad + (size_t)t * fsz;
      lc_sgemm(1, 0, crs, pq, K, 1.0f, w, crs, dy + (size_t)t * K * pq, pq, 0.0f, fg, pq);
      unfolded_acc(fg, dx + (size_t)t * C * H * W, S, R, sW, sH, pW, pH, C, W, H, oW, oH);
    }
    g_threads = save;
  }
  /* ConvGradParam CPU:589-620: sequential over the batch (accumulates into shared dw) */
  for (int t = 0; t < N; t++) {
    const float* dyt = dy + (size_t)t * K * pq;
    lc_sgemm(0, 1, K, crs, pq, 1.0f, dyt, pq, finput + (size_t)t * fsz, pq, 1.0f, dw, crs);
    if (db) {
      for (int i = 0; i < K; i++) {
        float sum = 0.0f;
        for (int k = 0; k < pq; k++) sum += dyt[(size_t)i * pq + k];
        db[i] += 1.0f * sum;
      }
    }
  }
}

/* ----------------------------------------------------------- activations */
void lc_unary(int op, const float* x, float* y, long n, float lo, float hi) {
  for (long i = 0; i < n; i++) {
    float v = x[i];
    switch (op) {
      case LC_RELU: y[i] = v < 0.0f ? 0.0f : v; break;                               /* CPU:711-720 */
      case LC_TANH: y[i] = (float)tanh((double)v); break;                           /* CPU:755 */
      case LC_SIGMOID: y[i] = 1.0f / ((float)exp((double)(-1.0f * v)) + 1.0f); break;/* CPU:760 */
      case LC_EXP: y[i] = (float)exp((double)v); break;                             /* CPU:771 */
      case LC_LOG: y[i] = (float)log((double)v); break;                             /* CPU:774 */
      case LC_SQRT: y[i] = (float)sqrt((double)v); break;                           /* CPU:777 */
      case LC_SQUARE: y[i] = v * v; break;                                          /* CPU:780 */
      default: y[i] = v < lo ? lo : (v > hi ? hi : v); break;                       /* CPU:733-742 */
    }
  }
}
/* inplace: x==y is the already-activated buffer and dx==dy.  The reference's
 * in-place relu_grad tests x<0 on the rectified buffer (CPU:725-726), which
 * never fires; the mask used here is y>0 (cuDNN's, CDN:1404-1405) -- the
 * mathematically right one.  hardTanh in-place likewise masks on the open
 * interval lo<y<hi. */
void lc_unary_grad(int op, const float* x, const float* y, const float* dy, float* dx, long n, int inplace, float lo, float hi) {
  for (long i = 0; i < n; i++) {
    switch (op) {
      case LC_RELU:
        if (inplace) { if (!(y[i] > 0.0f)) dx[i] = 0.0f; }
        else dx[i] += (x[i] < 0.0f ? 0.0f : dy[i]);                                  /* CPU:728 */
        break;
      case LC_TANH: dx[i] = dx[i] + (1.0f - y[i] * y[i]) * dy[i]; break;             /* TD:789-797 */
      case LC_SIGMOID: dx[i] = dx[i] + ((1.0f - y[i]) * y[i]) * dy[i]; break;        /* TD:799-809 */
      case LC_EXP: dx[i] += dy[i] * y[i]; break;                                     /* CPU:772 */
      case LC_LOG: dx[i] += dy[i] / x[i]; break;                                     /* CPU:775 */
      case LC_SQRT: dx[i] += dy[i] / y[i] / 2.0f; break;                             /* CPU:778 */
      case LC_SQUARE: dx[i] += dy[i] * x[i] * 2.0f; break;                           /* CPU:781 */
      default:
        if (inplace) { if (!(y[i] > lo && y[i] < hi)) dx[i] = 0.0f; }
        else dx[i] += ((x[i] < lo || x[i] > hi) ? 0.0f : dy[i]);                     /* CPU:750 */
        break;
    }
  }
}

/* -------------------------------------------------------- softmax / loss */
void lc_softmax(int is_log, const float* x, float* y, int rows, int cols) { lc_softmax3(is_log, x, y, rows, cols, 1); }
void lc_softmax_grad(int is_log, const float* y, const float* dy, float* dx, int rows, int cols) {
  lc_softmax3_grad(is_log, y, dy, dx, rows, cols, 1);
}
void lc_softmax3(int is_log, const float* x, float* y, int outer, int c, int inner) {
  /* CPU:784-832 per row: max (TD:555-573, init Float.MinValue = -FLT_MAX), exp in double narrowed,
     float row sum in index order (CPU:1125-1146), then divide / subtract log-sum. */
  for (int o = 0; o < outer; o++)
    for (int in = 0; in < inner; in++) {
      const float* xp = x + (size_t)o * c * inner + in;
      float* yp = y + (size_t)o * c * inner + in;
      float mx = -FLT_MAX;
      for (int j = 0; j < c; j++) if (xp[(size_t)j * inner] > mx) mx = xp[(size_t)j * inner];
      float sum = 0.0f;
      for (int j = 0; j < c; j++) { float e = (float)exp((double)(xp[(size_t)j * inner] - mx)); yp[(size_t)j * inner] = e; sum += e; }
      if (is_log) {
        float logsum = mx + (float)log((double)sum);
        for (int j = 0; j < c; j++) yp[(size_t)j * inner] = xp[(size_t)j * inner] - logsum;
      } else {
        for (int j = 0; j < c; j++) yp[(size_t)j * inner] = yp[(size_t)j * inner] / sum;
      }
    }
}
void lc_softmax3_grad(int is_log, const float* y, const float* dy, float* dx, int outer, int c, int inner) {
  for (int o = 0; o < outer; o++)
    for (int in = 0; in < inner; in++) {
      size_t base = (size_t)o * c * inner + in;
      if (is_log) { /* CPU:837-846 */
        float sum = 0.0f;
        for (int j = 0; j < c; j++) sum += dy[base + (size_t)j * inner];
        for (int j = 0; j < c; j++) {
          size_t i = base + (size_t)j * inner;
          dx[i] += dy[i] - (float)exp((double)y[i]) * sum;
        }
      } else { /* CPU ??? (835); cuDNN SOFTMAX_ACCURATE backward, beta=1: dx += y*(dy - sum(dy*y)) */
        float dot = 0.0f;
        for (int j = 0; j < c; j++) dot += dy[base + (size_t)j * inner] * y[base + (size_t)j * inner];
        for (int j = 0; j < c; j++) {
          size_t i = base + (size_t)j * inner;
          dx[i] += y[i] * (dy[i] - dot);
        }
      }
    }
}
void lc_nll(const float* x, const int* target, float* y, int batch, int stride) { /* CPU:1090-1101 */
  for (int b = 0; b < batch; b++) y[b] = -1.0f * x[(size_t)b * stride + target[b]];
}
void lc_nll_grad(float* dx, const int* target, const float* dy, int batch, int stride) { /* CPU:1103-1110 */
  for (int b = 0; b < batch; b++) dx[(size_t)b * stride + target[b]] += -1.0f * dy[b];
}

/* --------------------------------------------------------------- pooling */
/* CPU:848-948.  Scan order kernel rows then columns, strict '>' from -FLT_MAX
 * (first maximum wins).  The saved index is the global flat input index in
 * both branches: the reference's padded branch stores a per-sample index
 * (CPU:939), which its own scatter (CPU:955-957) then misplaces for n>0. */
void lc_maxpool_fwd(const float* x, float* y, int* idx, int N, int C, int H, int W, int kH, int kW, int sH, int sW, int pad) {
  int oH = (H + 2 * pad - kH) / sH + 1, oW = (W + 2 * pad - kW) / sW + 1;
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
  for (int nc = 0; nc < N * C; nc++) {
    const float* xp = x + (size_t)nc * H * W;
    for (int p = 0; p < oH; p++)
      for (int q = 0; q < oW; q++) {
        float best = -FLT_MAX; int bi = 0;
        for (int r = 0; r < kH; r++)
          for (int s = 0; s < kW; s++) {
            int h = p * sH - pad + r, w = q * sW - pad + s;
            if (h < 0 || h >= H || w < 0 || w >= W) continue;
            float v = xp[(size_t)h * W + w];
            if (v > best) { best = v; bi = (int)((size_t)nc * H * W + (size_t)h * W + w); }
          }
        size_t o = ((size_t)nc * oH + p) * oW + q;
        y[o] = best; idx[o] = bi;
      }
  }
}
void lc_maxpool_bwd(const float* dy, const int* idx, float* dx, long n_out) { /* CPU:950-959 */
  for (long i = 0; i < n_out; i++) dx[idx[i]] += dy[i];
}
void lc_avgpool_fwd(const float* x, float* y, int N, int C, int H, int W, int kH, int kW, int sH, int sW) { /* CPU:961-1006 */
  int oH = (H - kH) / sH + 1, oW = (W - kW) / sW + 1;
  float ks = kH * kW * 1.0f;
  for (int nc = 0; nc < N * C; nc++)
    for (int p = 0; p < oH; p++)
      for (int q = 0; q < oW; q++) {
        float sum = 0.0f;
        for (int r = 0; r < kH; r++)
          for (int s = 0; s < kW; s++) sum += x[(size_t)nc * H * W + (size_t)(p * sH + r) * W + q * sW + s];
        y[((size_t)nc * oH + p) * oW + q] = sum / ks;
      }
}
void lc_avgpool_bwd(const float* dy, float* dx, int N, int C, int H, int W, int kH, int kW, int sH, int sW) { /* CPU:1008-1038 */
  int oH = (H - kH) / sH + 1, oW = (W - kW) / sW + 1;
  int ks = kH * kW;
  for (int nc = 0; nc < N * C; nc++)
    for (int p = 0; p < oH; p++)
      for (int q = 0; q < oW; q++) {
        float d = dy[((size_t)nc * oH + p) * oW + q] / ks;
        for (int r = 0; r < kH; r++)
          for (int s = 0; s < kW; s++) dx[(size_t)nc * H * W + (size_t)(p * sH + r) * W + q * sW + s] += d;
      }
}

/* ------------------------------------------------------------ batch norm */
void lc_bn_infer(const float* x, const float* gamma, const float* beta, const float* rmean, const float* rvar,
                 float* y, int N, int C, int HW, float eps) { /* CPU:1040-1045 */
  for (int n = 0; n < N; n++)
    for (int c = 0; c < C; c++) {
      float den = (float)sqrt((double)(rvar[c] + eps));
      for (int l = 0; l < HW; l++) {
        size_t i = ((size_t)n * C + c) * HW + l;
        y[i] = (x[i] - rmean[c]) / den * gamma[c] + beta[c];
      }
    }
}
/* Forward value: CPU:1047-1056 (mean, biased variance of x-mean, (x-mean)/sqrt(var+eps)*gamma+beta).
 * Saved statistics and running-stat update: cuDNN spatial mode as called at
 * CDN:1025-1068 (save mean and 1/sqrt(var+eps); running = (1-f)*running + f*batch,
 * the variance entering the running average being the unbiased one).
 * Sums are carried in double so the oracle is a tight reference for any
 * summation order; the reference's float loop differs from it by rounding only. */
void lc_bn_train_fwd(const float* x, const float* gamma, const float* beta, float* rmean, float* rvar, float* y,
                     float* save_mean, float* save_invstd, int N, int C, int HW, float eps, float factor) {
  double cnt = (double)N * HW;
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
  for (int c = 0; c < C; c++) {
    double s = 0.0;
    for (int n = 0; n < N; n++) { const float* p = x + ((size_t)n * C + c) * HW; for (int l = 0; l < HW; l++) s += p[l]; }
    float mean = (float)(s / cnt);
    double v = 0.0;
    for (int n = 0; n < N; n++) { const float* p = x + ((size_t)n * C + c) * HW; for (int l = 0; l < HW; l++) { double d = (double)p[l] - mean; v += d * d; } }
    float var = (float)(v / cnt);
    float invstd = 1.0f / sqrtf(var + eps);
    for (int n = 0; n < N; n++) {
      const float* p = x + ((size_t)n * C + c) * HW; float* q = y + ((size_t)n * C + c) * HW;
      for (int l = 0; l < HW; l++) q[l] = (p[l] - mean) * invstd * gamma[c] + beta[c];
    }
    if (save_mean) save_mean[c] = mean;
    if (save_invstd) save_invstd[c] = invstd;
    if (rmean) rmean[c] = (1.0f - factor) * rmean[c] + factor * mean;
    if (rvar) { float unb = cnt > 1 ? (float)(v / (cnt - 1.0)) : var; rvar[c] = (1.0f - factor) * rvar[c] + factor * unb; }
  }
}
/* cudnnBatchNormalizationBackward with alpha=beta=1 for data and params (CDN:1101-1108):
 * dbeta += sum dy; dgamma += sum dy*xhat; dx += gamma*invstd*(dy - mean(dy) - xhat*mean(dy*xhat)). */
void lc_bn_bwd(const float* x, const float* dy, const float* gamma, const float* save_mean, const float* save_invstd,
               float* dx, float* dgamma, float* dbeta, int N, int C, int HW) {
  double cnt = (double)N * HW;
#pragma omp parallel for num_threads(g_threads) if (g_threads > 1)
  for (int c = 0; c < C; c++) {
    double s1 = 0.0, s2 = 0.0; float mean = save_mean[c], is = save_invstd[c];
    for (int n = 0; n < N; n++) {
      size_t b = ((size_t)n * C + c) * HW;
      for (int l = 0; l < HW; l++) { s1 += dy[b + l]; s2 += (double)dy[b + l] * ((x[b + l] - mean) * is); }
    }
    float m1 = (float)(s1 / cnt), m2 = (float)(s2 / cnt), g = gamma[c] * is;
    if (dx)
      for (int n = 0; n < N; n++) {
        size_t b = ((size_t)n * C + c) * HW;
        for (int l = 0; l < HW; l++) dx[b + l] += g * (dy[b + l] - m1 - (x[b + l] - mean) * is * m2);
      }
    if (dgamma) dgamma[c] += (float)s2;
    if (dbeta) dbeta[c] += (float)s1;
  }
}

/* --------------------------------------------------------------- dropout */
void lc_dropout_rand(const float* x, float* y, float* mask, long n, float p) { /* CPU:1066-1084 */
  float scale = 1.0f / (1.0f - p);
  for (long i = 0; i < n; i++) {
    if (ref_rand() > p) { y[i] = x[i] * scale; mask[i] = scale; } else { y[i] = 0.0f; mask[i] = 0.0f; }
  }
}
/* Counter-based uniform in [0,1): splitmix64 of (seed, index), top 24 bits.
 * The device draws the mask the same way, so masks compare bit for bit. */
float lc_ctr_uniform(uint64_t seed, uint64_t index) {
  uint64_t z = seed + 0x9E3779B97F4A7C15ULL * (index + 1);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
  z = z ^ (z >> 31);
  return (float)(z >> 40) * (1.0f / 16777216.0f);
}
void lc_dropout_ctr(const float* x, float* y, float* mask, long n, float p, uint64_t seed, uint64_t offset) {
  float scale = 1.0f / (1.0f - p);
  for (long i = 0; i < n; i++) {
    if (lc_ctr_uniform(seed, offset + (uint64_t)i) > p) { y[i] = x[i] * scale; mask[i] = scale; } else { y[i] = 0.0f; mask[i] = 0.0f; }
  }
}
void lc_dropout_bwd(const float* dy, const float* mask, float* dx, long n) { /* CPU:1086-1088 */
  for (long i = 0; i < n; i++) dx[i] += mask[i] * dy[i];
}

/* ------------------------------------------------------------ reductions */
void lc_sum_all(const float* x, float* out, long n) { float r = 0.0f; for (long i = 0; i < n; i++) r = r + x[i]; out[0] = r; }
void lc_mean_all(const float* x, float* out, long n) { lc_sum_all(x, out, n); out[0] = out[0] / n; }
void lc_add_scalar_from(float* dx, const float* dy1, float scale, long n) {
  /* sum_grad: dx += dy (broadcast) CPU:1118; mean_grad: dx += dy/n CPU:1122-1124 (scale = 1/n) */
  for (long i = 0; i < n; i++) dx[i] += dy1[0] * scale;
}
void lc_sum_dim(const float* x, float* y, int outer, int dim, int inner) { /* CPU:1125-1146; y must be zero */
  for (int h = 0; h < outer; h++)
    for (int s = 0; s < dim; s++)
      for (int l = 0; l < inner; l++) y[(size_t)h * inner + l] += x[((size_t)h * dim + s) * inner + l];
}
void lc_sum_dim_grad(float* dx, const float* dy, int outer, int dim, int inner) { /* CPU:1147-1164 */
  for (int h = 0; h < outer; h++)
    for (int s = 0; s < dim; s++)
      for (int l = 0; l < inner; l++) dx[((size_t)h * dim + s) * inner + l] += dy[(size_t)h * inner + l];
}

/* ---------------------------------------------------------------- concat */
/* sizes[t] = size of tensor t along the concat dim; stride of tensor t = sizes[t]*inner */
void lc_concat(int n, const float* const* in, const int* sizes, float* out, int outer, int inner) {
  size_t tgt = 0;
  for (int h = 0; h < outer; h++)
    for (int t = 0; t < n; t++) {
      size_t st = (size_t)sizes[t] * inner; const float* p = in[t] + (size_t)h * st;
      for (size_t l = 0; l < st; l++) out[tgt++] = p[l];
    }
}
void lc_concat_grad(int n, float* const* ind, const int* sizes, const float* outd, int outer, int inner) {
  size_t tgt = 0;
  for (int h = 0; h < outer; h++)
    for (int t = 0; t < n; t++) {
      size_t st = (size_t)sizes[t] * inner; float* p = ind[t] + (size_t)h * st;
      for (size_t l = 0; l < st; l++) p[l] += outd[tgt++];
    }
}
void lc_mask4d(float* x, const int* lengths, int n, int c, int d, int t) {
  for (int i = 0; i < n; i++) for (int j = 0; j < c; j++) for (int k = 0; k < d; k++) for (int u = 0; u < t; u++)
    if (u >= lengths[i]) x[(((size_t)i * c + j) * d + k) * t + u] = 0;
}

/* ------------------------------------------------------------ optimizers */
void lc_sgd(float* x, float* d, float lr, long n) { /* NN:265-287: geam(x,1,d,-lr) then clear_grad */
  for (long i = 0; i < n; i++) { x[i] = x[i] * 1.0f + d[i] * (-lr); d[i] = 0.0f; }
}
void lc_momentum(float* x, float* d, float* v, float lr, float mu, float clip, int nesterov, long n) { /* CPU:1232-1246 */
  for (long i = 0; i < n; i++) {
    float t = d[i];
    if (t > clip) t = clip;
    if (t < -clip) t = -clip;
    v[i] *= mu; v[i] += t;
    if (nesterov) t += mu * v[i]; else t = v[i];
    x[i] -= lr * t;
    d[i] = 0.0f;
  }
}
void lc_adagrad(float* x, float* d, float* m, float lr, float clip, long n) { /* CPU:1217-1230 */
  for (long i = 0; i < n; i++) {
    float t = d[i];
    if (t > clip) t = clip;
    if (t < -clip) t = -clip;
    m[i] += t * t;
    x[i] -= lr * t / (float)sqrt((double)(m[i] + 1e-8f));
    d[i] = 0.0f;
  }
}

/* ------------------------------------------------------------------- CTC */
/* parity unpinned against the reference (its tests only print).  Standard CTC
 * (Graves 2006) on softmax-ed probabilities probs[T,B,A], blank = 0, as
 * cudnnCTCLoss (deterministic) is called at CDN:1895-1938: costs[b] =
 * -log p(labels_b | probs), and the gradient written is with respect to the
 * *pre-softmax activations* (cuDNN's documented output): dact = probs -
 * (1/p(l|x)) * sum_{s: l'_s = k} alpha*beta.  Accumulated into dprobs unscaled:
 * the reference lets cuDNN write this gradient into probs.d during the forward
 * call and only averages the reported costs (CDN:1930-1937), so training
 * follows the gradient of the SUM of the per-sample costs. */
void lc_ctc_loss(const float* probs, float* dprobs, const int* labels, const int* label_len, const int* input_len,
                 float* costs, int T, int B, int A) {
  int loff = 0;
  for (int b = 0; b < B; b++) {
    int L = label_len[b], Tb = input_len[b], S = 2 * L + 1;
    const int* lab = labels + loff; loff += L;
    double* alpha = (double*)calloc((size_t)Tb * S, sizeof(double));
    double* beta = (double*)calloc((size_t)Tb * S, sizeof(double));
    #define LP(t, s) ((double)probs[((size_t)(t) * B + b) * A + (((s) & 1) ? lab[(s) >> 1] : 0)])
    /* scaled forward-backward with per-step normalisation */
    double* cn = (double*)calloc(Tb, sizeof(double));
    double ll = 0.0;
    alpha[0] = LP(0, 0); if (S > 1) alpha[1] = LP(0, 1);
    for (int t = 0; t < Tb; t++) {
      if (t > 0)
        for (int s = 0; s < S; s++) {
          double a = alpha[(size_t)(t - 1) * S + s];
          if (s >= 1) a += alpha[(size_t)(t - 1) * S + s - 1];
          if (s >= 2 && (s & 1) && lab[s >> 1] != lab[(s >> 1) - 1]) a += alpha[(size_t)(t - 1) * S + s - 2];
          alpha[(size_t)t * S + s] = a * LP(t, s);
        }
      double c = 0.0; for (int s = 0; s < S; s++) c += alpha[(size_t)t * S + s];
      cn[t] = c; if (c > 0) for (int s = 0; s < S; s++) alpha[(size_t)t * S + s] /= c;
      ll += log(c);
    }
    /* true log-likelihood needs only the last two states; recompute with beta */
    beta[(size_t)(Tb - 1) * S + S - 1] = 1.0; if (S > 1) beta[(size_t)(Tb - 1) * S + S - 2] = 1.0;
    for (int t = Tb - 2; t >= 0; t--) {
      for (int s = 0; s < S; s++) {
        double v = beta[(size_t)(t + 1) * S + s] * LP(t + 1, s);
        if (s + 1 < S) v += beta[(size_t)(t + 1) * S + s + 1] * LP(t + 1, s + 1);
        if (s + 2 < S && ((s + 2) & 1) && lab[(s + 2) >> 1] != lab[s >> 1]) v += beta[(size_t)(t + 1) * S + s + 2] * LP(t + 1, s + 2);
        beta[(size_t)t * S + s] = v / cn[t + 1];
      }
    }
    /* p(l|x)/prod(cn) = sum over final states of scaled alpha at T-1 */
    double pfin = alpha[(size_t)(Tb - 1) * S + S - 1] + (S > 1 ? alpha[(size_t)(Tb - 1) * S + S - 2] : 0.0);
    costs[b] = (float)(-(ll + log(pfin)));
    if (dprobs) {
      for (int t = 0; t < Tb; t++) {
        double* acc = (double*)calloc(A, sizeof(double));
        for (int s = 0; s < S; s++) acc[(s & 1) ? lab[s >> 1] : 0] += alpha[(size_t)t * S + s] * beta[(size_t)t * S + s];
        for (int k = 0; k < A; k++) {
          size_t i = ((size_t)t * B + b) * A + k;
          double post = acc[k] / pfin; /* alpha,beta scaled: sum_s alpha_t(s)beta_t(s)/pfin = posterior */
          dprobs[i] += (float)(probs[i] - post);
        }
        free(acc);
      }
    }
    #undef LP
    free(alpha); free(beta); free(cn);
  }
}

/* ------------------------------------------------------------------- RNN */
/* parity unpinned against the reference (no CPU implementation, CPU:??? ; the
 * GPU path is cudnnRNNForwardTraining / BackwardData / BackwardWeights at
 * CDN:1638-1893).  One layer of an Elman RNN, optionally bidirectional:
 *   h_t = act(W_ih x_t + b_ih + W_hh h_{t-1} + b_hh),  h_{-1} = 0,
 * act = tanh (mode 1) or relu (mode 0); y[t,b,:] = [h_t forward ; h_t reverse],
 * the reverse direction running t = T-1 .. 0.  Packed weights per direction in
 * the order of NN:378-390: W_ih[H,I], W_hh[H,H], b_ih[H], b_hh[H]; forward
 * direction first.  Checked against torch.nn.RNN in the tests. */
static size_t rnn_dir_params(int I, int H) { return (size_t)H * I + (size_t)H * H + 2 * (size_t)H; }

/* hx (may be NULL = zeros): initial hidden state [D, B, H], the `hx` of RNNBase.apply (NN:392) as cudnnRNNForwardTraining takes
 * it (CDN:1796); it receives no gradient (dhx is NULL at CDN:1843-1844). */
void lc_rnn_fwd_init(int mode, const float* x, const float* hx, const float* w, float* y, int T, int B, int I, int H, int bidir) {
  const int D = bidir ? 2 : 1, DH = D * H;
  float* pre = (float*)malloc((size_t)T * B * H * sizeof(float));
  float* hprev = (float*)calloc((size_t)B * H, sizeof(float));
  float* rec = (float*)malloc((size_t)B * H * sizeof(float));
  for (int d = 0; d < D; d++) {
    const float* Wih = w + d * rnn_dir_params(I, H); const float* Whh = Wih + (size_t)H * I;
    const float* bih = Whh + (size_t)H * H; const float* bhh = bih + H;
    /* input projection for all steps: pre[T*B, H] = x[T*B, I] * Wih^T */
    lc_sgemm(0, 1, T * B, H, I, 1.0f, x, I, Wih, I, 0.0f, pre, H);
    if (hx) memcpy(hprev, hx + (size_t)d * B * H, (size_t)B * H * sizeof(float));
    else memset(hprev, 0, (size_t)B * H * sizeof(float));
    for (int step = 0; step < T; step++) {
      const int t = d == 0 ? step : T - 1 - step;
      lc_sgemm(0, 1, B, H, H, 1.0f, hprev, H, Whh, H, 0.0f, rec, H);
      for (int b = 0; b < B; b++)
        for (int j = 0; j < H; j++) {
          float v = pre[((size_t)t * B + b) * H + j] + bih[j] + rec[(size_t)b * H + j] + bhh[j];
          v = mode == 1 ? (float)tanh((double)v) : (v < 0.f ? 0.f : v);
          y[((size_t)t * B + b) * DH + d * H + j] = v; hprev[(size_t)b * H + j] = v;
        }
    }
  }
  free(pre); free(hprev); free(rec);
}
void lc_rnn_fwd(int mode, const float* x, const float* w, float* y, int T, int B, int I, int H, int bidir) {
  lc_rnn_fwd_init(mode, x, NULL, w, y, T, B, I, H, bidir);
}

/* dx (may be NULL) and dw accumulate. */
void lc_rnn_bwd_init(int mode, const float* x, const float* hx, const float* y, const float* dy, const float* w, float* dx, float* dw,
                     int T, int B, int I, int H, int bidir) {
  const int D = bidir ? 2 : 1, DH = D * H;
  float* dpre = (float*)malloc((size_t)T * B * H * sizeof(float));
  float* hs = (float*)malloc((size_t)T * B * H * sizeof(float));      /* h_{t-1} for every step, in time order */
  float* dh = (float*)malloc((size_t)B * H * sizeof(float));
  for (int d = 0; d < D; d++) {
    const size_t off = d * rnn_dir_params(I, H);
    const float* Wih = w + off; const float* Whh = Wih + (size_t)H * I;
    float* dWih = dw + off; float* dWhh = dWih + (size_t)H * I; float* dbih = dWhh + (size_t)H * H; float* dbhh = dbih + H;
    memset(dh, 0, (size_t)B * H * sizeof(float));
    for (int step = T - 1; step >= 0; step--) {
      const int t = d == 0 ? step : T - 1 - step;
      const int tp = d == 0 ? t - 1 : t + 1;                              /* time index of the previous hidden state */
      for (int b = 0; b < B; b++)
        for (int j = 0; j < H; j++) {
          const float h = y[((size_t)t * B + b) * DH + d * H + j];
          const float g = dy[((size_t)t * B + b) * DH + d * H + j] + dh[(size_t)b * H + j];
          dpre[((size_t)t * B + b) * H + j] = mode == 1 ? g * (1.0f - h * h) : (h > 0.f ? g : 0.f);
          hs[((size_t)t * B + b) * H + j] = step == 0 ? (hx ? hx[((size_t)d * B + b) * H + j] : 0.f) : y[((size_t)tp * B + b) * DH + d * H + j];
        }
      /* dh_{prev}[B,H] = dpre_t[B,H] * Whh[H,H] */
      lc_sgemm(0, 0, B, H, H, 1.0f, dpre + (size_t)t * B * H, H, Whh, H, 0.0f, dh, H);
    }
    /* dWih[H,I] += dpre^T x ; dWhh[H,H] += dpre^T hs ; biases += column sums ; dx += dpre Wih */
    lc_sgemm(1, 0, H, I, T * B, 1.0f, dpre, H, x, I, 1.0f, dWih, I);
    lc_sgemm(1, 0, H, H, T * B, 1.0f, dpre, H, hs, H, 1.0f, dWhh, H);
    for (int j = 0; j < H; j++) {
      double s = 0.0; for (size_t r = 0; r < (size_t)T * B; r++) s += dpre[r * H + j];
      dbih[j] += (float)s; dbhh[j] += (float)s;
    }
    if (dx) lc_sgemm(0, 0, T * B, I, H, 1.0f, dpre, H, Wih, I, 1.0f, dx, I);
  }
  free(dpre); free(hs); free(dh);
}
void lc_rnn_bwd(int mode, const float* x, const float* y, const float* dy, const float* w, float* dx, float* dw,
                int T, int B, int I, int H, int bidir) {
  lc_rnn_bwd_init(mode, x, NULL, y, dy, w, dx, dw, T, B, I, H, bidir);
}

/* ---------------------------------------------------------- LSTM and GRU
 * parity unpinned against the reference (no CPU implementation and no asserted vector; the GPU path is the same cuDNN
 * calls as above with CUDNN_LSTM / CUDNN_GRU, NN:324-330).  cuDNN's documented formulas, gates in its order:
 *   LSTM: i, f, o = sigmoid, g = tanh of (W x + b_i + R h + b_h), order i f g o;  c' = f c + i g;  h' = o tanh(c')
 *   GRU:  r, z = sigmoid(W x + b_i + R h + b_h);  n = tanh(W_n x + b_in + r (R_n h + b_hn));  h' = (1 - z) n + z h
 * Packed weights per direction as NN:378-390 with G = 4H / 3H rows.  Written per sample and per step with double
 * accumulation; the backward pass keeps no state from the forward one (it recomputes it) and adds each step's outer
 * products into dw as it goes.  Checked against torch.nn.LSTM / torch.nn.GRU (CPU) in the tests. */
static int gated_ng(int mode) { return mode == 2 ? 4 : 3; }
static size_t gated_dir_params(int mode, int I, int H) { size_t G = (size_t)gated_ng(mode) * H; return G * I + G * H + 2 * G; }
static double sigm_d(double v) { return 1.0 / (1.0 + exp(-v)); }

/* One direction of one sample, forward; fills (when not NULL) per-step records for the backward pass:
 * gate[T][G] activations, cell[T][H] (LSTM: c_t; GRU: q_t = R_n h + b_hn), hid[T][H] = h_t. */
static void gated_forward_sample(int mode, const float* x, size_t xs, const float* Wih, const float* Whh, const float* bih, const float* bhh,
                                 int T, int I, int H, int reverse, double* gate, double* cell, double* hid, const float* h0, const float* c0) {
  const int ng = gated_ng(mode), G = ng * H;
  double* h = (double*)calloc((size_t)H, sizeof(double));
  double* c = (double*)calloc((size_t)H, sizeof(double));
  for (int j = 0; j < H; j++) { if (h0) h[j] = h0[j]; if (c0) c[j] = c0[j]; }    /* initial state of this sample and direction */
  double* px = (double*)malloc((size_t)G * sizeof(double));
  double* ph = (double*)malloc((size_t)G * sizeof(double));
  for (int step = 0; step < T; step++) {
    const int t = reverse ? T - 1 - step : step;
    const float* xt = x + (size_t)t * xs;
    for (int g = 0; g < G; g++) {
      double a = 0.0, r = 0.0;
      for (int k = 0; k < I; k++) a += (double)Wih[(size_t)g * I + k] * xt[k];
      for (int k = 0; k < H; k++) r += (double)Whh[(size_t)g * H + k] * h[k];
      px[g] = a + bih[g]; ph[g] = r + bhh[g];
    }
    double* gt = gate + (size_t)t * G;
    for (int j = 0; j < H; j++) {
      if (mode == 2) {
        const double ig = sigm_d(px[j] + ph[j]), fg = sigm_d(px[H + j] + ph[H + j]);
        const double gg = tanh(px[2 * H + j] + ph[2 * H + j]), og = sigm_d(px[3 * H + j] + ph[3 * H + j]);
        c[j] = fg * c[j] + ig * gg;
        gt[j] = ig; gt[H + j] = fg; gt[2 * H + j] = gg; gt[3 * H + j] = og;
        cell[(size_t)t * H + j] = c[j];
        hid[(size_t)t * H + j] = og * tanh(c[j]);
      } else {
        const double r = sigm_d(px[j] + ph[j]), z = sigm_d(px[H + j] + ph[H + j]);
        const double n = tanh(px[2 * H + j] + r * ph[2 * H + j]);
        gt[j] = r; gt[H + j] = z; gt[2 * H + j] = n;
        cell[(size_t)t * H + j] = ph[2 * H + j];
        hid[(size_t)t * H + j] = (1.0 - z) * n + z * h[j];
      }
    }
    for (int j = 0; j < H; j++) h[j] = hid[(size_t)t * H + j];
  }
  free(h); free(c); free(px); free(ph);
}

/* hx, cx (each may be NULL = zeros): initial hidden and cell state [D, B, H] (cx: LSTM only); no gradient flows to them. */
void lc_rnn_gated_fwd_init(int mode, const float* x, const float* hx, const float* cx, const float* w, float* y, int T, int B, int I, int H, int bidir) {
  const int D = bidir ? 2 : 1, G = gated_ng(mode) * H;
  double* gate = (double*)malloc((size_t)T * G * sizeof(double));
  double* cell = (double*)malloc((size_t)T * H * sizeof(double));
  double* hid = (double*)malloc((size_t)T * H * sizeof(double));
  for (int d = 0; d < D; d++) {
    const float* Wih = w + d * gated_dir_params(mode, I, H); const float* Whh = Wih + (size_t)G * I;
    const float* bih = Whh + (size_t)G * H; const float* bhh = bih + G;
    for (int b = 0; b < B; b++) {
      gated_forward_sample(mode, x + (size_t)b * I, (size_t)B * I, Wih, Whh, bih, bhh, T, I, H, d, gate, cell, hid,
                           hx ? hx + ((size_t)d * B + b) * H : NULL, cx ? cx + ((size_t)d * B + b) * H : NULL);
      for (int t = 0; t < T; t++)
        for (int j = 0; j < H; j++) y[((size_t)t * B + b) * D * H + (size_t)d * H + j] = (float)hid[(size_t)t * H + j];
    }
  }
  free(gate); free(cell); free(hid);
}
void lc_rnn_gated_fwd(int mode, const float* x, const float* w, float* y, int T, int B, int I, int H, int bidir) {
  lc_rnn_gated_fwd_init(mode, x, NULL, NULL, w, y, T, B, I, H, bidir);
}

/* dx (may be NULL) and dw accumulate. */
void lc_rnn_gated_bwd_init(int mode, const float* x, const float* hx, const float* cx, const float* dy, const float* w, float* dx, float* dw,
                           int T, int B, int I, int H, int bidir) {
  const int D = bidir ? 2 : 1, ng = gated_ng(mode), G = ng * H;
  double* gate = (double*)malloc((size_t)T * G * sizeof(double));
  double* cell = (double*)malloc((size_t)T * H * sizeof(double));
  double* hid = (double*)malloc((size_t)T * H * sizeof(double));
  double* dh = (double*)malloc((size_t)H * sizeof(double));
  double* dc = (double*)malloc((size_t)H * sizeof(double));
  double* gx = (double*)malloc((size_t)G * sizeof(double));       /* gradient of the input-side pre-activations */
  double* gh = (double*)malloc((size_t)G * sizeof(double));       /* ... of the hidden-side ones */
  double* h0d = (double*)malloc((size_t)H * sizeof(double));      /* the initial hidden state of the current sample */
  const size_t np = gated_dir_params(mode, I, H);
  double* acc = (double*)calloc(np, sizeof(double));
  for (int d = 0; d < D; d++) {
    const size_t off = d * np;
    const float* Wih = w + off; const float* Whh = Wih + (size_t)G * I; const float* bih = Whh + (size_t)G * H; const float* bhh = bih + G;
    double* aWih = acc; double* aWhh = aWih + (size_t)G * I; double* abih = aWhh + (size_t)G * H; double* abhh = abih + G;
    memset(acc, 0, np * sizeof(double));
    for (int b = 0; b < B; b++) {
      const float* h0 = hx ? hx + ((size_t)d * B + b) * H : NULL;
      const float* c0 = cx ? cx + ((size_t)d * B + b) * H : NULL;
      gated_forward_sample(mode, x + (size_t)b * I, (size_t)B * I, Wih, Whh, bih, bhh, T, I, H, d, gate, cell, hid, h0, c0);
      for (int j = 0; j < H; j++) dh[j] = dc[j] = 0.0;
      for (int step = T - 1; step >= 0; step--) {
        const int t = d ? T - 1 - step : step;
        const int tp = d ? t + 1 : t - 1;
        const double* gt = gate + (size_t)t * G;
        const double* hp = step == 0 ? NULL : hid + (size_t)tp * H;
        if (step == 0 && h0) { for (int j = 0; j < H; j++) h0d[j] = h0[j]; hp = h0d; }
        for (int j = 0; j < H; j++) {
          const double g = dh[j] + dy[((size_t)t * B + b) * D * H + (size_t)d * H + j];
          if (mode == 2) {
            const double ig = gt[j], fg = gt[H + j], gg = gt[2 * H + j], og = gt[3 * H + j];
            const double tc = tanh(cell[(size_t)t * H + j]);
            const double cp = step == 0 ? (c0 ? (double)c0[j] : 0.0) : cell[(size_t)tp * H + j];
            const double dcell = dc[j] + g * og * (1.0 - tc * tc);
            gx[j] = dcell * gg * ig * (1.0 - ig);
            gx[H + j] = dcell * cp * fg * (1.0 - fg);
            gx[2 * H + j] = dcell * ig * (1.0 - gg * gg);
            gx[3 * H + j] = g * tc * og * (1.0 - og);
            gh[j] = gx[j]; gh[H + j] = gx[H + j]; gh[2 * H + j] = gx[2 * H + j]; gh[3 * H + j] = gx[3 * H + j];
            dc[j] = dcell * fg;
            dh[j] = 0.0;
          } else {
            const double r = gt[j], z = gt[H + j], n = gt[2 * H + j], q = cell[(size_t)t * H + j];
            const double hprev = hp ? hp[j] : 0.0;
            const double dn = g * (1.0 - z) * (1.0 - n * n);
            gx[j] = dn * q * r * (1.0 - r);
            gx[H + j] = g * (hprev - n) * z * (1.0 - z);
            gx[2 * H + j] = dn;
            gh[j] = gx[j]; gh[H + j] = gx[H + j]; gh[2 * H + j] = dn * r;
            dh[j] = g * z;
          }
        }
        const float* xt = x + ((size_t)t * B + b) * I;
        for (int g = 0; g < G; g++) {
          for (int k = 0; k < I; k++) aWih[(size_t)g * I + k] += gx[g] * xt[k];
          if (hp) for (int k = 0; k < H; k++) aWhh[(size_t)g * H + k] += gh[g] * hp[k];
          abih[g] += gx[g]; abhh[g] += gh[g];
        }
        for (int k = 0; k < H; k++) { double s = 0.0; for (int g = 0; g < G; g++) s += gh[g] * Whh[(size_t)g * H + k]; dh[k] += s; }
        if (dx) for (int k = 0; k < I; k++) {
          double s = 0.0; for (int g = 0; g < G; g++) s += gx[g] * Wih[(size_t)g * I + k];
          dx[((size_t)t * B + b) * I + k] += (float)s;
        }
      }
    }
    for (size_t i = 0; i < np; i++) dw[off + i] += (float)acc[i];
  }
  free(gate); free(cell); free(hid); free(dh); free(dc); free(gx); free(gh); free(acc); free(h0d);
}
void lc_rnn_gated_bwd(int mode, const float* x, const float* dy, const float* w, float* dx, float* dw, int T, int B, int I, int H, int bidir) {
  lc_rnn_gated_bwd_init(mode, x, NULL, NULL, dy, w, dx, dw, T, B, I, H, bidir);
}

/* ------------------------------------------ average pooling with padding
 * parity unpinned against the reference (CPU:1003-1005 and 1035-1037 are ???; the GPU path is cudnnPoolingForward /
 * Backward with CUDNN_POOLING_AVERAGE_COUNT_EXCLUDE_PADDING, CDN:975-982): each output is the mean of the window's
 * elements that lie inside the image.  The backward pass scatters from the outputs.  Checked against
 * torch.nn.functional.avg_pool2d(count_include_pad=False) forward and autograd in the tests. */
void lc_avgpool_pad_fwd(const float* x, float* y, int N, int C, int H, int W, int kH, int kW, int sH, int sW, int pH, int pW) {
  const int oH = (H + 2 * pH - kH) / sH + 1, oW = (W + 2 * pW - kW) / sW + 1;
  for (long nc = 0; nc < (long)N * C; nc++)
    for (int oh = 0; oh < oH; oh++)
      for (int ow = 0; ow < oW; ow++) {
        float sum = 0.0f; int cnt = 0;
        for (int r = 0; r < kH; r++)
          for (int q = 0; q < kW; q++) {
            const int h = oh * sH - pH + r, w = ow * sW - pW + q;
            if (h >= 0 && h < H && w >= 0 && w < W) { sum += x[(nc * H + h) * W + w]; cnt++; }
          }
        y[(nc * oH + oh) * oW + ow] = cnt ? sum / (float)cnt : 0.0f;
      }
}
void lc_avgpool_pad_bwd(const float* dy, float* dx, int N, int C, int H, int W, int kH, int kW, int sH, int sW, int pH, int pW) {
  const int oH = (H + 2 * pH - kH) / sH + 1, oW = (W + 2 * pW - kW) / sW + 1;
  for (long nc = 0; nc < (long)N * C; nc++)
    for (int oh = 0; oh < oH; oh++)
      for (int ow = 0; ow < oW; ow++) {
        int cnt = 0;
        for (int r = 0; r < kH; r++)
          for (int q = 0; q < kW; q++) {
            const int h = oh * sH - pH + r, w = ow * sW - pW + q;
            if (h >= 0 && h < H && w >= 0 && w < W) cnt++;
          }
        if (!cnt) continue;
        const float g = dy[(nc * oH + oh) * oW + ow] / (float)cnt;
        for (int r = 0; r < kH; r++)
          for (int q = 0; q < kW; q++) {
            const int h = oh * sH - pH + r, w = ow * sW - pW + q;
            if (h >= 0 && h < H && w >= 0 && w < W) dx[(nc * H + h) * W + w] += g;
          }
      }
}

/* ------------------------------------------------------------- repeat0
 * TD:1446-1451; the reference's CPU backend has ??? (CPU:1214-1215), its GPU backend the repeat0 / shift0 kernels
 * (API:625-650, CDN:378-399): out[i0][i1][:] = in[i0 + i1][:].  The gradient scatters every window back, all rows
 * included.  Pinned by what the definition fixes: against numpy's sliding windows and a finite-difference-free identity
 * (the gradient of sum(out * g) with respect to in is the scatter of g) in the tests. */
void lc_repeat0(const float* in, float* out, int rows, int context, long inner) {
  for (long i0 = 0; i0 < rows - context; i0++)
    for (long i1 = 0; i1 <= context; i1++)
      memcpy(out + (i0 * (context + 1) + i1) * inner, in + (i0 + i1) * inner, (size_t)inner * sizeof(float));
}
void lc_repeat0_grad(float* ind, const float* outd, int rows, int context, long inner) {
  for (long i0 = 0; i0 < rows - context; i0++)
    for (long i1 = 0; i1 <= context; i1++)
      for (long j = 0; j < inner; j++) ind[(i0 + i1) * inner + j] += outd[(i0 * (context + 1) + i1) * inner + j];
}
