/* A host program in plain C99 that drives liblantern_hip.so the way the reference's emitted programs drive their
 * backend: straight-line calls over a bump-pointer arena, one mark taken after the parameters and a rewind at the end
 * of every step (src/out/NIPS18evaluation/evaluationCNN/Lantern/Lantern.cpp: the training loop of the MNIST CNN;
 * network from src/main/scala/lantern/NIPS18App/MnistCNN.scala:38-59 without the dropout, so that both sides are
 * deterministic).  It includes only the public header, links no Python and no torch, and runs the same five SGD steps
 * through the CPU oracle in the same process; it exits non-zero when a loss differs by more than 1e-4 relative or a
 * parameter by more than 1e-3 of the largest parameter.
 *
 * Build:  gcc -std=c99 -O1 -Wall -Werror -I include -I oracle tests/host_c/lenet_step.c \
 *             -L lantern_amd/csrc -llantern_hip -L oracle -llantern_cpu -lm -o tests/host_c/_build/lenet_step
 * With LENET_STEP_LINK_ONLY defined at run time (environment) the program returns before touching the device: the
 * link check for machines without one.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "lantern_hip.h"
#include "lantern_cpu.h"

enum { B = 32, STEPS = 5 };
#define LR 0.002f   /* the loss is a sum over the batch */

/* shapes */
enum {
  X_N = B * 1 * 28 * 28,
  W1_N = 10 * 1 * 5 * 5, C1_N = B * 10 * 24 * 24, P1_N = B * 10 * 12 * 12,
  W2_N = 20 * 10 * 5 * 5, C2_N = B * 20 * 8 * 8, P2_N = B * 320,
  L1_N = 320 * 50, H1_N = B * 50, L2_N = 50 * 10, Z_N = B * 10,
  N_PARAMS = 8
};
static const int64_t kParamSize[N_PARAMS] = { W1_N, 10, W2_N, 20, L1_N, 50, L2_N, 10 };

static uint32_t g_lcg = 12345u;
static float frand(void) {                       /* uniform in [-0.5, 0.5) */
  g_lcg = g_lcg * 1664525u + 1013904223u;
  return (float)(g_lcg >> 8) / 16777216.0f - 0.5f;
}

typedef struct { float* x[N_PARAMS]; float* d[N_PARAMS]; } Params;

static void init_host(float* hx, int* ht, float* hp[N_PARAMS]) {
  static const float scale[N_PARAMS] = { 0.4f, 0.1f, 0.12f, 0.1f, 0.1f, 0.1f, 0.25f, 0.1f };
  for (int i = 0; i < X_N; i++) hx[i] = frand() + 0.5f;
  for (int i = 0; i < B; i++) { g_lcg = g_lcg * 1664525u + 1013904223u; ht[i] = (int)((g_lcg >> 16) % 10u); }
  for (int p = 0; p < N_PARAMS; p++) {
    hp[p] = (float*)malloc(sizeof(float) * (size_t)kParamSize[p]);
    for (int64_t i = 0; i < kParamSize[p]; i++) hp[p][i] = frand() * 2.0f * scale[p];
  }
}

/* ------------------------------------------------------------------ device */
static float* dmalloc(int64_t n) { return (float*)lh_malloc(sizeof(float) * (size_t)n); }       /* reads as zero */
static float* dmalloc_u(int64_t n) { return (float*)lh_malloc_uninit(sizeof(float) * (size_t)n); }

static void run_hip(const float* hx, const int* ht, float* const hp[N_PARAMS], float* losses, float* out[N_PARAMS]) {
  lh_setup((size_t)256 << 20);
  Params P;
  for (int p = 0; p < N_PARAMS; p++) {
    P.x[p] = dmalloc_u(kParamSize[p]); lh_h2d(P.x[p], hp[p], sizeof(float) * (size_t)kParamSize[p]);
    P.d[p] = dmalloc(kParamSize[p]);
  }
  float* x = dmalloc_u(X_N); lh_h2d(x, hx, sizeof(float) * X_N);
  int* tgt = (int*)lh_malloc_uninit(sizeof(int) * B); lh_h2d(tgt, ht, sizeof(int) * B);
  float* ones = dmalloc_u(B); lh_fill(ones, 1.0f, B);
  const size_t mark = lh_mark();

  for (int s = 0; s < STEPS; s++) {
    /* forward */
    float* c1 = dmalloc_u(C1_N); lh_conv2d_fwd(x, P.x[0], P.x[1], c1, B, 1, 28, 28, 10, 5, 5, 1, 1, 0, 0);
    float* r1 = dmalloc_u(C1_N); lh_unary(LH_RELU, c1, r1, C1_N, 0.f, 0.f);
    float* p1 = dmalloc_u(P1_N); int* a1 = (int*)lh_malloc_uninit(sizeof(int) * P1_N);
    lh_maxpool_fwd(r1, p1, a1, B, 10, 24, 24, 2, 2, 2, 2, 0);
    float* c2 = dmalloc_u(C2_N); lh_conv2d_fwd(p1, P.x[2], P.x[3], c2, B, 10, 12, 12, 20, 5, 5, 1, 1, 0, 0);
    float* r2 = dmalloc_u(C2_N); lh_unary(LH_RELU, c2, r2, C2_N, 0.f, 0.f);
    float* p2 = dmalloc_u(P2_N); int* a2 = (int*)lh_malloc_uninit(sizeof(int) * P2_N);
    lh_maxpool_fwd(r2, p2, a2, B, 20, 8, 8, 2, 2, 2, 2, 0);
    float* h1 = dmalloc_u(H1_N); lh_fill_with_bias(h1, P.x[5], B, 50, 1);
    lh_sgemm(0, 0, B, 50, 320, 1.f, p2, 320, P.x[4], 50, 1.f, h1, 50);
    float* z = dmalloc_u(Z_N); lh_fill_with_bias(z, P.x[7], B, 10, 1);
    lh_sgemm(0, 0, B, 10, 50, 1.f, h1, 50, P.x[6], 10, 1.f, z, 10);
    float* ls = dmalloc_u(Z_N); lh_softmax(1, z, ls, B, 10, 1);
    float* nl = dmalloc_u(B); lh_nll(ls, tgt, nl, B, 10);
    float* loss = dmalloc_u(1); lh_sum_all(nl, loss, B);
    /* backward: every gradient buffer comes zeroed from the arena and the gradient entry points add into it */
    float* dls = dmalloc(Z_N); lh_nll_grad(dls, tgt, ones, B, 10);
    float* dz = dmalloc(Z_N); lh_softmax_grad(1, ls, dls, dz, B, 10, 1);
    float* t10 = dmalloc_u(10); lh_sum_dim(dz, t10, 1, B, 10); lh_geam(P.d[7], 1.f, t10, 1.f, P.d[7], 10);
    lh_sgemm(1, 0, 50, 10, B, 1.f, h1, 50, dz, 10, 1.f, P.d[6], 10);
    float* dh1 = dmalloc_u(H1_N); lh_sgemm(0, 1, B, 50, 10, 1.f, dz, 10, P.x[6], 10, 0.f, dh1, 50);
    float* t50 = dmalloc_u(50); lh_sum_dim(dh1, t50, 1, B, 50); lh_geam(P.d[5], 1.f, t50, 1.f, P.d[5], 50);
    lh_sgemm(1, 0, 320, 50, B, 1.f, p2, 320, dh1, 50, 1.f, P.d[4], 50);
    float* dp2 = dmalloc_u(P2_N); lh_sgemm(0, 1, B, 320, 50, 1.f, dh1, 50, P.x[4], 50, 0.f, dp2, 320);
    float* dr2 = dmalloc(C2_N); lh_maxpool_bwd(dp2, a2, dr2, P2_N);
    float* dc2 = dmalloc(C2_N); lh_unary_grad(LH_RELU, c2, r2, dr2, dc2, C2_N, 0, 0.f, 0.f);
    lh_conv2d_bwd_filter(p1, dc2, P.d[2], P.d[3], 1.f, B, 10, 12, 12, 20, 5, 5, 1, 1, 0, 0);
    float* dp1 = dmalloc_u(P1_N); lh_conv2d_bwd_data(dc2, P.x[2], dp1, 0.f, B, 10, 12, 12, 20, 5, 5, 1, 1, 0, 0);
    float* dr1 = dmalloc(C1_N); lh_maxpool_bwd(dp1, a1, dr1, P1_N);
    float* dc1 = dmalloc(C1_N); lh_unary_grad(LH_RELU, c1, r1, dr1, dc1, C1_N, 0, 0.f, 0.f);
    lh_conv2d_bwd_filter(x, dc1, P.d[0], P.d[1], 1.f, B, 1, 28, 28, 10, 5, 5, 1, 1, 0, 0);   /* x is the input: no dx */
    /* update; lh_sgd also clears the gradient */
    for (int p = 0; p < N_PARAMS; p++) lh_sgd(P.x[p], P.d[p], LR, kParamSize[p]);
    lh_d2h(&losses[s], loss, sizeof(float));
    lh_rewind(mark);
  }
  for (int p = 0; p < N_PARAMS; p++) {
    out[p] = (float*)malloc(sizeof(float) * (size_t)kParamSize[p]);
    lh_d2h(out[p], P.x[p], sizeof(float) * (size_t)kParamSize[p]);
  }
  lh_cleanup();
}

/* ------------------------------------------------------------------ oracle */
static float* hcalloc(int64_t n) { return (float*)calloc((size_t)n, sizeof(float)); }

static void run_cpu(const float* hx, const int* ht, float* const hp[N_PARAMS], float* losses, float* out[N_PARAMS]) {
  Params P;
  for (int p = 0; p < N_PARAMS; p++) {
    P.x[p] = hcalloc(kParamSize[p]); memcpy(P.x[p], hp[p], sizeof(float) * (size_t)kParamSize[p]);
    P.d[p] = hcalloc(kParamSize[p]);
  }
  float ones[B]; for (int i = 0; i < B; i++) ones[i] = 1.f;
  const int64_t F1_N = (int64_t)B * 25 * 576, F2_N = (int64_t)B * 250 * 64;
  for (int s = 0; s < STEPS; s++) {
    float *c1 = hcalloc(C1_N), *f1 = hcalloc(F1_N), *r1 = hcalloc(C1_N), *p1 = hcalloc(P1_N);
    int *a1 = (int*)calloc(P1_N, sizeof(int)), *a2 = (int*)calloc(P2_N, sizeof(int));
    float *c2 = hcalloc(C2_N), *f2 = hcalloc(F2_N), *r2 = hcalloc(C2_N), *p2 = hcalloc(P2_N);
    float *h1 = hcalloc(H1_N), *z = hcalloc(Z_N), *ls = hcalloc(Z_N), *nl = hcalloc(B), loss = 0.f;
    lc_conv2d_fwd(hx, P.x[0], P.x[1], c1, f1, B, 1, 28, 28, 10, 5, 5, 1, 1, 0, 0);
    lc_unary(LH_RELU, c1, r1, C1_N, 0.f, 0.f);
    lc_maxpool_fwd(r1, p1, a1, B, 10, 24, 24, 2, 2, 2, 2, 0);
    lc_conv2d_fwd(p1, P.x[2], P.x[3], c2, f2, B, 10, 12, 12, 20, 5, 5, 1, 1, 0, 0);
    lc_unary(LH_RELU, c2, r2, C2_N, 0.f, 0.f);
    lc_maxpool_fwd(r2, p2, a2, B, 20, 8, 8, 2, 2, 2, 2, 0);
    lc_fill_with_bias(h1, P.x[5], B, 50, 1);
    lc_sgemm(0, 0, B, 50, 320, 1.f, p2, 320, P.x[4], 50, 1.f, h1, 50);
    lc_fill_with_bias(z, P.x[7], B, 10, 1);
    lc_sgemm(0, 0, B, 10, 50, 1.f, h1, 50, P.x[6], 10, 1.f, z, 10);
    lc_softmax(1, z, ls, B, 10);
    lc_nll(ls, ht, nl, B, 10);
    lc_sum_all(nl, &loss, B);
    float *dls = hcalloc(Z_N), *dz = hcalloc(Z_N), t10[10] = {0}, t50[50] = {0};   /* lc_sum_dim adds into y */
    float *dh1 = hcalloc(H1_N), *dp2 = hcalloc(P2_N);
    float *dr2 = hcalloc(C2_N), *dc2 = hcalloc(C2_N), *dp1 = hcalloc(P1_N), *dr1 = hcalloc(C1_N), *dc1 = hcalloc(C1_N);
    float *g2 = hcalloc(F2_N);
    lc_nll_grad(dls, ht, ones, B, 10);
    lc_softmax_grad(1, ls, dls, dz, B, 10);
    lc_sum_dim(dz, t10, 1, B, 10); lc_geam(P.d[7], 1.f, t10, 1.f, P.d[7], 10);
    lc_sgemm(1, 0, 50, 10, B, 1.f, h1, 50, dz, 10, 1.f, P.d[6], 10);
    lc_sgemm(0, 1, B, 50, 10, 1.f, dz, 10, P.x[6], 10, 0.f, dh1, 50);
    lc_sum_dim(dh1, t50, 1, B, 50); lc_geam(P.d[5], 1.f, t50, 1.f, P.d[5], 50);
    lc_sgemm(1, 0, 320, 50, B, 1.f, p2, 320, dh1, 50, 1.f, P.d[4], 50);
    lc_sgemm(0, 1, B, 320, 50, 1.f, dh1, 50, P.x[4], 50, 0.f, dp2, 320);
    lc_maxpool_bwd(dp2, a2, dr2, P2_N);
    lc_unary_grad(LH_RELU, c2, r2, dr2, dc2, C2_N, 0, 0.f, 0.f);
    lc_conv2d_bwd(f2, P.x[2], dc2, dp1, P.d[2], P.d[3], g2, B, 10, 12, 12, 20, 5, 5, 1, 1, 0, 0);
    lc_maxpool_bwd(dp1, a1, dr1, P1_N);
    lc_unary_grad(LH_RELU, c1, r1, dr1, dc1, C1_N, 0, 0.f, 0.f);
    lc_conv2d_bwd(f1, P.x[0], dc1, NULL, P.d[0], P.d[1], NULL, B, 1, 28, 28, 10, 5, 5, 1, 1, 0, 0);
    for (int p = 0; p < N_PARAMS; p++) lc_sgd(P.x[p], P.d[p], LR, (long)kParamSize[p]);
    losses[s] = loss;
    free(c1); free(f1); free(r1); free(p1); free(a1); free(a2); free(c2); free(f2); free(r2); free(p2);
    free(h1); free(z); free(ls); free(nl); free(dls); free(dz); free(dh1); free(dp2); free(dr2); free(dc2);
    free(dp1); free(dr1); free(dc1); free(g2);
  }
  for (int p = 0; p < N_PARAMS; p++) { out[p] = P.x[p]; free(P.d[p]); }
}

int main(void) {
  if (getenv("LENET_STEP_LINK_ONLY")) { printf("linked\n"); return 0; }
  float* hx = (float*)malloc(sizeof(float) * X_N);
  int ht[B];
  float* hp[N_PARAMS];
  init_host(hx, ht, hp);
  float lg[STEPS], lc[STEPS], *pg[N_PARAMS], *pc[N_PARAMS];
  run_cpu(hx, ht, hp, lc, pc);
  run_hip(hx, ht, hp, lg, pg);
  int bad = 0;
  for (int s = 0; s < STEPS; s++) {
    const float rel = fabsf(lg[s] - lc[s]) / fmaxf(fabsf(lc[s]), 1e-6f);
    printf("step %d loss hip %.6f cpu %.6f rel %.2e\n", s, lg[s], lc[s], rel);
    if (!(rel <= 1e-4f)) bad = 1;
  }
  if (!(lc[STEPS - 1] < lc[0])) { printf("loss did not fall\n"); bad = 1; }
  for (int p = 0; p < N_PARAMS; p++) {
    float mx = 0.f, err = 0.f, moved = 0.f;
    for (int64_t i = 0; i < kParamSize[p]; i++) {
      mx = fmaxf(mx, fabsf(pc[p][i])); err = fmaxf(err, fabsf(pg[p][i] - pc[p][i]));
      moved = fmaxf(moved, fabsf(pc[p][i] - hp[p][i]));
    }
    printf("param %d size %ld max|p| %.4f moved %.2e max err %.2e\n", p, (long)kParamSize[p], mx, moved, err);
    if (!(err <= 1e-3f * mx) || !(moved > 0.f)) bad = 1;
  }
  printf(bad ? "MISMATCH\n" : "ok\n");
  return bad;
}
