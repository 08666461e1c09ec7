/* The sentiment TreeLSTM training loop as a host program in plain C99 over liblantern_hip.so, in the shape of the program
 * the reference emits for src/main/scala/lantern/PLDI19APP/SentimentTreeLSTM.scala:242-345 (GPU variant): a recursion over
 * the tree arrays lch / rch with the forward operators on the way down and their gradient operators on the way back, every
 * tensor and gradient cut from the bump-pointer arena (gradients read zero), an Adagrad step and an arena rewind after each
 * tree.  One library call per trait call, in the reference's order; with `cmdlist` = 1 the small calls are executed from
 * the library's command list (lh_cmdlist_begin), which changes nothing in this program.
 *
 * The reference binds the pair a Leaf / Node returns, (hidden, cell), to `val ArrayBuffer(cell, hidden)` (:302, :307): the
 * classifier reads the cell state and the two vectors change roles on the way up.  Kept.
 *
 *   treelstm_step <params.bin> <trees.txt> <out.bin> <steps> <warmup> <cmdlist 0|1>
 *
 * params.bin: int32 vocab, emb, hidden, classes; then fp32 arrays: embedding [vocab, emb]; leaf Wi [h, emb], bi, Wo, bo,
 *   Wu, bu; node U0i U1i bbi U00f U01f U10f U11f bbf U0o U1o bbo U0u U1u bbu ([h, h] or [h]); output Why [classes, h], by.
 * trees.txt: the reference's array_tree.txt layout: number of trees, then per tree its size and four arrays of that length
 *   (scores, words with -1 for inner nodes, left child, right child with -1 for leaves); the root is node 0.
 * out.bin: `steps` losses (fp32), then the 22 parameter arrays after the last step, in the order above.
 * stdout: one line `trees_per_s <value> ms_per_tree <value> nodes <total> host_issue_ms_per_tree <value>` over the `steps` trees
 *   behind the warm-up ones (tree t of the run is tree t modulo the number of trees in the file); the last figure is the time
 *   the host needed to issue a tree's calls, the device running behind it.
 * TREELSTM_STEP_LINK_ONLY in the environment: return before touching the device (link check without one).
 */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "lantern_hip.h"

typedef struct { float* x; float* d; } T;          /* a TensorR: value and gradient */

static int EMB, HID, CLS, VOCAB;
static int dimH[1];

static T tnew(int n) {                                /* result of an operator: value written by it, gradient reads zero */
  T t;
  t.x = (float*)lh_malloc_uninit(sizeof(float) * (size_t)n);
  t.d = (float*)lh_malloc(sizeof(float) * (size_t)n);
  return t;
}

enum { N_PARAMS = 22 };
static T P[N_PARAMS];
static float* M[N_PARAMS];                            /* Adagrad moments */
static int64_t PN[N_PARAMS];
enum { Wi, bi, Wo, bo, Wu, bu, U0i, U1i, bbi, U00f, U01f, U10f, U11f, bbf, U0o, U1o, bbo, U0u, U1u, bbu, Why, by };
static float* embedding;

/* ---- forward operators (one library call each) and what the backward pass needs of them ------------------------------- */
static T dot(T W, const float* v, int m, int n) { T y = tnew(m); lh_sgemv(0, m, n, 1.f, W.x, n, v, 0.f, y.x); return y; }
static void plus_in_place(T y, const float* z, int n) { lh_geam(y.x, 1.f, z, 1.f, y.x, n); }      /* plusBias, plusEqual */
static T unary(int op, T x, int n) { T y = tnew(n); lh_unary(op, x.x, y.x, n, -1.f, 1.f); return y; }
static T mul(T a, T b) { T y = tnew(HID); lh_bcast_op(LH_MUL, a.x, dimH, b.x, dimH, y.x, dimH, 1); return y; }

static void dot_grad(T W, T v, int v_is_input, T y, int m, int n) {        /* CPU:171-184: add_cartesian, add_composition */
  lh_ger(m, n, y.d, v.x, W.d);
  if (!v_is_input) lh_sgemv(1, m, n, 1.f, W.x, n, y.d, 1.f, v.d);
}
static void plus_grad(float* zd, T y, int n) { lh_geam(zd, 1.f, y.d, 1.f, zd, n); }
static void unary_grad(int op, T x, T y, int n) { lh_unary_grad(op, x.x, y.x, y.d, x.d, n, 0, -1.f, 1.f); }
static void mul_grad(T a, T b, T y) { lh_bcast_op_grad(LH_MUL, a.x, a.d, dimH, 0, b.x, b.d, dimH, 0, y.d, dimH, 1); }

/* what one tree node keeps between its forward and its backward part */
typedef struct {
  T pre[5], second[5], act[5];          /* gate pre-activations (first product, in-place sums), second products, activations */
  T iu, flc, frc, cell, tcell, hidden;  /* products of the cell update, the cell, tanh(cell), the hidden state */
  T pred, ls, loss;                     /* classifier */
  T emb;                                /* leaf: the embedding row (an input: no gradient) */
  T up_hidden, up_cell;                 /* what the parent sees (the pair as the reference binds it) */
} Node;

static Node* nodes;
static const int *scores_h, *words, *lch, *rch;
static int* scores_dev;

static void classifier_forward(Node* nd, int i) {
  nd->pred = dot(P[Why], nd->up_hidden.x, CLS, HID);
  plus_in_place(nd->pred, P[by].x, CLS);
  nd->ls = tnew(CLS); lh_softmax(1, nd->pred.x, nd->ls.x, 1, CLS, 1);
  nd->loss = tnew(1); lh_nll(nd->ls.x, scores_dev + i, nd->loss.x, 1, CLS);
}
static void classifier_backward(Node* nd, int i) {
  lh_nll_grad(nd->ls.d, scores_dev + i, nd->loss.d, 1, CLS);
  lh_softmax_grad(1, nd->ls.x, nd->ls.d, nd->pred.d, 1, CLS, 1);
  plus_grad(P[by].d, nd->pred, CLS);
  dot_grad(P[Why], nd->up_hidden, 0, nd->pred, CLS, HID);
}

static void forward(int i) {
  Node* nd = &nodes[i];
  if (lch[i] < 0) {                                   /* Leaf (:244-258) */
    static const int W3[3] = { Wi, Wo, Wu }, B3[3] = { bi, bo, bu }, OP3[3] = { LH_SIGMOID, LH_SIGMOID, LH_TANH };
    nd->emb.x = embedding + (size_t)words[i] * EMB; nd->emb.d = NULL;
    for (int g = 0; g < 3; g++) {
      nd->pre[g] = dot(P[W3[g]], nd->emb.x, HID, EMB);
      plus_in_place(nd->pre[g], P[B3[g]].x, HID);
      nd->act[g] = unary(OP3[g], nd->pre[g], HID);
    }
    nd->cell = mul(nd->act[0], nd->act[2]);           /* i * u */
    nd->tcell = unary(LH_TANH, nd->cell, HID);
    nd->hidden = mul(nd->act[1], nd->tcell);          /* o * tanh(cell) */
  } else {                                            /* Node (:260-292) */
    forward(lch[i]); forward(rch[i]);
    const Node* L = &nodes[lch[i]]; const Node* R = &nodes[rch[i]];
    static const int A5[5] = { U0i, U00f, U10f, U0o, U0u }, B5[5] = { U1i, U01f, U11f, U1o, U1u }, C5[5] = { bbi, bbf, bbf, bbo, bbu };
    static const int OP5[5] = { LH_SIGMOID, LH_SIGMOID, LH_SIGMOID, LH_SIGMOID, LH_TANH };
    for (int g = 0; g < 5; g++) {                     /* gates i, f_left, f_right, o, u */
      nd->pre[g] = dot(P[A5[g]], L->up_hidden.x, HID, HID);
      nd->second[g] = dot(P[B5[g]], R->up_hidden.x, HID, HID);
      plus_in_place(nd->pre[g], nd->second[g].x, HID);
      plus_in_place(nd->pre[g], P[C5[g]].x, HID);
      nd->act[g] = unary(OP5[g], nd->pre[g], HID);
    }
    nd->iu = mul(nd->act[0], nd->act[4]);
    nd->flc = mul(nd->act[1], L->up_cell);
    plus_in_place(nd->iu, nd->flc.x, HID);
    nd->frc = mul(nd->act[2], R->up_cell);
    plus_in_place(nd->iu, nd->frc.x, HID);
    nd->cell = nd->iu;                                /* the sum was built in place */
    nd->tcell = unary(LH_TANH, nd->cell, HID);
    nd->hidden = mul(nd->act[3], nd->tcell);
  }
  nd->up_cell = nd->hidden; nd->up_hidden = nd->cell; /* `val ArrayBuffer(cell, hidden) = ...` of a (hidden, cell) pair */
  classifier_forward(nd, i);
  if (lch[i] >= 0) {
    plus_in_place(nd->loss, nodes[lch[i]].loss.x, 1);
    plus_in_place(nd->loss, nodes[rch[i]].loss.x, 1);
  }
}

static void backward(int i) {
  Node* nd = &nodes[i];
  if (lch[i] >= 0) {
    plus_grad(nodes[rch[i]].loss.d, nd->loss, 1);
    plus_grad(nodes[lch[i]].loss.d, nd->loss, 1);
  }
  classifier_backward(nd, i);
  if (lch[i] < 0) {
    static const int W3[3] = { Wi, Wo, Wu }, B3[3] = { bi, bo, bu }, OP3[3] = { LH_SIGMOID, LH_SIGMOID, LH_TANH };
    mul_grad(nd->act[1], nd->tcell, nd->hidden);
    unary_grad(LH_TANH, nd->cell, nd->tcell, HID);
    mul_grad(nd->act[0], nd->act[2], nd->cell);
    for (int g = 2; g >= 0; g--) {
      unary_grad(OP3[g], nd->pre[g], nd->act[g], HID);
      plus_grad(P[B3[g]].d, nd->pre[g], HID);
      dot_grad(P[W3[g]], nd->emb, 1, nd->pre[g], HID, EMB);
    }
  } else {
    Node* L = &nodes[lch[i]]; Node* R = &nodes[rch[i]];
    static const int A5[5] = { U0i, U00f, U10f, U0o, U0u }, B5[5] = { U1i, U01f, U11f, U1o, U1u }, C5[5] = { bbi, bbf, bbf, bbo, bbu };
    static const int OP5[5] = { LH_SIGMOID, LH_SIGMOID, LH_SIGMOID, LH_SIGMOID, LH_TANH };
    static const int ORDER[5] = { 4, 3, 2, 1, 0 };    /* reverse of the forward order */
    mul_grad(nd->act[3], nd->tcell, nd->hidden);
    unary_grad(LH_TANH, nd->cell, nd->tcell, HID);
    plus_grad(nd->frc.d, nd->cell, HID);
    mul_grad(nd->act[2], R->up_cell, nd->frc);
    plus_grad(nd->flc.d, nd->cell, HID);
    mul_grad(nd->act[1], L->up_cell, nd->flc);
    mul_grad(nd->act[0], nd->act[4], nd->iu);
    for (int k = 0; k < 5; k++) {
      const int g = ORDER[k];
      unary_grad(OP5[g], nd->pre[g], nd->act[g], HID);
      plus_grad(P[C5[g]].d, nd->pre[g], HID);
      plus_grad(nd->second[g].d, nd->pre[g], HID);
      dot_grad(P[B5[g]], R->up_hidden, 0, nd->second[g], HID, HID);
      dot_grad(P[A5[g]], L->up_hidden, 0, nd->pre[g], HID, HID);
    }
    backward(rch[i]); backward(lch[i]);
  }
}

/* ---- files --------------------------------------------------------------------------------------------------------------- */
static void die(const char* what) { fprintf(stderr, "treelstm_step: %s\n", what); exit(2); }

typedef struct { int size; int *scores, *words, *lch, *rch; } Tree;

static Tree* read_trees(const char* path, int* count) {
  FILE* f = fopen(path, "r");
  if (!f) die("cannot open the tree file");
  if (fscanf(f, "%d", count) != 1 || *count < 1) die("bad tree count");
  Tree* ts = (Tree*)calloc((size_t)*count, sizeof(Tree));
  for (int t = 0; t < *count; t++) {
    if (fscanf(f, "%d", &ts[t].size) != 1 || ts[t].size < 1) die("bad tree size");
    int** arrs[4] = { &ts[t].scores, &ts[t].words, &ts[t].lch, &ts[t].rch };
    for (int a = 0; a < 4; a++) {
      *arrs[a] = (int*)malloc(sizeof(int) * (size_t)ts[t].size);
      for (int i = 0; i < ts[t].size; i++) if (fscanf(f, "%d", &(*arrs[a])[i]) != 1) die("short tree file");
    }
    for (int i = 0; i < ts[t].size; i++) {
      const int leaf = ts[t].lch[i] < 0;
      if (leaf != (ts[t].rch[i] < 0) || (leaf && (ts[t].words[i] < 0 || ts[t].words[i] >= VOCAB)) ||
          (!leaf && (ts[t].lch[i] == i || ts[t].rch[i] == i || ts[t].lch[i] >= ts[t].size || ts[t].rch[i] >= ts[t].size)) ||
          ts[t].scores[i] < 0 || ts[t].scores[i] >= CLS) die("tree arrays out of range");
    }
  }
  fclose(f);
  return ts;
}

static double now_s(void) { struct timespec ts; clock_gettime(CLOCK_MONOTONIC, &ts); return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec; }

int main(int argc, char** argv) {
  if (getenv("TREELSTM_STEP_LINK_ONLY")) { printf("linked\n"); return 0; }
  if (argc != 7) die("usage: treelstm_step <params.bin> <trees.txt> <out.bin> <steps> <warmup> <cmdlist 0|1>");
  const int steps = atoi(argv[4]), warmup = atoi(argv[5]), cmdlist = atoi(argv[6]);
  FILE* pf = fopen(argv[1], "rb");
  if (!pf) die("cannot open the parameter file");
  int hdr[4];
  if (fread(hdr, sizeof(int), 4, pf) != 4) die("short parameter file");
  VOCAB = hdr[0]; EMB = hdr[1]; HID = hdr[2]; CLS = hdr[3]; dimH[0] = HID;
  if (VOCAB < 1 || EMB < 1 || HID < 1 || CLS < 2 || steps < 1 || warmup < 0) die("bad sizes");
  int ntrees = 0, max_size = 0;
  Tree* trees = read_trees(argv[2], &ntrees);
  for (int t = 0; t < ntrees; t++) if (trees[t].size > max_size) max_size = trees[t].size;
  nodes = (Node*)calloc((size_t)max_size, sizeof(Node));

  lh_setup((size_t)2 << 30);
  const int64_t hh = (int64_t)HID * HID, he = (int64_t)HID * EMB;
  const int64_t sizes[N_PARAMS] = { he, HID, he, HID, he, HID, hh, hh, HID, hh, hh, hh, hh, HID, hh, hh, HID, hh, hh, HID, (int64_t)CLS * HID, CLS };
  float* stage = (float*)malloc(sizeof(float) * (size_t)((int64_t)VOCAB * EMB > he ? (int64_t)VOCAB * EMB : he));
  embedding = (float*)lh_malloc_uninit(sizeof(float) * (size_t)VOCAB * EMB);
  if (fread(stage, sizeof(float), (size_t)VOCAB * EMB, pf) != (size_t)VOCAB * EMB) die("short parameter file");
  lh_h2d(embedding, stage, sizeof(float) * (size_t)VOCAB * EMB);
  for (int p = 0; p < N_PARAMS; p++) {
    PN[p] = sizes[p];
    P[p].x = (float*)lh_malloc_uninit(sizeof(float) * (size_t)PN[p]);
    P[p].d = (float*)lh_malloc(sizeof(float) * (size_t)PN[p]);
    M[p] = (float*)lh_malloc(sizeof(float) * (size_t)PN[p]);
    if (fread(stage, sizeof(float), (size_t)PN[p], pf) != (size_t)PN[p]) die("short parameter file");
    lh_h2d(P[p].x, stage, sizeof(float) * (size_t)PN[p]);
  }
  fclose(pf);
  float* losses = (float*)calloc((size_t)(steps + warmup), sizeof(float));
  float* loss_dev = (float*)lh_malloc(sizeof(float) * (size_t)(steps + warmup));   /* below the mark: read back once, at the end */
  const size_t mark = lh_mark();
  if (cmdlist) lh_cmdlist_begin();

  double t0 = 0.0; long total_nodes = 0;
  for (int s = 0; s < steps + warmup; s++) {
    if (s == warmup) { lh_sync(); t0 = now_s(); }
    const Tree* tr = &trees[s % ntrees];
    scores_h = tr->scores; words = tr->words; lch = tr->lch; rch = tr->rch;
    scores_dev = (int*)lh_malloc_uninit(sizeof(int) * (size_t)tr->size);
    lh_h2d(scores_dev, scores_h, sizeof(int) * (size_t)tr->size);                   /* scores.toGPU(size) (:336) */
    forward(0);
    lh_fill(nodes[0].loss.d, 1.0f, 1);                                              /* gradR_loss seeds the root with one */
    lh_d2d(loss_dev + s, nodes[0].loss.x, sizeof(float));
    backward(0);
    for (int p = 0; p < N_PARAMS; p++) lh_adagrad(P[p].x, P[p].d, M[p], 0.05f, 1.0f, PN[p]);
    lh_rewind(mark);
    if (s >= warmup) total_nodes += tr->size;
  }
  const double issued = now_s() - t0;               /* the host is done; the device may still be working */
  lh_sync();
  const double dt = now_s() - t0;
  if (cmdlist) lh_cmdlist_end();
  lh_d2h(losses, loss_dev, sizeof(float) * (size_t)(steps + warmup));

  FILE* of = fopen(argv[3], "wb");
  if (!of) die("cannot open the output file");
  fwrite(losses + warmup, sizeof(float), (size_t)steps, of);
  for (int p = 0; p < N_PARAMS; p++) {
    lh_d2h(stage, P[p].x, sizeof(float) * (size_t)PN[p]);
    fwrite(stage, sizeof(float), (size_t)PN[p], of);
  }
  fclose(of);
  printf("trees_per_s %.2f ms_per_tree %.4f nodes %ld host_issue_ms_per_tree %.4f\n", (double)steps / dt, 1e3 * dt / (double)steps, total_nodes,
         1e3 * issued / (double)steps);
  lh_cleanup();
  return 0;
}
