// Brute-force check of the command list's record-time analysis (lantern_amd/csrc/lh_cmdlist_levels.h), built as plain host
// code with -fsanitize=address,undefined.  Seeded random command streams over a synthetic address space (vectors, slices of
// vectors at odd offsets, matrices, large fills, buffers shared between element-wise and matrix commands) are placed one
// command at a time; after every command the level and chain it got are compared with every earlier command of the window:
//   * two commands that touch overlapping bytes, at least one of them writing, must be on different levels in recording
//     order, or on ONE level as members of ONE chain;
//   * members of one chain on one level must map their operands onto wavefronts alike: the same class, (rank-1 updates) the
//     same row length, and every conflicting pair of ranges starting at the same address; a matrix command may meet a
//     chain mate only through what both WRITE;
//   * a level is never lower than 1 and never more than one above the highest level so far.
// Usage: levels_check [streams] [commands per stream] [seed]; exit status 0 = no violation.
#include <stdio.h>
#include <stdlib.h>
#include <vector>
#include "../../lantern_amd/csrc/lh_cmdlist_levels.h"

static uint64_t g_rng = 1;
static uint32_t rnd() { g_rng = g_rng * 6364136223846793005ull + 1442695040888963407ull; return (uint32_t)(g_rng >> 33); }
static int ri(int lo, int hi) { return lo + (int)(rnd() % (uint32_t)(hi - lo + 1)); }

struct Buf { uintptr_t p; int n; };      // n floats at p (256-byte aligned, like arena blocks)

int main(int argc, char** argv) {
  const int streams = argc > 1 ? atoi(argv[1]) : 200, per = argc > 2 ? atoi(argv[2]) : 600;
  g_rng = argc > 3 ? (uint64_t)atoll(argv[3]) : 12345;
  Window* Wp = window_new();
  Window& W = *Wp;
  long long placed = 0, chained = 0, resets = 0, pairs = 0, max_level = 0;
  for (int st = 0; st < streams; st++) {
    window_reset(W);
    const bool chains = (st % 5) != 4;
    // a fresh address space: small vectors, a few matrices, one large region for fills and wide element-wise commands
    std::vector<Buf> vec, mat;
    uintptr_t top = 0x7f0000000000ull + (uintptr_t)ri(0, 1 << 20) * 256;
    const int nvec = ri(4, 40), nmat = ri(1, 6);
    const int dim = ri(0, 3) == 0 ? ri(3, 40) : 150;            // mostly the tree model's 150-element vectors
    for (int i = 0; i < nvec; i++) { int n = ri(0, 4) == 0 ? ri(1, 1200) : dim; vec.push_back({top, n}); top += ((uintptr_t)n * 4 + 255) & ~(uintptr_t)255; if (ri(0, 9) == 0) top += 256 * (uintptr_t)ri(1, 64); }
    for (int i = 0; i < nmat; i++) { int m = ri(2, 300), n = ri(2, 300); mat.push_back({top, m * n}); top += ((uintptr_t)m * n * 4 + 255) & ~(uintptr_t)255; }
    Buf wide = {top, ri(4096, 60000)}; top += ((uintptr_t)wide.n * 4 + 255) & ~(uintptr_t)255;
    std::vector<Extent> ext; std::vector<int> ext_of, ext_idx;   // ranges of the commands placed in this window
    int first_in_window = 0; (void)first_in_window;
    auto slice = [&](const Buf& b, int need) -> uintptr_t { int off = b.n > need && ri(0, 3) == 0 ? ri(0, b.n - need) : 0; return b.p + (uintptr_t)off * 4; };
    for (int k = 0; k < per; k++) {
      LhCmd c{};
      const int kind = ri(0, 19);
      auto v = [&]() -> const Buf& { return vec[ri(0, nvec - 1)]; };
      if (kind <= 7) {                     // element-wise over (slices of) vectors
        const Buf &a = v(), &b = v(), &d = v();
        int n = a.n < b.n ? a.n : b.n; if (d.n < n) n = d.n; n = ri(1, n);
        static const int ops[] = {CL_FILL, CL_COPY, CL_GEAM, CL_SCALAR, CL_BIN, CL_ACC, CL_ACCNEG, CL_ACCMUL, CL_UNARY, CL_UNARY_GRAD, CL_ADAGRAD, CL_SGD};
        c.op = ops[ri(0, 11)]; c.i0 = n;
        c.p0 = (void*)slice(a, n); c.p1 = (void*)slice(b, n); c.p2 = (void*)slice(d, n); c.p3 = (void*)slice(v().n >= n ? v() : a, n);
        if (ri(0, 2) == 0) c.p1 = c.p0;                         // in-place forms
      } else if (kind <= 11) {             // matrix-vector products and rank-1 updates
        const Buf& M = mat[ri(0, nmat - 1)];
        int m = ri(1, 40), n = M.n / m; if (n > 300) n = 300; if (n < 1) { n = 1; m = M.n; }
        const int op = ri(0, 2);
        c.op = op == 0 ? CL_GEMV_N : op == 1 ? CL_GEMV_T : CL_GER;
        c.i0 = m; c.i1 = n; c.i2 = n;
        const Buf *x = &v(), *y = &v();
        if (c.op == CL_GEMV_N) { while (x->n < n) x = &wide; while (y->n < m) y = &wide; c.p0 = (void*)y->p; c.p1 = (void*)M.p; c.p2 = (void*)x->p; }
        else if (c.op == CL_GEMV_T) { while (x->n < m) x = &wide; while (y->n < n) y = &wide; c.p0 = (void*)y->p; c.p1 = (void*)M.p; c.p2 = (void*)x->p; }
        else { while (x->n < m) x = &wide; while (y->n < n) y = &wide; c.p0 = (void*)M.p; c.p1 = (void*)x->p; c.p2 = (void*)y->p; }
      } else if (kind <= 13) {             // reductions to a scalar, scalar times vector
        const Buf &a = v(), &b = v(), &d = v();
        int n = ri(1, a.n < b.n ? a.n : b.n);
        if (ri(0, 1)) { c.op = CL_DOT; c.i0 = n; c.p0 = (void*)slice(d, 1); c.p1 = (void*)a.p; c.p2 = (void*)b.p; }
        else { c.op = CL_AXPY_DEV; c.i0 = n; c.p0 = (void*)a.p; c.p1 = (void*)slice(d, 1); c.p2 = (void*)b.p; }
      } else if (kind <= 15) {             // rows of classes
        const Buf &a = v(), &b = v(), &d = v();
        int cls = ri(2, 7), rows = (a.n < b.n ? a.n : b.n) / cls; if (rows < 1) { rows = 1; cls = 1; } if (rows > 5) rows = ri(1, 5);
        const int op = ri(0, 3);
        c.i0 = rows; c.i1 = cls;
        if (op == 0) { c.op = CL_SOFTMAX; c.p0 = (void*)a.p; c.p1 = (void*)b.p; }
        else if (op == 1) { c.op = CL_SOFTMAX_GRAD; c.p0 = (void*)a.p; c.p1 = (void*)b.p; c.p2 = (void*)(d.n >= rows * cls ? d.p : b.p); }
        else if (op == 2) { c.op = CL_NLL; c.p0 = (void*)(d.n >= rows ? d.p : a.p); c.p1 = (void*)a.p; c.p2 = (void*)b.p; }
        else { c.op = CL_NLL_GRAD; c.p0 = (void*)a.p; c.p1 = (void*)b.p; c.p2 = (void*)(d.n >= rows ? d.p : b.p); }
      } else if (kind <= 17) {             // wide element-wise commands and large fills over the shared region (and over the vectors behind it)
        const int n = ri(4096, wide.n);
        if (ri(0, 2) == 0) { c.op = CL_ZERO16; c.i0 = (n / 4); c.p0 = (void*)(ri(0, 3) == 0 ? vec[0].p : wide.p); if (c.p0 == (void*)vec[0].p) c.i0 = ri(16, 4000); }
        else { c.op = ri(0, 1) ? CL_SGD : CL_GEAM; c.i0 = n; c.p0 = (void*)wide.p; c.p1 = (void*)(ri(0, 1) ? wide.p : mat[0].p); c.p2 = (void*)wide.p; if (c.p1 == (void*)mat[0].p && mat[0].n < n) c.p1 = (void*)wide.p; }
      } else {                             // a matrix used element-wise (a parameter update over a weight matrix)
        const Buf& M = mat[ri(0, nmat - 1)];
        c.op = ri(0, 1) ? CL_ADAGRAD : CL_SGD; c.i0 = M.n; c.p0 = (void*)M.p; c.p1 = (void*)M.p; c.p2 = (void*)M.p;
        if (c.op == CL_ADAGRAD || ri(0, 1)) { const Buf& M2 = mat[ri(0, nmat - 1)]; if (M2.n >= M.n) c.p1 = (void*)M2.p; }
      }
      int lv = 0, chain = -1;
      bool ok = window_place(W, c, chains, lv, chain);
      if (!ok || W.n == CL_BUF_CMDS) {     // a table is full (or the buffer): the library hands the buffer over and starts a new window
        window_reset(W); ext.clear(); ext_of.clear(); ext_idx.clear(); resets++;
        if (!ok) { ok = window_place(W, c, chains, lv, chain); if (!ok) { fprintf(stderr, "stream %d command %d: does not fit an empty window\n", st, k); return 1; } }
        else continue;
      }
      const int j = W.n - 1;
      placed++; if (lv > max_level) max_level = lv;
      if (lv < 1 || lv > W.top) { fprintf(stderr, "stream %d command %d: level %d outside 1..%d\n", st, k, lv, W.top); return 1; }
      Extent xj[4]; const int kj = cmd_extents(c, xj);
      const int cls_j = cmd_class(c);
      for (size_t e = 0; e < ext.size(); e++) {
        const int i = ext_of[e];
        for (int q = 0; q < kj; q++) {
          if (!(ext[e].s < xj[q].e && xj[q].s < ext[e].e) || !(ext[e].w || xj[q].w)) continue;
          pairs++;
          const int li = W.level[i];
          if (li < lv) continue;
          const char* why = nullptr;
          if (li > lv) why = "an earlier command it conflicts with is on a LATER level";
          else if (chain < 0 || W.chain[i] != chain) why = "a conflicting earlier command shares its level without sharing its chain";
          else {
            const int cls_i = cmd_class(W.cmd[i]);
            if (cls_i != cls_j || cls_j == 0) why = "chain mates of different classes";
            else if (cls_j == 4 && W.cmd[i].i1 != c.i1) why = "rank-1 updates with different row lengths in one chain";
            else if (ext[e].s != xj[q].s) why = "chain mates conflict through ranges that start at different addresses";
            else if (cls_j >= 2 && (ext_idx[e] != 0 || q != 0)) why = "matrix commands of one chain meet through something one of them only reads";
          }
          if (why) {
            fprintf(stderr, "stream %d (seed state), command %d (op %d, level %d, chain %d) against window entry %d (op %d, level %d, chain %d): %s\n",
                    st, k, c.op, lv, chain, i, W.cmd[i].op, li, W.chain[i], why);
            return 1;
          }
          if (li == lv) chained++;
        }
      }
      for (int q = 0; q < kj; q++) { ext.push_back(xj[q]); ext_of.push_back(j); ext_idx.push_back(q); }
    }
  }
  printf("levels_check: %lld commands placed in %d streams, %lld conflicting range pairs compared, %lld of them inside chains, %lld window resets, highest level %lld: no violation\n",
         placed, streams, pairs, chained, resets, max_level);
  delete Wp;
  return 0;
}
