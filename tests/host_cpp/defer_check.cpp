// Host-only check of the library's deferred-work bookkeeping (lantern_amd/csrc/lh_defer.hip: parked launches, zero fills on
// demand, results produced on demand), built with -fsanitize=address,undefined against a simulated device: the arena is
// host memory, every "kernel" is a loop over it, and the entry points below follow the same protocol as the library's
// (state what is read and written, park what may fuse, run as called while deferred work is launched).
// Seeded random programs in the shape of generated code (conv -> batch norm -> [+ shortcut] -> relu in place, pools of
// element-wise calls on whole buffers and on slices, gradients in reverse order with beta = 1 into fresh lh_malloc blocks,
// one optimizer call per parameter, read-backs at random points, rewinds that hand the same memory out again full of
// garbage) run twice, with the bookkeeping on and with it off (every call runs as issued, every block cleared when handed
// out).  Every read-back and, at the end, the whole arena must be identical bit for bit.
// Usage: defer_check [programs] [seed]; exit status 0 = identical everywhere.
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <vector>

#include "../../lantern_amd/csrc/lh_defer.hip"
#include "../../lantern_amd/csrc/lh_arena.h"

// ---- what the bookkeeping needs from the rest of the library ------------------------------------------------------------
namespace lh {
hipStream_t g_stream_raw = (hipStream_t)0x10, g_stream_cur = (hipStream_t)0x10;
int g_rec_pending = 0, g_rec_on = 0, g_error_mode = 0, g_num_cu = 256, g_kernel_cat = 0;
unsigned g_prof_mask = 0;
double g_work[CAT_COUNT];
void rec_flush() {}
void prof_begin(int) {}
void prof_end(int) {}
bool fail(const char* file, int line, const char* fmt, ...) { fprintf(stderr, "%s:%d: %s\n", file, line, fmt); exit(2); }
bool failed() { return false; }
void side_wait_for_main() {}
void side_join() {}
bool g_capturing = false;
static long long g_layout_builds = 0;
void* persistent_alloc(size_t bytes) { return malloc(bytes); }
void persistent_free(void* p) { free(p); }
bool side_work_begin() { return true; }
void side_work_end() {}
// the simulated filter layout is a plain copy: a stale one still shows, because the values differ
void build_filter_layout(int, const int*, const float* w, float* dst) { (void)ordered_stream(); memcpy(dst, w, 12 * sizeof(float)); g_layout_builds++; }
void build_filter_layouts(int n, const int* kinds, const int* const* prms, const float* const* ws, float* const* dsts) { for (int i = 0; i < n; i++) build_filter_layout(kinds[i], prms[i], ws[i], dsts[i]); }
static const float* sim_filter(const float* w) {
  bool build = false; const int prm[LAYOUT_PRM] = {4, 3, 1};
  float* c = lazy::layout_lookup(w, 12 * sizeof(float), LAYOUT_KRSC, prm, 12 * sizeof(float), build);
  if (c == nullptr) return w;
  if (build) build_filter_layout(LAYOUT_KRSC, prm, w, c);
  return c;
}
static long long g_kernels = 0;           // simulated launches (the two modes differ in how many they need)
void zero_bytes_async(void* p, size_t bytes) { (void)ordered_stream(); memset(p, 0, bytes); g_kernels++; }
void mask_relu(float* dst, const float* src, const float* y, int64_t n) { (void)ordered_stream(); for (int64_t i = 0; i < n; i++) dst[i] = y[i] > 0.f ? src[i] : 0.f; g_kernels++; }
void add_plain(const float* a, const float* b, float* out, int64_t n) { (void)ordered_stream(); for (int64_t i = 0; i < n; i++) out[i] = a[i] + b[i]; g_kernels++; }
void relu_grad_inplace_now(const float* y, float* d, int64_t n) { (void)ordered_stream(); for (int64_t i = 0; i < n; i++) d[i] = y[i] > 0.f ? d[i] : 0.f; g_kernels++; }
static void sim_conv_relu(const float* x, const float* w, const float* bias, float* y);
void conv2d_fwd_relu_now(const float* x, const float* w, const float* bias, float* y, int, int, int, int, int, int, int, int, int, int, int) { (void)ordered_stream(); sim_conv_relu(x, w, bias, y); }
static void sim_bias_grad(const float* y, float* dy, float* db);
void conv_bwd_bias_mask_now(const float* y, float* dy, float* db, int, int, int) { (void)ordered_stream(); sim_bias_grad(y, dy, db); }
static void k_update(int mode, float* x, float* d, float* v, float lr, float mu, float clip, int nesterov, int64_t n) {
  for (int64_t i = 0; i < n; i++) {
    if (mode == 0) { x[i] = x[i] * 1.0f + d[i] * (-lr); d[i] = 0.f; continue; }
    float t = d[i]; if (t > clip) t = clip; if (t < -clip) t = -clip;
    float vv = v[i] * mu; vv += t;
    if (nesterov) t += mu * vv; else t = vv;
    x[i] -= lr * t; v[i] = vv; d[i] = 0.f;
  }
}
void multi_update_now(int mode, int count, float* const* hx, float* const* hd, float* const* hv, const int64_t* hn, float lr, float mu, float clip, int nesterov) {
  (void)ordered_stream();
  for (int t = 0; t < count; t++) k_update(mode, hx[t], hd[t], hv ? hv[t] : nullptr, lr, mu, clip, nesterov, hn[t]);
  g_kernels++;
}
}  // namespace lh
using namespace lh;

// ---- the arena: the library's own bookkeeping (lh_arena.h) over host memory, acted on as lh_runtime.hip acts on it ----------
static char* g_heap; static ArenaState g_arena;
static const size_t ZERO_AHEAD = 1024, LAZY_MIN = 512;     // the library uses 1 MiB and 16 KiB; here four 256-byte blocks make a window and every activation (768 bytes) is "large"
static void* sim_malloc(size_t bytes, bool zero) {
  const ArenaGrant g = arena_bump(g_arena, bytes, zero, lazy::defer_zero(), ZERO_AHEAD, LAZY_MIN);
  if (!g.ok) { fprintf(stderr, "simulated arena exhausted\n"); exit(2); }
  void* p = g_heap + g.offset;
  if (g.lazy) lazy::note_zero_block(p, g.need);
  else if (g.zero_to > g.zero_from) { lazy::Scope s_; zero_bytes_async(g_heap + g.zero_from, g.zero_to - g.zero_from); }
  // the arena's own promise, checked where the simulation can see it at once: a block that was not put off reads zero now
  if (zero && !g.lazy) for (size_t i = 0; i < g.need; i++) if (((char*)p)[i] != 0) { fprintf(stderr, "lh_malloc handed out a block of %zu bytes at offset %zu that does not read zero (byte %zu)\n", g.need, g.offset, i); exit(1); }
  return p;
}
static void sim_rewind(size_t mark) {
  lazy::Scope s_;
  if (lazy::g_busy) lazy::on_rewind(g_heap + mark);
  memset(g_heap + mark, 0xCD, g_arena.bytes - mark);  // what is handed out again is full of garbage (the zero window above the old top included)
  if (!arena_rewind(g_arena, mark)) { fprintf(stderr, "bad mark\n"); exit(2); }
}
static void sim_pop(size_t bytes) {                   // lh_free_top: scratch taken from the top and given back
  const size_t need = arena_round(bytes);
  if (lazy::g_busy) { if (lazy::g_depth == 0) { LZ_ENTER(); } lazy::arena_released(g_heap + g_arena.top - need); }
  memset(g_heap + g_arena.top - need, 0xCD, g_arena.bytes - (g_arena.top - need));
  if (!arena_pop(g_arena, bytes)) { fprintf(stderr, "bad pop\n"); exit(2); }
}

// ---- simulated kernels: any deterministic functions will do, as long as a fused form computes what its parts compute ------
static const int N_ = 2, C_ = 4, HW_ = 24, NE = N_ * C_ * HW_;      // every activation: 192 floats = 768 bytes (a "large" block)
static inline int chan(int i) { return (i / HW_) % C_; }
static void k_conv(const float* x, const float* w, const float* bias, float* y) { for (int i = 0; i < NE; i++) { float a = bias ? bias[chan(i)] : 0.f; for (int k = 0; k < 3; k++) a += x[(i + 7 * k) % NE] * w[(chan(i) + k) % 12]; y[i] = a; } g_kernels++; }
static void k_conv_bwd_data(const float* dy, const float* w, float* dx, float beta) { for (int i = 0; i < NE; i++) { float a = 0.f; for (int k = 0; k < 3; k++) a += dy[(i + NE - 7 * k) % NE] * w[(chan((i + NE - 7 * k) % NE) + k) % 12]; dx[i] = (beta != 0.f ? dx[i] : 0.f) + a; } g_kernels++; }
static void k_conv_bwd_filter(const float* x, const float* dy, float* dw, float beta) { for (int j = 0; j < 12; j++) { float a = 0.f; for (int i = 0; i < NE; i++) for (int k = 0; k < 3; k++) if ((chan(i) + k) % 12 == j) a += dy[i] * x[(i + 7 * k) % NE]; dw[j] = (beta != 0.f ? dw[j] : 0.f) + a; } g_kernels++; }
namespace lh {
static void sim_conv_relu(const float* x, const float* w, const float* bias, float* y) { k_conv(x, sim_filter(w), bias, y); for (int i = 0; i < NE; i++) y[i] = y[i] < 0.f ? 0.f : y[i]; }
// bias gradient: channel sums of dy in element order; with y, dy is masked by y > 0 on the way (and written back)
static void sim_bias_grad(const float* y, float* dy, float* db) { for (int i = 0; i < NE; i++) { if (y) dy[i] = y[i] > 0.f ? dy[i] : 0.f; db[chan(i)] += dy[i]; } g_kernels++; }
}
static void k_stats(const float* x, float* sm, float* si, float* rm, float* rv) {
  for (int c = 0; c < C_; c++) {
    double s = 0, q = 0; int cnt = 0;
    for (int i = 0; i < NE; i++) if (chan(i) == c) { s += x[i]; q += (double)x[i] * x[i]; cnt++; }
    const double mean = s / cnt, var = q / cnt - mean * mean;
    sm[c] = (float)mean; si[c] = (float)(1.0 / sqrt((var > 0 ? var : 0) + 1e-5));
    if (rm) rm[c] = 0.9f * rm[c] + 0.1f * (float)mean;
    if (rv) rv[c] = 0.9f * rv[c] + 0.1f * (float)var;
  }
  g_kernels++;
}
static inline float affine(float v, float m, float is, float g, float b) { return g * ((v - m) * is) + b; }
static void k_apply(const float* x, const float* g, const float* b, const float* sm, const float* si, const float* shortcut, float* out, int relu) {
  for (int i = 0; i < NE; i++) { const int c = chan(i); float r = affine(x[i], sm[c], si[c], g[c], b[c]); if (shortcut) r += shortcut[i]; if (relu) r = r < 0.f ? 0.f : r; out[i] = r; }
  g_kernels++;
}
// the "batch-norm gradient" of the simulation: linear in the masked gradient m, with sums over the channel
static void k_bn_bwd(const float* x, const float* m, const float* g, const float* sm, const float* si, float* dx, float beta, float* dg, float* db) {
  for (int c = 0; c < C_; c++) {
    float s1 = 0.f, s2 = 0.f;
    for (int i = 0; i < NE; i++) if (chan(i) == c) { s1 += m[i]; s2 += m[i] * ((x[i] - sm[c]) * si[c]); }
    if (dx) for (int i = 0; i < NE; i++) if (chan(i) == c) dx[i] = (beta != 0.f ? dx[i] : 0.f) + g[c] * si[c] * (m[i] - s1 / (N_ * HW_) - ((x[i] - sm[c]) * si[c]) * s2 / (N_ * HW_));
    dg[c] += s2; db[c] += s1;
  }
  g_kernels++;
}

// ---- entry points with the library's names: the protocol of the real ones over the simulated kernels --------------------
#define SZ(n) ((size_t)(n) * 4)
extern "C" {
void lh_conv2d_fwd(const float* x, const float* w, const float* bias, float* y, int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW) {
  LZ_SCOPE();
  if (lazy::park_conv_fwd(x, w, bias, y, N, C, H, W, K, R, S, sH, sW, pH, pW)) return;
  if (lazy::g_busy && !lazy::g_replay) { lazy::flush_parked(); lazy::rd(x, SZ(NE)); lazy::rd(w, SZ(12)); lazy::rd(bias, SZ(C_)); lazy::wr(y, SZ(NE)); }
  (void)ordered_stream(); k_conv(x, sim_filter(w), bias, y);
}
void lh_bn_stats(const float* x, float* sm, float* si, float* rm, float* rv, int, int, int, float, float) {
  LZ_ENTER(); lazy::rd_f(x, NE); lazy::wr_f(sm, C_); lazy::wr_f(si, C_); lazy::rw_f(rm, C_); lazy::rw_f(rv, C_);
  (void)ordered_stream(); k_stats(x, sm, si, rm, rv);
}
void lh_bn_apply(const float* x, const float* g, const float* b, const float* sm, const float* si, float* y, int, int, int, int relu) {
  LZ_ENTER(); lazy::rd_f(x, NE); lazy::rd_f(g, C_); lazy::rd_f(b, C_); lazy::rd_f(sm, C_); lazy::rd_f(si, C_); lazy::out_f(y, NE, y == x);
  (void)ordered_stream(); k_apply(x, g, b, sm, si, nullptr, y, relu);
}
void lh_bn_apply_add_relu(const float* x, const float* g, const float* b, const float* sm, const float* si, const float* sc, float* out, int, int, int) {
  LZ_ENTER(); lazy::rd_f(x, NE); lazy::rd_f(sc, NE); lazy::rd_f(g, C_); lazy::rd_f(b, C_); lazy::rd_f(sm, C_); lazy::rd_f(si, C_); lazy::out_f(out, NE, out == x || out == sc);
  (void)ordered_stream(); k_apply(x, g, b, sm, si, sc, out, 1);
}
static void bn_fwd_now(bool relu, const float* x, const float* g, const float* b, float* rm, float* rv, float* y, float* sm, float* si) {
  if (lazy::g_busy && !lazy::g_replay) { lazy::flush_parked(); lazy::rd_f(x, NE); lazy::rd_f(g, C_); lazy::rd_f(b, C_); lazy::rw_f(rm, C_); lazy::rw_f(rv, C_); lazy::out_f(y, NE, y == x); lazy::wr_f(sm, C_); lazy::wr_f(si, C_); }
  (void)ordered_stream(); k_stats(x, sm, si, rm, rv); k_apply(x, g, b, sm, si, nullptr, y, relu);
}
void lh_bn_train_fwd(const float* x, const float* g, const float* b, float* rm, float* rv, float* y, float* sm, float* si, int N, int C, int HW, float eps, float factor) {
  LZ_SCOPE();
  if (lazy::park_bn_train_fwd(x, g, b, rm, rv, y, sm, si, N, C, HW, eps, factor)) return;
  bn_fwd_now(false, x, g, b, rm, rv, y, sm, si);
}
void lh_bn_train_fwd_relu(const float* x, const float* g, const float* b, float* rm, float* rv, float* y, float* sm, float* si, int, int, int, float, float) {
  LZ_SCOPE(); bn_fwd_now(true, x, g, b, rm, rv, y, sm, si);
}
void lh_conv2d_fwd_bn_apply(const float* x, const float* w, const float* bias, float* y, int, int, int, int, int, int, int, int, int, int, int,
                            const float* g, const float* b, float* sm, float* si, float* rm, float* rv, float, float, const float* sc, float* out, int relu) {
  LZ_SCOPE();
  if (lazy::g_busy && !lazy::g_replay) {
    lazy::flush_parked(); lazy::rd_f(x, NE); lazy::rd_f(w, 12); lazy::rd_f(bias, C_); lazy::wr_f(y, NE); lazy::rd_f(g, C_); lazy::rd_f(b, C_); lazy::rd_f(sc, NE);
    lazy::wr_f(sm, C_); lazy::wr_f(si, C_); lazy::rw_f(rm, C_); lazy::rw_f(rv, C_); lazy::wr_f(out, NE);
  }
  (void)ordered_stream(); k_conv(x, sim_filter(w), bias, y); k_stats(y, sm, si, rm, rv); k_apply(y, g, b, sm, si, sc, out, relu);
}
void lh_add_relu(const float* a, const float* b, float* out, int64_t n) {
  LZ_ENTER(); lazy::rd_f(a, n); lazy::rd_f(b, n); lazy::out_f(out, n, out == a || out == b);
  (void)ordered_stream(); for (int64_t i = 0; i < n; i++) { float r = a[i] + b[i]; out[i] = r < 0.f ? 0.f : r; } g_kernels++;
}
void lh_add_relu_grad(const float* y, const float* dy, float* ad, float abeta, float* bd, float bbeta, int64_t n) {
  LZ_ENTER(); lazy::rd_f(y, n); lazy::rd_f(dy, n);
  if (ad) abeta = lazy::beta_f(ad, n, abeta);
  if (bd && bd != ad) bbeta = lazy::beta_f(bd, n, bbeta);
  (void)ordered_stream();
  for (int64_t i = 0; i < n; i++) { const float g = y[i] > 0.f ? dy[i] : 0.f; if (ad) ad[i] = (abeta != 0.f ? ad[i] : 0.f) + g; if (bd) bd[i] = (bbeta != 0.f ? bd[i] : 0.f) + g; }
  g_kernels++;
}
static float bn_bwd_declare(const float* x, const float* y, const float* dy, const float* g, const float* bias, const float* sm, const float* si, float* dx, float beta, float* dg, float* db) {
  if (!lazy::g_busy || lazy::g_replay) return beta;
  lazy::flush_parked();
  lazy::rd_f(x, NE); lazy::rd_f(y, NE); lazy::rd_f(dy, NE); lazy::rd_f(g, C_); lazy::rd_f(bias, C_); lazy::rd_f(sm, C_); lazy::rd_f(si, C_);
  if (dx) beta = lazy::beta_f(dx, NE, beta);
  lazy::rw_f(dg, C_); lazy::rw_f(db, C_);
  return beta;
}
void lh_bn_bwd(const float* x, const float* dy, const float* g, const float* sm, const float* si, float* dx, float beta, float* dg, float* db, int N, int C, int HW) {
  LZ_SCOPE();
  if (lazy::g_busy && !lazy::g_replay && lazy::take_bn_bwd(x, dy, g, sm, si, dx, beta, dg, db, N, C, HW)) return;
  beta = bn_bwd_declare(x, nullptr, dy, g, nullptr, sm, si, dx, beta, dg, db);
  (void)ordered_stream(); k_bn_bwd(x, dy, g, sm, si, dx, beta, dg, db);
}
void lh_bn_bwd_relu(const float* x, const float* y, const float* dy, const float* g, const float* bias, const float* sm, const float* si, float* dx, float beta, float* dg, float* db, int, int, int) {
  LZ_SCOPE();
  beta = bn_bwd_declare(x, bias ? nullptr : y, dy, g, bias, sm, si, dx, beta, dg, db);
  (void)ordered_stream();
  std::vector<float> m(NE);
  for (int i = 0; i < NE; i++) { const int c = chan(i); const float yv = bias ? affine(x[i], sm[c], si[c], g[c], bias[c]) : y[i]; m[i] = yv > 0.f ? dy[i] : 0.f; }
  k_bn_bwd(x, m.data(), g, sm, si, dx, beta, dg, db);
}
void lh_bn_bwd_add_relu(const float* x, const float* out, float* dout, const float* g, const float* sm, const float* si, float* dx, float beta_dx, float* ds, float beta_ds,
                        float* dg, float* db, int, int, int) {
  LZ_SCOPE();
  if (lazy::g_busy && !lazy::g_replay) {
    lazy::flush_parked(); lazy::rd_f(x, NE); lazy::rd_f(out, NE); lazy::rw_f(dout, NE); lazy::rd_f(g, C_); lazy::rd_f(sm, C_); lazy::rd_f(si, C_);
    if (dx) beta_dx = lazy::beta_f(dx, NE, beta_dx);
    if (ds) beta_ds = lazy::beta_f(ds, NE, beta_ds);
    lazy::rw_f(dg, C_); lazy::rw_f(db, C_);
  }
  (void)ordered_stream();
  std::vector<float> m(NE);
  for (int i = 0; i < NE; i++) m[i] = out[i] > 0.f ? dout[i] : 0.f;
  if (ds) for (int i = 0; i < NE; i++) ds[i] = (beta_ds != 0.f ? ds[i] : 0.f) + m[i];
  if (ds == nullptr || beta_ds != 0.f) for (int i = 0; i < NE; i++) dout[i] = m[i];       // as the two-pass path of the library does; otherwise dout stays as it was
  k_bn_bwd(x, m.data(), g, sm, si, dx, beta_dx, dg, db);
}
}  // extern "C"

// trait-level calls that have no fused form of their own in lh_defer.hip
static void t_relu_inplace(float* y, int64_t n) {
  LZ_SCOPE();
  if (lazy::g_busy && !lazy::g_replay && lazy::take_relu_inplace(y, n)) return;
  if (lazy::g_busy && !lazy::g_replay) { lazy::flush_parked(); lazy::rw_f(y, n); }
  (void)ordered_stream(); for (int64_t i = 0; i < n; i++) y[i] = y[i] < 0.f ? 0.f : y[i]; g_kernels++;
}
static void t_add(const float* a, const float* b, float* out, int64_t n) {
  LZ_SCOPE();
  if (lazy::park_add(a, b, out, n)) return;
  if (lazy::g_busy && !lazy::g_replay) { lazy::flush_parked(); lazy::rd_f(a, n); lazy::rd_f(b, n); lazy::wr_f(out, n); }
  add_plain(a, b, out, n);
}
static void t_relu_grad_inplace(const float* y, float* d, int64_t n) {
  LZ_SCOPE();
  if (lazy::park_relu_grad_inplace(y, d, n)) return;
  if (lazy::g_busy && !lazy::g_replay) { lazy::flush_parked(); lazy::rd_f(y, n); lazy::rw_f(d, n); }
  relu_grad_inplace_now(y, d, n);
}
static void t_add_grad(float* ad, float* bd, const float* outd, int64_t n) {      // ad += outd; bd += outd
  LZ_SCOPE();
  if (lazy::g_busy && !lazy::g_replay && lazy::park_add_grad(ad, bd, outd, n)) return;
  bool af = false, bf = false;
  if (lazy::g_busy && !lazy::g_replay) { lazy::flush_parked(); lazy::rd_f(outd, n); if (ad) af = lazy::acc_f(ad, n); if (bd && bd != ad) bf = lazy::acc_f(bd, n); }
  (void)ordered_stream();
  if (ad) for (int64_t i = 0; i < n; i++) ad[i] = (af ? 0.f : ad[i]) + outd[i];
  if (bd) for (int64_t i = 0; i < n; i++) bd[i] = (bf ? 0.f : bd[i]) + outd[i];
  g_kernels++;
}
static void t_conv_bwd(const float* x, const float* dy, const float* w, float* dx, float* dw) {
  { LZ_ENTER(); lazy::rd_f(dy, NE); lazy::rd_f(w, 12); float beta = lazy::beta_f(dx, NE, 1.f); (void)ordered_stream(); k_conv_bwd_data(dy, sim_filter(w), dx, beta); }
  { LZ_ENTER(); lazy::rd_f(x, NE); lazy::rd_f(dy, NE); float beta = lazy::beta_f(dw, 12, 1.f); (void)ordered_stream(); k_conv_bwd_filter(x, dy, dw, beta); }
}
// a convolution with a bias: the filter gradient (bias sums included) goes first, as the backends issue it
static void t_conv_bwd_bias(const float* x, float* dy, const float* w, float* dx, float* dw, float* db) {
  { LZ_SCOPE();
    const bool done = lazy::g_busy && !lazy::g_replay && lazy::take_relu_grad_bias(dy, db, N_, C_, HW_);
    if (lazy::g_busy && !lazy::g_replay) lazy::flush_parked();
    lazy::rd_f(x, NE); lazy::rd_f(dy, NE); float beta = lazy::beta_f(dw, 12, 1.f); lazy::rw_f(db, C_);
    (void)ordered_stream(); k_conv_bwd_filter(x, dy, dw, beta); if (!done) sim_bias_grad(nullptr, dy, db); }
  if (dx) { LZ_ENTER(); lazy::rd_f(dy, NE); lazy::rd_f(w, 12); float beta = lazy::beta_f(dx, NE, 1.f); (void)ordered_stream(); k_conv_bwd_data(dy, sim_filter(w), dx, beta); }
}
static void t_momentum(float* x, float* d, float* v, float lr, float mu, float clip, int nesterov, int64_t n) {
  LZ_SCOPE();
  if (lazy::gather_update(1, x, d, v, lr, mu, clip, nesterov, n)) return;
  if (lazy::g_busy && !lazy::g_replay) { lazy::flush_parked(); lazy::forget_forward_records(); lazy::rw_f(x, n); lazy::rw_f(d, n); lazy::rw_f(v, n); }
  (void)ordered_stream(); k_update(1, x, d, v, lr, mu, clip, nesterov, n); g_kernels++;
}
static void t_geam(const float* x, float a, const float* y, float b, float* out, int64_t n) {
  LZ_ENTER(); lazy::rd_f(x, n); lazy::rd_f(y, n); lazy::out_f(out, n, out == x || out == y);
  (void)ordered_stream(); for (int64_t i = 0; i < n; i++) out[i] = x[i] * a + y[i] * b; g_kernels++;
}
static void t_fill(float* x, float v, int64_t n) { LZ_ENTER(); lazy::wr_f(x, n); (void)ordered_stream(); for (int64_t i = 0; i < n; i++) x[i] = v; g_kernels++; }
static void t_d2h(std::vector<float>& trace, const float* p, int64_t n) { LZ_ENTER(); lazy::rd(p, SZ(n)); (void)ordered_stream(); trace.insert(trace.end(), p, p + n); }
static void t_undeclared(float* p, int64_t n) { (void)ordered_stream(); for (int64_t i = 0; i < n; i++) p[i] = p[i] * 0.5f + 1.0f; g_kernels++; }     // an entry point that states nothing

// ---- random programs --------------------------------------------------------------------------------------------------------
static uint64_t g_rng;
static uint32_t rnd() { g_rng = g_rng * 6364136223846793005ull + 1442695040888963407ull; return (uint32_t)(g_rng >> 33); }
static int ri(int lo, int hi) { return lo + (int)(rnd() % (uint32_t)(hi - lo + 1)); }
static float rf() { return (float)((int)(rnd() % 2001) - 1000) / 500.0f; }

struct TR { float* x; float* d; };                 // a TensorR: value and gradient, both from the zero-filled arena
struct Layer { int kind; TR in, conv, bn, sc, out; float *w, *dw, *wv, *g, *dg, *gv, *b, *db, *bv, *rm, *rv, *sm, *si; bool relu, join, has_conv, nobn; };

static void run_program(uint64_t seed, bool enabled, std::vector<float>& trace, std::vector<char>& image, long long& kernels) {
  g_rng = seed;
  lazy::reset(); lazy::g_enabled = enabled; lazy::g_depth = 0;
  memset(g_heap, 0xCD, g_arena.bytes); { const size_t b = g_arena.bytes; g_arena = ArenaState(); g_arena.bytes = b; } g_kernels = 0;
  auto vec = [&](int n, bool random) { float* p = (float*)sim_malloc(SZ(n), true); if (random) { std::vector<float> h(n); for (auto& v : h) v = rf(); lazy::Scope s_; lazy::wr(p, SZ(n)); memcpy(p, h.data(), SZ(n)); } return p; };
  auto tr = [&](float* x) { TR t; t.x = x; t.d = (float*)sim_malloc(SZ(NE), true); return t; };
  // parameters below the mark (gradients and momentum buffers start as untouched zero blocks of their own)
  const int nlayers = ri(1, 5);
  std::vector<Layer> L(nlayers);
  for (auto& l : L) {
    l.w = vec(12, true); l.dw = vec(12, false); l.wv = vec(12, false);
    l.g = vec(C_, true); l.dg = vec(C_, false); l.gv = vec(C_, false); l.b = vec(C_, true); l.db = vec(C_, false); l.bv = vec(C_, false);
    l.rm = vec(C_, false); l.rv = vec(C_, false);
  }
  float* input = vec(NE, true);
  float* big_d = (float*)sim_malloc(SZ(NE), true);       // a parameter-like large block: its first gradient overwrites it
  const size_t mark = g_arena.top;
  const int steps = ri(1, 3);
  for (int step = 0; step < steps; step++) {
    // forward
    TR h; h.x = input; h.d = nullptr;
    for (auto& l : L) {
      l.in = h; l.has_conv = ri(0, 4) != 0; l.join = ri(0, 2) == 0 && h.d != nullptr; l.relu = l.join || ri(0, 3) != 0;
      l.nobn = ri(0, 3) == 0;
      if (l.nobn) {                 // conv + bias -> relu in place, no batch norm (networks of that kind)
        l.has_conv = true; l.join = false;
        float* y = (float*)sim_malloc(SZ(NE), true); lh_conv2d_fwd(h.x, l.w, l.b, y, N_, C_, 1, HW_, C_, 1, 1, 1, 1, 0, 0); l.conv = tr(y);
        if (ri(0, 9) == 0) t_d2h(trace, y, 5);
        if (ri(0, 11) == 0) { float* tmp = (float*)sim_malloc(SZ(NE), true); t_geam(y, 1.f, y, 0.f, tmp, NE); }
        if (l.relu) t_relu_inplace(y, NE);
        l.bn = l.conv; l.out = l.conv; h = l.conv;
        if (ri(0, 7) == 0) t_d2h(trace, y + ri(0, NE - 4), 4);
        continue;
      }
      const float* x = h.x;
      if (l.has_conv) { float* y = (float*)sim_malloc(SZ(NE), true); lh_conv2d_fwd(h.x, l.w, nullptr, y, N_, C_, 1, HW_, C_, 1, 1, 1, 1, 0, 0); l.conv = tr(y); x = y; }
      if (ri(0, 9) == 0) t_d2h(trace, x, 5);                                        // a read in between ends the chain
      float* t = (float*)sim_malloc(SZ(NE), true); l.sm = (float*)sim_malloc(SZ(C_), true); l.si = (float*)sim_malloc(SZ(C_), true);
      lh_bn_train_fwd(x, l.g, l.b, l.rm, l.rv, t, l.sm, l.si, N_, C_, HW_, 1e-5f, 0.1f);
      l.bn = tr(t);
      TR o = l.bn;
      if (l.join) {
        l.sc = ri(0, 3) == 0 ? (l.has_conv ? l.conv : h) : h;                        // mostly the block input; sometimes the batch norm's own input
        float* out = (float*)sim_malloc(SZ(NE), true);
        if (ri(0, 1)) t_add(l.bn.x, l.sc.x, out, NE); else t_add(l.sc.x, l.bn.x, out, NE);
        o = tr(out);
      }
      if (ri(0, 11) == 0) { float* tmp = (float*)sim_malloc(SZ(NE), true); t_geam(o.x, 1.f, o.x, 0.f, tmp, NE); }     // something else before the relu
      if (l.relu) t_relu_inplace(o.x, NE);
      l.out = o; h = o;
      if (ri(0, 7) == 0) t_d2h(trace, o.x + ri(0, NE - 4), 4);
    }
    // loss gradient, then the tape in reverse
    { std::vector<float> gsrc(NE); for (auto& v : gsrc) v = rf(); lazy::Scope s_; if (lazy::g_busy) lazy::flush_parked(); lazy::wr(h.d, SZ(NE)); memcpy(h.d, gsrc.data(), SZ(NE)); }
    for (int li = nlayers - 1; li >= 0; li--) {
      Layer& l = L[li];
      if (l.relu) t_relu_grad_inplace(l.out.x, l.out.d, NE);
      if (ri(0, 13) == 0) t_d2h(trace, l.out.d, 6);
      if (l.nobn) { t_conv_bwd_bias(l.in.x, l.conv.d, l.w, l.in.d, l.dw, l.db); continue; }
      if (l.join) t_add_grad(l.bn.d, l.sc.d, l.out.d, NE);
      const TR& bx = l.has_conv ? l.conv : l.in;
      lh_bn_bwd(bx.x, l.bn.d, l.g, l.sm, l.si, bx.d, 1.0f, l.dg, l.db, N_, C_, HW_);
      if (l.has_conv) {
        if (l.in.d) t_conv_bwd(l.in.x, l.conv.d, l.w, l.in.d, l.dw);
        else { LZ_ENTER(); lazy::rd_f(l.in.x, NE); lazy::rd_f(l.conv.d, NE); float beta = lazy::beta_f(l.dw, 12, 1.f); (void)ordered_stream(); k_conv_bwd_filter(l.in.x, l.conv.d, l.dw, beta); }
      }
      if (ri(0, 9) == 0) t_geam(big_d, 1.f, l.bn.x, 0.25f, big_d, NE);                // reads a batch norm's output that a join may not have stored
    }
    if (ri(0, 2) == 0) t_d2h(trace, L[0].dw, 12);                                      // the loss read-back of the reference's loop comes before the optimizer
    for (auto& l : L) {
      t_momentum(l.w, l.dw, l.wv, 0.05f, 0.9f, 1.0f, 0, 12);
      t_momentum(l.g, l.dg, l.gv, 0.05f, 0.9f, 1.0f, 0, C_);
      if (ri(0, 5) == 0) t_momentum(l.b, l.db, l.bv, 0.02f, 0.9f, 1.0f, 1, C_); else t_momentum(l.b, l.db, l.bv, 0.05f, 0.9f, 1.0f, 0, C_);
    }
    // now and then: reads of what the fused chains did not store, slices, an undeclared call, a fill over part of a block
    const int extras = ri(0, 4);
    for (int e = 0; e < extras; e++) {
      Layer& l = L[ri(0, nlayers - 1)];
      switch (ri(0, 9)) {
        case 7: t_geam(l.out.x, -1.f, l.out.x, 0.f, l.out.x, NE); t_d2h(trace, l.out.d, NE); break;       // in place over what a recipe still has to read (the relu mask)
        case 8: t_geam(l.out.d, 3.f, l.out.d, 0.f, l.out.d, NE); t_d2h(trace, l.bn.d, NE); break;         // in place over the gradient a recipe copies from
        case 0: t_d2h(trace, l.bn.x, NE); break;
        case 1: t_d2h(trace, l.bn.d + 3, 9); break;
        case 2: t_d2h(trace, l.out.d, NE); break;
        case 3: t_undeclared(l.out.x, 7); break;
        case 4: t_fill(l.bn.d + 8, 2.5f, 16); break;
        case 5: { float* z = (float*)sim_malloc(SZ(NE), true); t_geam(z + 4, 1.f, l.out.x, 1.f, z + 4, 20); t_d2h(trace, z, NE); break; }
        case 6: { float* z = (float*)sim_malloc(SZ(NE), true); t_d2h(trace, z + 10, 3); break; }
        default: {      // scratch from the top, used and popped; then small zero blocks out of the same memory
          float* sc = (float*)sim_malloc(SZ(NE), false); t_fill(sc, 9.f, NE); sim_pop(SZ(NE));
          float* z1 = (float*)sim_malloc(SZ(5), true); float* z2 = (float*)sim_malloc(SZ(40), true); float* z3 = (float*)sim_malloc(SZ(NE), true);
          t_d2h(trace, z1, 5); t_d2h(trace, z2, 40); t_geam(z3, 1.f, z2, 1.f, z3, 40); t_d2h(trace, z3 + 30, 20); break;
        }
      }
    }
    if (step + 1 < steps || ri(0, 1)) sim_rewind(mark);
  }
  { lazy::Scope s_; lazy::flush_all(); }
  image.assign(g_heap, g_heap + g_arena.top);
  kernels = g_kernels;
}

int main(int argc, char** argv) {
  const int programs = argc > 1 ? atoi(argv[1]) : 2000;
  const uint64_t seed0 = argc > 2 ? (uint64_t)atoll(argv[2]) : 1;
  g_arena.bytes = 4u << 20;
  lazy::g_layout_refresh_min = 1;           // (the library asks for eight stale copies before it uses the side stream; here every program has fewer)
  g_heap = (char*)aligned_alloc(256, g_arena.bytes);
  long long k_on = 0, k_off = 0, fused = 0;
  for (int p = 0; p < programs; p++) {
    std::vector<float> t_off, t_on; std::vector<char> i_off, i_on; long long a = 0, b = 0;
    run_program(seed0 * 1000003ull + p, false, t_off, i_off, a);
    const int64_t f0 = lazy::g_stat[lazy::ST_FUSED_FWD] + lazy::g_stat[lazy::ST_FUSED_BWD];
    run_program(seed0 * 1000003ull + p, true, t_on, i_on, b);
    fused += lazy::g_stat[lazy::ST_FUSED_FWD] + lazy::g_stat[lazy::ST_FUSED_BWD] - f0;
    k_off += a; k_on += b;
    if (t_off.size() != t_on.size() || (!t_off.empty() && memcmp(t_off.data(), t_on.data(), t_off.size() * 4) != 0)) {
      size_t i = 0; while (i < t_off.size() && i < t_on.size() && memcmp(&t_off[i], &t_on[i], 4) == 0) i++;
      fprintf(stderr, "program %d (seed %llu): read-back %zu differs: %g as issued, %g with deferred work\n", p, (unsigned long long)(seed0 * 1000003ull + p), i,
              i < t_off.size() ? t_off[i] : NAN, i < t_on.size() ? t_on[i] : NAN);
      return 1;
    }
    if (i_off.size() != i_on.size() || (!i_off.empty() && memcmp(i_off.data(), i_on.data(), i_off.size()) != 0)) {
      size_t i = 0; while (i < i_off.size() && i_off[i] == i_on[i]) i++;
      fprintf(stderr, "program %d (seed %llu): the arena differs at byte %zu of %zu after everything deferred was brought up to date\n", p,
              (unsigned long long)(seed0 * 1000003ull + p), i, i_off.size());
      return 1;
    }
  }
  printf("defer_check: %d programs identical with and without deferred work; %lld chains fused; simulated launches %lld as issued, %lld with deferred work\n",
         programs, fused, k_off, k_on);
  printf("filter copies: %lld made, %lld lookups served from a kept copy\n", g_layout_builds, (long long)lazy::g_stat[lazy::ST_LAYOUTS]);
  lazy::reset();
  free(g_heap);
  return 0;
}
