// Deferred work: what lets a program that issues ONE library call per method of Lantern's Backend trait
// (TensorDifferentiation.scala:137-379: conv2D_batch, batchNormTraining, relu(inPlace), `+`, their gradients, one
// momentum_update per parameter, every buffer from the zero-filled arena and every gradient accumulated) run the fused
// kernels a hand-fused call sequence would run.  The reference's generated code for ResNet (ONNXLib.scala:847-872) issues
// convBBP -> batchNorm -> relu(true) as three operator calls, NNModule.scala:296-303 one optimizer call per parameter, and
// TensorR allocates every gradient zero-filled at construction (TensorDifferentiation.scala:1509-1514).  Three mechanisms:
//
//  1. Parked launches.  conv2d_fwd, bn_train_fwd, a same-shape `+`, relu_grad(inPlace) and its following add_grad do not
//     launch when called: they wait for the next call.  If that call continues one of the known chains
//     (conv -> bn -> [+ shortcut] -> relu in place; relu_grad -> [add_grad] -> bn_bwd) the chain runs as its fused entry
//     point (lh_conv2d_fwd_bn_apply, lh_bn_train_fwd_relu, lh_add_relu, lh_bn_bwd_relu, lh_bn_bwd_add_relu); any other
//     call first launches what is parked, unfused.  lh_malloc, lh_malloc_uninit and lh_mark do not count as calls here.
//     Optimizer calls (lh_momentum, lh_sgd) with equal hyper-parameters are gathered into one multi-tensor launch.
//  2. Zero fills on demand.  A block of more than 16 KiB from lh_malloc is not cleared when handed out; it is noted.  An
//     entry point that overwrites the block drops the note; one that would add into it (beta = 1) overwrites instead;
//     anything that reads it gets it cleared first.  lh_rewind drops the notes of what it releases.
//  3. Unwritten results.  A fused chain leaves out stores nobody normally reads: the batch norm's own output under a
//     residual join, and the in-place masking of the gradient buffer by relu_grad.  Each is noted with the recipe that
//     produces it; a later read of the range (or a write to what the recipe reads) runs the recipe first.
//  4. Filter layouts.  The copies of a filter in the layouts the convolution kernels read are kept while nothing writes the
//     filter, and made again beside the next step's first kernels after the optimizer launch that does (see below).
//
// Entry points that state their operands (lazy::Scope, rd / wr / acc / rw) are served exactly; every other entry point
// reaches lh::ordered_stream() at depth 0, which brings all deferred work up to date before it enqueues anything.
// Apart from the memory of the filter copies (allocated when a filter is first seen, released with it), nothing here
// allocates device memory or waits for the device.
#include "lh_common.h"
#include <string.h>
#include <algorithm>
#include <vector>

namespace lh {
void side_wait_for_main();      // lh_runtime.hip
namespace lazy {

bool g_enabled = getenv("LH_NO_FUSION") == nullptr;
bool g_busy = false;
int g_depth = 0;
bool g_replay = false;
static int64_t g_stat[8];        // fused chains, gathered updates, zero fills avoided / done, recipes run (lh_fusion_stats)
enum { ST_FUSED_FWD, ST_FUSED_BWD, ST_GATHERED, ST_ZERO_SKIPPED, ST_ZERO_DONE, ST_RECIPES, ST_UNFUSED, ST_LAYOUTS };

static inline size_t round256(size_t b) { b = (b + 255) & ~(size_t)255; return b ? b : 256; }
static inline bool overlap(const char* a, size_t an, const char* b, size_t bn) { return a < b + bn && b < a + an; }
static inline bool covers(const char* a, size_t an, const char* b, size_t bn) { return a <= b && b + bn <= a + an; }

struct ZeroBlock { char* p; size_t bytes; };
static std::vector<ZeroBlock> g_zero;          // ascending addresses: the arena is a bump allocator

enum { V_MASK = 0, V_BN_OUT = 1 };
struct Unwritten {
  int kind; char* dst; size_t bytes;
  const float* src; const float* y; int64_t n;                                           // V_MASK: dst = y > 0 ? src : 0
  const float* x; const float* gamma; const float* beta; const float* sm; const float* si; int N, C, HW;   // V_BN_OUT: dst = bn(x)
};
static std::vector<Unwritten> g_unwritten;

struct FwdRecord { const float* y; const float* x; const float* bias; int64_t n; };   // y = relu(bn(x)) as the fused kernels compute it
static std::vector<FwdRecord> g_records;

struct ConvArgs { const float* x; const float* w; const float* bias; float* y; int N, C, H, W, K, R, S, sH, sW, pH, pW, P, Q; };
struct BnArgs { const float* x; const float* gamma; const float* beta; float* rm; float* rv; float* y; float* sm; float* si; int N, C, HW; float eps, factor; int64_t n; };
struct AddArgs { const float* a; const float* b; float* out; int64_t n; };
enum { P_NONE = 0, P_CONV, P_BN, P_ADD, P_RELU_GRAD, P_RELU_ADD_GRAD, P_UPDATE };
struct Parked {
  int kind = P_NONE;
  bool has_conv = false, has_add = false;
  ConvArgs conv; BnArgs bn; AddArgs add;
  const float* gy = nullptr; float* gd = nullptr; int64_t gn = 0;                         // relu_grad in place: gd masked by gy > 0
  float* ad = nullptr; float* bd = nullptr; bool a_fresh = false, b_fresh = false;       // the add_grad behind it
  int umode = 0; float lr = 0.f, mu = 0.f, clip = 0.f; int nesterov = 0;                  // gathered optimizer calls
  std::vector<float*> ux, ud, uv; std::vector<int64_t> un;
};
static Parked g_p;

static int g_layouts_valid_count();
static inline void refresh_busy() { g_busy = g_p.kind != P_NONE || !g_zero.empty() || !g_unwritten.empty() || g_layouts_valid_count() > 0; }
static inline bool can_park() { return g_enabled && !g_replay && g_stream_cur == g_stream_raw && !g_rec_on; }

// Launches made in a Replay's lifetime run as called (no parking, no declarations) and on the main stream; a side stream
// that is current waits for them.
struct Replay {
  bool saved_replay; hipStream_t saved_stream;
  Replay() : saved_replay(g_replay), saved_stream(g_stream_cur) { g_replay = true; g_depth++; g_stream_cur = g_stream_raw; }
  ~Replay() {
    g_stream_cur = saved_stream; g_depth--; g_replay = saved_replay;
    if (saved_stream != g_stream_raw) side_wait_for_main();
  }
};

// ---- filter layouts ---------------------------------------------------------------------------------------------------
// The convolution kernels read their filter in a layout of their own (tap-major for the forward pass, one transposed copy per
// residue class for the input gradient): a copy kernel per layer and pass, 5-7 us each in the chain of a training step.  A copy
// is kept in memory of its own for as long as nothing writes the filter: every stated write into the filter's range, every
// call that states nothing, a rewind or pop that releases the filter, ends it.  After the gathered optimizer launch, which is
// such a write, the copies that were in use are made again on the side stream, beside whatever the program does next; the
// convolution that needs one waits for the side stream then (lh::side_join) instead of making it itself.
struct Layout { const char* w; size_t wbytes; int kind; int prm[LAYOUT_PRM]; float* copy; size_t bytes; bool valid, used; };
static std::vector<Layout> g_layouts;
static int g_layouts_valid = 0;
static size_t g_layout_bytes = 0;
int g_layout_refresh_min = 8;                            // stale copies it takes for the side stream to be used (see layouts_refresh)
static bool g_layouts_on_side = false;                   // copies made on the side stream that the main stream has not waited for yet
static const size_t LAYOUT_CAP = (size_t)1 << 30;        // all copies together; filters beyond that are copied per call as before

static int g_layouts_valid_count() { return g_layouts_valid; }
static inline void layout_set(Layout& l, bool v) { if (l.valid != v) { l.valid = v; g_layouts_valid += v ? 1 : -1; } }
static void layouts_written(const char* lo, size_t nb) {
  if (g_layouts_valid == 0) return;
  for (auto& l : g_layouts) if (l.valid && overlap(lo, nb, l.w, l.wbytes)) layout_set(l, false);
}
static void layouts_all_stale() { if (g_layouts_valid) for (auto& l : g_layouts) layout_set(l, false); }
static void layouts_released(const char* from) {
  for (size_t i = 0; i < g_layouts.size();) {
    if (g_layouts[i].w + g_layouts[i].wbytes > from) {
      layout_set(g_layouts[i], false);
      g_layout_bytes -= g_layouts[i].bytes;
      persistent_free(g_layouts[i].copy);       // (waits for the device: only when a filter itself is released)
      g_layouts.erase(g_layouts.begin() + i);
    } else i++;
  }
}
static void layouts_drop() { layouts_released(nullptr); }

float* layout_lookup(const float* w, size_t wbytes, int kind, const int* prm, size_t bytes, bool& build) {
  build = false;
  if (!g_enabled || g_rec_on || g_capturing || g_prof_mask != 0 || g_stream_cur != g_stream_raw || w == nullptr) return nullptr;
  // Copies made on the side stream since the last lookup: the main stream waits for them once, whether it is about to read one
  // or to write one again (later lookups of the step must not wait for the filter gradients that run there by then).
  if (g_layouts_on_side) { side_join(); g_layouts_on_side = false; }
  for (auto& l : g_layouts) {
    if (l.w != (const char*)w || l.kind != kind || l.bytes != bytes || memcmp(l.prm, prm, sizeof l.prm) != 0) continue;
    l.used = true;
    if (l.valid) { g_stat[ST_LAYOUTS]++; return l.copy; }
    // stale: the caller makes it again, in stream order in front of its use, and it holds until the filter is written again
    layout_set(l, true); g_busy = true; build = true;
    return l.copy;
  }
  if (g_layout_bytes + bytes > LAYOUT_CAP) return nullptr;
  float* copy = (float*)persistent_alloc(bytes);
  if (copy == nullptr) return nullptr;
  Layout l{}; l.w = (const char*)w; l.wbytes = wbytes; l.kind = kind; memcpy(l.prm, prm, sizeof l.prm); l.copy = copy; l.bytes = bytes; l.valid = false; l.used = true;
  g_layouts.push_back(l);
  g_layout_bytes += bytes;
  layout_set(g_layouts.back(), true); g_busy = true; build = true;
  return copy;
}
// behind the optimizer launch: the copies the last step used, made again beside what comes next
static void layouts_refresh() {
  // Only where it pays: handing work to the second stream and waiting for it once costs a few tens of microseconds of
  // latency on both streams (LeNet's 0.26 ms step became 0.29 ms with its one copy made there, DeepSpeech2's 11.5 ms step
  // 12.8: its 1110 back-to-back step kernels are dispatched more slowly while the second queue is in use), which a handful
  // of 5 us copy kernels in the chain do not.  Networks with many filters to copy (8 or more) come out ahead.
  // Fewer than that (or no second stream to use): two or more are still made in one launch, here on the main stream, instead of
  // one launch each where they are next looked up.
  int stale = 0;
  for (auto& l : g_layouts) stale += (l.used && !l.valid) ? 1 : 0;
  const bool side = stale >= g_layout_refresh_min && side_work_begin();
  if (!side && (stale < 2 || g_rec_on || g_capturing || g_prof_mask != 0 || g_stream_cur != g_stream_raw)) return;
  std::vector<int> kinds; std::vector<const int*> prms; std::vector<const float*> ws; std::vector<float*> dsts;
  for (auto& l : g_layouts) {
    if (!l.used || l.valid) continue;
    kinds.push_back(l.kind); prms.push_back(l.prm); ws.push_back((const float*)l.w); dsts.push_back(l.copy);
    layout_set(l, true);
    l.used = false;
  }
  build_filter_layouts((int)kinds.size(), kinds.data(), prms.data(), ws.data(), dsts.data());
  if (side) { side_work_end(); g_layouts_on_side = true; }
}

// ---- zero blocks ---------------------------------------------------------------------------------------------------
void note_zero_block(void* p, size_t bytes) {
  g_zero.push_back({(char*)p, bytes});
  g_busy = true;
}
bool defer_zero() { return g_enabled && !g_rec_on && !g_replay; }

// indices [first, last) of the noted blocks that overlap [lo, hi)
static void zero_span(const char* lo, const char* hi, size_t& first, size_t& last) {
  auto it = std::upper_bound(g_zero.begin(), g_zero.end(), lo, [](const char* v, const ZeroBlock& b) { return v < b.p + b.bytes; });
  first = (size_t)(it - g_zero.begin());
  last = first;
  while (last < g_zero.size() && g_zero[last].p < hi) last++;
}
static void clear_blocks(size_t first, size_t last) {
  if (first >= last) return;
  Replay r_;
  for (size_t i = first; i < last; i++) { zero_bytes_async(g_zero[i].p, g_zero[i].bytes); g_stat[ST_ZERO_DONE]++; }
  g_zero.erase(g_zero.begin() + first, g_zero.begin() + last);
}

// ---- unwritten results -----------------------------------------------------------------------------------------------
static void produce(const Unwritten& v) {
  // what the recipe reads may itself be deferred
  if (v.kind == V_MASK) { rd(v.src, (size_t)v.n * 4); rd(v.y, (size_t)v.n * 4); }
  else { rd(v.x, (size_t)v.n * 4); }
  Replay r_;
  g_stat[ST_RECIPES]++;
  if (v.kind == V_MASK) mask_relu((float*)v.dst, v.src, v.y, v.n);
  else lh_bn_apply(v.x, v.gamma, v.beta, v.sm, v.si, (float*)v.dst, v.N, v.C, v.HW, 0);
}
static bool reads(const Unwritten& v, const char* lo, size_t nb) {
  if (v.kind == V_MASK) return overlap(lo, nb, (const char*)v.src, (size_t)v.n * 4) || overlap(lo, nb, (const char*)v.y, (size_t)v.n * 4);
  const size_t cb = (size_t)v.C * 4;
  return overlap(lo, nb, (const char*)v.x, (size_t)v.n * 4) || overlap(lo, nb, (const char*)v.gamma, cb) || overlap(lo, nb, (const char*)v.beta, cb) ||
         overlap(lo, nb, (const char*)v.sm, cb) || overlap(lo, nb, (const char*)v.si, cb);
}
// mode 0: the range is read; 1: overwritten as a whole; 2: read and written
static void settle_unwritten(const char* lo, size_t nb, int mode) {
  for (size_t i = 0; i < g_unwritten.size();) {
    const Unwritten& v = g_unwritten[i];
    const bool hit_dst = overlap(lo, nb, v.dst, v.bytes);
    if (mode == 1 && hit_dst && covers(lo, round256(nb), v.dst, v.bytes)) { g_unwritten.erase(g_unwritten.begin() + i); continue; }   // replaced before anyone saw it
    if (hit_dst || (mode != 0 && reads(v, lo, nb))) {
      const Unwritten copy = v;
      g_unwritten.erase(g_unwritten.begin() + i);
      produce(copy);
      i = 0;                        // producing may have settled others
      continue;
    }
    i++;
  }
}

void rd(const void* p, size_t bytes) {
  if (!g_busy || g_replay || p == nullptr || bytes == 0) return;
  const char* lo = (const char*)p;
  size_t a, b; zero_span(lo, lo + bytes, a, b); clear_blocks(a, b);
  if (!g_unwritten.empty()) settle_unwritten(lo, bytes, 0);
  refresh_busy();
}
void wr(const void* p, size_t bytes) {
  if (!g_busy || g_replay || p == nullptr || bytes == 0) return;
  const char* lo = (const char*)p;
  layouts_written(lo, bytes);
  size_t a, b; zero_span(lo, lo + bytes, a, b);
  // blocks the write covers need no clearing; a block it only touches is cleared first
  while (a < b) {
    if (covers(lo, round256(bytes), g_zero[a].p, g_zero[a].bytes)) { g_zero.erase(g_zero.begin() + a); b--; g_stat[ST_ZERO_SKIPPED]++; }
    else { clear_blocks(a, a + 1); b--; }
  }
  if (!g_unwritten.empty()) settle_unwritten(lo, bytes, 1);
  refresh_busy();
}
void rw(const void* p, size_t bytes) {
  if (!g_busy || g_replay || p == nullptr || bytes == 0) return;
  const char* lo = (const char*)p;
  layouts_written(lo, bytes);
  size_t a, b; zero_span(lo, lo + bytes, a, b); clear_blocks(a, b);
  if (!g_unwritten.empty()) settle_unwritten(lo, bytes, 2);
  refresh_busy();
}
bool acc(const void* p, size_t bytes) {
  if (!g_busy || g_replay || p == nullptr || bytes == 0) return false;
  const char* lo = (const char*)p;
  layouts_written(lo, bytes);
  size_t a, b; zero_span(lo, lo + bytes, a, b);
  if (b == a + 1 && g_zero[a].p == lo && g_zero[a].bytes == round256(bytes)) {       // the whole block, still untouched: overwrite it
    g_zero.erase(g_zero.begin() + a);
    g_stat[ST_ZERO_SKIPPED]++;
    refresh_busy();
    return true;
  }
  clear_blocks(a, b);
  if (!g_unwritten.empty()) settle_unwritten(lo, bytes, 2);
  refresh_busy();
  return false;
}

// ---- parked launches ---------------------------------------------------------------------------------------------------
static void launch_bn_chain(const Parked& p, int relu, const float* shortcut, float* out) {
  const BnArgs& b = p.bn;
  if (p.has_conv) {
    const ConvArgs& c = p.conv;
    lh_conv2d_fwd_bn_apply(c.x, c.w, c.bias, c.y, c.N, c.C, c.H, c.W, c.K, c.R, c.S, c.sH, c.sW, c.pH, c.pW,
                           b.gamma, b.beta, b.sm, b.si, b.rm, b.rv, b.eps, b.factor, shortcut, out, relu);
  } else if (shortcut) {
    lh_bn_stats(b.x, b.sm, b.si, b.rm, b.rv, b.N, b.C, b.HW, b.eps, b.factor);
    lh_bn_apply_add_relu(b.x, b.gamma, b.beta, b.sm, b.si, shortcut, out, b.N, b.C, b.HW);
  } else if (relu) {
    lh_bn_train_fwd_relu(b.x, b.gamma, b.beta, b.rm, b.rv, out, b.sm, b.si, b.N, b.C, b.HW, b.eps, b.factor);
  } else {
    lh_bn_train_fwd(b.x, b.gamma, b.beta, b.rm, b.rv, out, b.sm, b.si, b.N, b.C, b.HW, b.eps, b.factor);
  }
}
static void note_mask(float* dst, const float* src, const float* y, int64_t n) {
  Unwritten v{}; v.kind = V_MASK; v.dst = (char*)dst; v.bytes = (size_t)n * 4; v.src = src; v.y = y; v.n = n;
  g_unwritten.push_back(v);
}

void flush_parked() {
  if (g_p.kind == P_NONE) return;
  Parked p = std::move(g_p);
  g_p = Parked();
  if (p.kind == P_UPDATE) {
    // stated now, not when the calls were gathered: a rewind in between has released what depended on the old parameter values
    for (size_t i = 0; i < p.ux.size(); i++) {
      rw(p.ux[i], (size_t)p.un[i] * 4); rw(p.ud[i], (size_t)p.un[i] * 4);
      if (p.uv[i]) rw(p.uv[i], (size_t)p.un[i] * 4);
    }
  }
  {
    Replay r_;
    switch (p.kind) {
      case P_CONV: {
        const ConvArgs& c = p.conv;
        lh_conv2d_fwd(c.x, c.w, c.bias, c.y, c.N, c.C, c.H, c.W, c.K, c.R, c.S, c.sH, c.sW, c.pH, c.pW);
        break;
      }
      case P_BN:
        launch_bn_chain(p, 0, nullptr, p.bn.y);
        if (p.has_add) add_plain(p.add.a, p.add.b, p.add.out, p.add.n);
        if (p.has_conv || p.has_add) g_stat[ST_UNFUSED]++;
        break;
      case P_ADD: add_plain(p.add.a, p.add.b, p.add.out, p.add.n); break;
      case P_RELU_GRAD: relu_grad_inplace_now(p.gy, p.gd, p.gn); break;
      case P_RELU_ADD_GRAD:
        if (p.ad || p.bd) lh_add_relu_grad(p.gy, p.gd, p.ad, p.a_fresh ? 0.f : 1.f, p.bd, p.b_fresh ? 0.f : 1.f, p.gn);
        break;
      case P_UPDATE:
        multi_update_now(p.umode, (int)p.ux.size(), p.ux.data(), p.ud.data(), p.umode ? p.uv.data() : nullptr, p.un.data(), p.lr, p.mu, p.clip, p.nesterov);
        g_stat[ST_GATHERED] += (int64_t)p.ux.size();
        break;
    }
  }
  if (p.kind == P_UPDATE) layouts_refresh();
  if (p.kind == P_RELU_ADD_GRAD) note_mask(p.gd, p.gd, p.gy, p.gn);      // relu_grad(inPlace) leaves its gradient buffer masked; nobody has done that yet
  refresh_busy();
}

void flush_all() {
  flush_parked();
  while (!g_unwritten.empty()) {
    const Unwritten v = g_unwritten.back();
    g_unwritten.pop_back();
    produce(v);
  }
  clear_blocks(0, g_zero.size());
  refresh_busy();
}
void flush_undeclared() { Scope s_; flush_all(); layouts_all_stale(); refresh_busy(); }   // whoever states nothing may have written anything

static bool conv_shape_ok(int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW, int& P, int& Q) {
  if (N <= 0 || C <= 0 || H <= 0 || W <= 0 || K <= 0 || R <= 0 || S <= 0 || sH <= 0 || sW <= 0 || pH < 0 || pW < 0) return false;
  if (H + 2 * pH < R || W + 2 * pW < S) return false;
  P = (H + 2 * pH - R) / sH + 1; Q = (W + 2 * pW - S) / sW + 1;
  const double lim = 2147483647.0 / 4.0;
  return (double)N * C * H * W < lim && (double)N * K * P * Q < lim && (double)K * C * R * S < lim;
}

bool park_conv_fwd(const float* x, const float* w, const float* bias, float* y, int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW) {
  int P = 0, Q = 0;
  if (!can_park() || !x || !w || !y || !conv_shape_ok(N, C, H, W, K, R, S, sH, sW, pH, pW, P, Q)) return false;
  flush_parked();
  rd(x, (size_t)N * C * H * W * 4); rd(w, (size_t)K * C * R * S * 4); if (bias) rd(bias, (size_t)K * 4);
  wr(y, (size_t)N * K * P * Q * 4);
  g_p.kind = P_CONV; g_p.has_conv = true; g_p.has_add = false;
  g_p.conv = {x, w, bias, y, N, C, H, W, K, R, S, sH, sW, pH, pW, P, Q};
  g_busy = true;
  return true;
}

bool park_bn_train_fwd(const float* x, const float* gamma, const float* beta, float* rm, float* rv, float* y, float* sm, float* si,
                       int N, int C, int HW, float eps, float factor) {
  if (!can_park() || !x || !gamma || !beta || !y || !sm || !si || N <= 0 || C <= 0 || HW <= 0 || y == x || C > 65536) return false;
  const int64_t n = (int64_t)N * C * HW;
  if (n * 4 > 2147483647LL) return false;
  const bool behind_conv = g_p.kind == P_CONV && g_p.conv.y == x && g_p.conv.N == N && g_p.conv.K == C && (int64_t)g_p.conv.P * g_p.conv.Q == HW;
  if (!behind_conv) { flush_parked(); rd(x, (size_t)n * 4); g_p.has_conv = false; }
  rd(gamma, (size_t)C * 4); rd(beta, (size_t)C * 4);
  if (rm) rw(rm, (size_t)C * 4);
  if (rv) rw(rv, (size_t)C * 4);
  wr(y, (size_t)n * 4); wr(sm, (size_t)C * 4); wr(si, (size_t)C * 4);
  g_p.kind = P_BN; g_p.has_add = false;
  g_p.bn = {x, gamma, beta, rm, rv, y, sm, si, N, C, HW, eps, factor, n};
  g_busy = true;
  return true;
}

bool park_add(const float* a, const float* b, float* out, int64_t n) {
  if (!can_park() || !a || !b || !out || n <= 0 || out == a || out == b) return false;
  if (g_p.kind == P_BN && !g_p.has_add && a != b && n == g_p.bn.n && (g_p.bn.y == a || g_p.bn.y == b)) {
    const float* other = g_p.bn.y == a ? b : a;
    // relu(bn(h) + h): the fused backward would have one buffer for both of its gradients; that join stays unfused
    if (other != g_p.bn.x && !overlap((const char*)other, (size_t)n * 4, (const char*)out, (size_t)n * 4)) {
      rd(other, (size_t)n * 4); wr(out, (size_t)n * 4);
      g_p.has_add = true; g_p.add = {a, b, out, n};
      return true;
    }
  }
  flush_parked();
  rd(a, (size_t)n * 4); rd(b, (size_t)n * 4); wr(out, (size_t)n * 4);
  g_p.kind = P_ADD; g_p.has_conv = false; g_p.has_add = true; g_p.add = {a, b, out, n};
  g_busy = true;
  return true;
}

bool take_relu_inplace(float* y, int64_t n) {
  if (g_p.kind == P_CONV && g_p.conv.y == y && (int64_t)g_p.conv.N * g_p.conv.K * g_p.conv.P * g_p.conv.Q == n) {
    Parked p = std::move(g_p); g_p = Parked();
    const ConvArgs& c = p.conv;
    { Replay r_; conv2d_fwd_relu_now(c.x, c.w, c.bias, c.y, c.N, c.C, c.H, c.W, c.K, c.R, c.S, c.sH, c.sW, c.pH, c.pW); }
    g_stat[ST_FUSED_FWD]++;
    refresh_busy();
    return true;
  }
  if (g_p.kind == P_BN && !g_p.has_add && g_p.bn.y == y && g_p.bn.n == n) {
    Parked p = std::move(g_p); g_p = Parked();
    { Replay r_; launch_bn_chain(p, 1, nullptr, y); }
    g_records.push_back({y, p.bn.x, p.bn.beta, n});
    g_stat[ST_FUSED_FWD]++;
    refresh_busy();
    return true;
  }
  if (g_p.kind == P_BN && g_p.has_add && g_p.add.out == y && g_p.add.n == n) {
    Parked p = std::move(g_p); g_p = Parked();
    const float* other = p.bn.y == p.add.a ? p.add.b : p.add.a;
    { Replay r_; launch_bn_chain(p, 1, other, y); }
    // the batch norm's own output was never stored
    Unwritten v{}; v.kind = V_BN_OUT; v.dst = (char*)p.bn.y; v.bytes = (size_t)n * 4; v.n = n;
    v.x = p.bn.x; v.gamma = p.bn.gamma; v.beta = p.bn.beta; v.sm = p.bn.sm; v.si = p.bn.si; v.N = p.bn.N; v.C = p.bn.C; v.HW = p.bn.HW;
    g_unwritten.push_back(v);
    g_stat[ST_FUSED_FWD]++;
    refresh_busy();
    return true;
  }
  if (g_p.kind == P_ADD && g_p.add.out == y && g_p.add.n == n) {
    Parked p = std::move(g_p); g_p = Parked();
    { Replay r_; lh_add_relu(p.add.a, p.add.b, p.add.out, n); }
    g_stat[ST_FUSED_FWD]++;
    refresh_busy();
    return true;
  }
  return false;
}

bool park_relu_grad_inplace(const float* y, float* d, int64_t n) {
  if (!can_park() || !y || !d || n <= 0 || (const float*)d == y) return false;
  flush_parked();
  rd(y, (size_t)n * 4); rw(d, (size_t)n * 4);
  g_p.kind = P_RELU_GRAD; g_p.gy = y; g_p.gd = d; g_p.gn = n; g_p.ad = g_p.bd = nullptr;
  g_busy = true;
  return true;
}

// A convolution's bias gradient asked for while relu_grad(in place) on the same output gradient is parked: one pass masks
// the gradient and sums it per channel.
bool take_relu_grad_bias(const float* dy, float* db, int N, int K, int PQ) {
  if (g_p.kind != P_RELU_GRAD || (const float*)g_p.gd != dy || g_p.gn != (int64_t)N * K * PQ || !db) return false;
  if (overlap((const char*)db, (size_t)K * 4, (const char*)g_p.gd, (size_t)g_p.gn * 4) || overlap((const char*)db, (size_t)K * 4, (const char*)g_p.gy, (size_t)g_p.gn * 4)) return false;
  Parked p = std::move(g_p); g_p = Parked();
  rw(db, (size_t)K * 4);
  { Replay r_; conv_bwd_bias_mask_now(p.gy, p.gd, db, N, K, PQ); }
  g_stat[ST_FUSED_BWD]++;
  refresh_busy();
  return true;
}

bool park_add_grad(float* ad, float* bd, const float* outd, int64_t n) {
  if (g_p.kind != P_RELU_GRAD || g_p.gd != outd || g_p.gn != n) return false;
  if ((ad && ad == bd) || ad == outd || bd == outd) return false;
  g_p.kind = P_RELU_ADD_GRAD; g_p.ad = ad; g_p.bd = bd;
  g_p.a_fresh = ad ? acc(ad, (size_t)n * 4) : false;
  g_p.b_fresh = bd ? acc(bd, (size_t)n * 4) : false;
  g_busy = true;
  return true;
}

bool take_bn_bwd(const float* x, const float* dy, const float* gamma, const float* sm, const float* si,
                 float* dx, float beta_dx, float* dgamma, float* dbeta, int N, int C, int HW) {
  const int64_t n = (int64_t)N * C * HW;
  if (g_p.kind != P_RELU_GRAD && g_p.kind != P_RELU_ADD_GRAD) return false;
  if (g_p.gn != n || !x || !dy || (beta_dx != 0.f && beta_dx != 1.f) || N <= 0 || C <= 0 || HW <= 0 || C > 65536) return false;
  if (g_p.kind == P_RELU_GRAD) {
    if (g_p.gd != dy || dx == dy) return false;
    Parked p = std::move(g_p); g_p = Parked();
    rd(x, (size_t)n * 4); rd(gamma, (size_t)C * 4); rd(sm, (size_t)C * 4); rd(si, (size_t)C * 4);
    if (dx) { if (beta_dx != 0.f) { if (acc(dx, (size_t)n * 4)) beta_dx = 0.f; } else wr(dx, (size_t)n * 4); }
    rw(dgamma, (size_t)C * 4); rw(dbeta, (size_t)C * 4);
    const float* bias = nullptr;
    for (const FwdRecord& r : g_records) if (r.y == p.gy && r.x == x && r.n == n) { bias = r.bias; break; }
    { Replay r_; lh_bn_bwd_relu(x, p.gy, dy, gamma, bias, sm, si, dx, beta_dx, dgamma, dbeta, N, C, HW); }
    note_mask(p.gd, p.gd, p.gy, n);
    g_stat[ST_FUSED_BWD]++;
    refresh_busy();
    return true;
  }
  // relu_grad -> add_grad -> this: the gradient this layer's output received is exactly the masked one (its buffer was untouched)
  const bool via_a = g_p.ad && dy == g_p.ad && g_p.a_fresh, via_b = g_p.bd && dy == g_p.bd && g_p.b_fresh;
  if (!via_a && !via_b) return false;
  float* ds = via_a ? g_p.bd : g_p.ad;
  const bool ds_fresh = via_a ? g_p.b_fresh : g_p.a_fresh;
  if (dx && (dx == ds || dx == g_p.gd || (const float*)dx == dy)) return false;
  Parked p = std::move(g_p); g_p = Parked();
  rd(x, (size_t)n * 4); rd(gamma, (size_t)C * 4); rd(sm, (size_t)C * 4); rd(si, (size_t)C * 4);
  if (dx) { if (beta_dx != 0.f) { if (acc(dx, (size_t)n * 4)) beta_dx = 0.f; } else wr(dx, (size_t)n * 4); }
  rw(dgamma, (size_t)C * 4); rw(dbeta, (size_t)C * 4);
  { Replay r_; lh_bn_bwd_add_relu(x, p.gy, p.gd, gamma, sm, si, dx, beta_dx, ds, ds_fresh ? 0.f : 1.f, dgamma, dbeta, N, C, HW); }
  note_mask((float*)dy, p.gd, p.gy, n);         // the absorbed gradient buffer: never stored
  note_mask(p.gd, p.gd, p.gy, n);               // relu_grad's in-place masking (done already on some paths; masking twice changes nothing)
  g_stat[ST_FUSED_BWD]++;
  refresh_busy();
  return true;
}

bool gather_update(int mode, float* x, float* d, float* v, float lr, float mu, float clip, int nesterov, int64_t n) {
  if (!can_park() || n <= 0) return false;
  if (g_p.kind != P_UPDATE || g_p.umode != mode || g_p.lr != lr || g_p.mu != mu || g_p.clip != clip || g_p.nesterov != nesterov || g_p.ux.size() >= 4096) {
    flush_parked();
    g_p.kind = P_UPDATE; g_p.umode = mode; g_p.lr = lr; g_p.mu = mu; g_p.clip = clip; g_p.nesterov = nesterov;
    g_records.clear();                           // parameters change: the bias a backward pass would recompute a relu mask from is no longer the forward pass's
  }
  g_p.ux.push_back(x); g_p.ud.push_back(d); g_p.uv.push_back(v); g_p.un.push_back(n);
  g_busy = true;
  return true;
}
void forget_forward_records() { g_records.clear(); }
void reset() { g_p = Parked(); g_zero.clear(); g_unwritten.clear(); g_records.clear(); layouts_drop(); g_busy = false; g_replay = false; }

void arena_released(char* from) {
  if (!g_layouts.empty()) layouts_released(from);
  while (!g_zero.empty() && g_zero.back().p >= from) g_zero.pop_back();
  for (size_t i = 0; i < g_unwritten.size();) {
    if (g_unwritten[i].dst >= from) g_unwritten.erase(g_unwritten.begin() + i); else i++;
  }
  for (size_t i = 0; i < g_records.size();) {
    if ((const char*)g_records[i].y >= from) g_records.erase(g_records.begin() + i); else i++;
  }
  refresh_busy();
}

void on_rewind(char* new_top) {
  // A gathered optimizer batch whose tensors all lie below the new top stays parked across the rewind: launched first, it
  // would have to produce every unwritten batch-norm output that depends on the parameters it changes, for nobody to read.
  bool keep = g_p.kind == P_UPDATE;
  if (keep) for (size_t i = 0; i < g_p.ux.size(); i++) {
    if ((char*)g_p.ux[i] >= new_top || (char*)g_p.ud[i] >= new_top || (g_p.uv[i] && (char*)g_p.uv[i] >= new_top)) { keep = false; break; }
  }
  if (!keep) flush_parked();
  arena_released(new_top);
  // a result kept below the new top whose recipe reads released memory is produced now
  for (size_t i = 0; i < g_unwritten.size();) {
    const Unwritten& v = g_unwritten[i];
    const bool dangling = v.kind == V_MASK ? ((const char*)v.src >= new_top || (const char*)v.y >= new_top)
                                           : ((const char*)v.x >= new_top || (const char*)v.sm >= new_top || (const char*)v.si >= new_top);
    if (dangling) { const Unwritten copy = v; g_unwritten.erase(g_unwritten.begin() + i); produce(copy); i = 0; } else i++;
  }
  refresh_busy();
}

}  // namespace lazy
}  // namespace lh

using namespace lh;

extern "C" {
void lh_set_fusion(int on) {
  lazy::Scope s_;
  lazy::flush_all();
  lazy::layouts_all_stale();
  lazy::refresh_busy();
  lazy::g_enabled = on != 0;
}
int lh_get_fusion(void) { return lazy::g_enabled ? 1 : 0; }
void lh_flush_deferred(void) { lazy::Scope s_; lazy::flush_all(); }
void lh_fusion_stats(int64_t* h_out, int n) {
  for (int i = 0; i < n; i++) h_out[i] = i < 8 ? lazy::g_stat[i] : 0;
}
}
