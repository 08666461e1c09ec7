// Record-time analysis of a command-list buffer: which byte ranges each command reads and writes, which earlier commands of
// the buffer it therefore has to follow, and the level (and chain) it gets.  Host code only, no device headers: the library
// includes it (lh_cmdlist.hip), and tests/host_cpp/levels_check.cpp builds it with the address and undefined-behaviour
// sanitizers and checks its levels against a brute-force comparison of every pair of commands.
#pragma once
#include <stdint.h>
#include "lh_cmd.h"
using namespace lh;

// ---- dependence levels of the commands in the buffer being recorded ------------------------------------------------------------
namespace {
struct Extent { uintptr_t s, e; bool w; };            // a byte range a command reads (w = false) or writes / updates (w = true)

// The byte ranges a command touches.  Returns how many of o[0..3] are filled.
static int cmd_extents(const LhCmd& c, Extent* o) {
  int k = 0;
  auto add = [&](const void* p, int64_t bytes, bool w) { if (p && bytes > 0) { o[k].s = (uintptr_t)p; o[k].e = (uintptr_t)p + (uintptr_t)bytes; o[k].w = w; k++; } };
  const int64_t n4 = (int64_t)c.i0 * 4;
  switch (c.op) {
    case CL_ZERO16: add(c.p0, (int64_t)c.i0 * 16, true); break;
    case CL_FILL: add(c.p0, n4, true); break;
    case CL_COPY: case CL_SCALAR: case CL_UNARY: add(c.p0, n4, true); add(c.p1, n4, false); break;
    case CL_GEAM: case CL_BIN: case CL_ACC: case CL_ACCNEG: case CL_ACCMUL: add(c.p0, n4, true); add(c.p1, n4, false); add(c.p2, n4, false); break;
    case CL_UNARY_GRAD: add(c.p0, n4, true); add(c.p1, n4, false); add(c.p2, n4, false); add(c.p3, n4, false); break;
    case CL_GEMV_N: add(c.p0, n4, true); add(c.p1, ((int64_t)(c.i0 - 1) * c.i2 + c.i1) * 4, false); add(c.p2, (int64_t)c.i1 * 4, false); break;
    case CL_GEMV_T: add(c.p0, (int64_t)c.i1 * 4, true); add(c.p1, ((int64_t)(c.i0 - 1) * c.i2 + c.i1) * 4, false); add(c.p2, n4, false); break;
    case CL_GER: add(c.p0, (int64_t)c.i0 * c.i1 * 4, true); add(c.p1, n4, false); add(c.p2, (int64_t)c.i1 * 4, false); break;
    case CL_DOT: add(c.p0, 4, true); add(c.p1, n4, false); add(c.p2, n4, false); break;
    case CL_AXPY_DEV: add(c.p0, n4, true); add(c.p1, 4, false); add(c.p2, n4, false); break;
    case CL_SOFTMAX: add(c.p0, n4 * c.i1, true); add(c.p1, n4 * c.i1, false); break;
    case CL_SOFTMAX_GRAD: add(c.p0, n4 * c.i1, true); add(c.p1, n4 * c.i1, false); add(c.p2, n4 * c.i1, false); break;
    case CL_NLL: add(c.p0, n4, true); add(c.p1, n4 * c.i1, false); add(c.p2, n4, false); break;
    case CL_NLL_GRAD: add(c.p0, n4 * c.i1, true); add(c.p1, n4, false); add(c.p2, n4, false); break;
    case CL_ADAGRAD: add(c.p0, n4, true); add(c.p1, n4, true); add(c.p2, n4, true); break;
    case CL_SGD: add(c.p0, n4, true); add(c.p1, n4, true); break;
    default: break;
  }
  return k;
}
// How many wavefronts of work a command is (where the next command of its level should start).
// Element i of every operand is handled by lane i mod 1024 (see "Chains" below).
static bool cmd_lanewise(const LhCmd& c) {
  switch (c.op) {
    case CL_FILL: case CL_COPY: case CL_GEAM: case CL_SCALAR: case CL_BIN: case CL_ACC: case CL_ACCNEG: case CL_ACCMUL:
    case CL_UNARY: case CL_UNARY_GRAD: case CL_ADAGRAD: case CL_SGD: return true;
    default: return false;
  }
}
// How a command maps what it writes onto wavefronts: 1 element-wise (element i: thread i mod 1024), 2 rows of a matrix-vector
// product (ten to a wavefront), 3 columns of a transposed product (eight to a wavefront), 4 rows of a rank-1 update (five to a
// wavefront), 5 element-wise over the wavefronts of all workgroups (a parameter update over a whole weight matrix: one compute unit
// alone would draw it at 25 GB/s); 0: none of these.
constexpr int WIDE_ELEMS = 4096;          // element-wise commands from this size on are shared by the wavefronts of all workgroups
static int cmd_class(const LhCmd& c) {
  if (cmd_lanewise(c)) return c.i0 >= WIDE_ELEMS ? 5 : 1;
  return c.op == CL_GEMV_N ? 2 : c.op == CL_GEMV_T ? 3 : c.op == CL_GER ? 4 : 0;
}
static bool cmd_splits(const LhCmd& c) {
  return c.op == CL_GEMV_N || c.op == CL_GER || c.op == CL_GEMV_T || (cmd_lanewise(c) && c.i0 >= WIDE_ELEMS) || (c.op == CL_ZERO16 && c.i0 >= WIDE_ELEMS / 4);
}
static int cmd_waves(const LhCmd& c) {
  switch (c.op) {
    case CL_GEMV_N: return (c.i0 + 9) / 10;
    case CL_GEMV_T: return (c.i1 + 7) / 8;
    case CL_GER: return (c.i0 + 4) / 5;
    case CL_SOFTMAX: case CL_SOFTMAX_GRAD: return c.i0;
    default: return (c.i0 + 63) / 64;
  }
}

// Ranges of up to SMALL_BYTES are tracked per 256-byte block in a hash table (arena blocks are 256-byte aligned, so two
// buffers share a block only when one lies inside the other's allocation: then the dependence is real or harmless);
// larger ranges (matrices, zero fills) in a short table of distinct ranges.  A level is a uint16: 1 + highest level touched.
constexpr uintptr_t SMALL_BYTES = 4096;
constexpr int HASH_N = 8192, BIG_N = 96, PAGE_N = 16384, PAGE_SCAN_MAX = 512;
// Chains.  An element-wise command gives element i of every operand to the same lane (thread i mod 1024 of the workgroup and
// wavefront rotation it runs on).  If everything such a command must follow at the highest level L is ONE chain of element-wise
// commands, through ranges that start at the very addresses this command's operands start at, then each lane only ever needs what
// it read or wrote itself, program order within the lane is enough, and the command joins that chain AT level L (same workgroup,
// same rotation, recording order) instead of opening level L + 1: bias add, second product's add and activation of a gate are one
// level, not three.
// The matrix commands chain the same way through what they WRITE: a wavefront owns the same rows (or columns) of the result in every
// command of the chain, so five transposed products that add into one gradient vector, or the rank-1 updates of one weight
// gradient, are one level (the same wavefronts take them in recording order) instead of five.  What a matrix command READS is
// needed whole by every wavefront: a conflict through an input at the highest level always opens a new level.
struct Window {
  LhCmd cmd[CL_BUF_CMDS]; uint16_t level[CL_BUF_CMDS]; int16_t chain[CL_BUF_CMDS]; uint8_t chain_class[CL_BUF_CMDS + 1]; int32_t chain_row[CL_BUF_CMDS + 1]; int n; int top, nchains;       // top: highest level handed out
  int entries;                                                                // upper bound of the entries the workgroups' lists will hold
  // per 256-byte block: the highest level that writes / reads it, by which chain, through a range starting where (16 bits of the
  // start's float index tell two ranges over one block apart); four neighbouring blocks share a 64-byte bucket
  struct Slot { uint16_t wbase, rbase, w, r; int16_t wchain, rchain; };
  struct Bucket { uintptr_t key; uint32_t epoch; Slot sub[4]; uint32_t pad; } slot[HASH_N]; uint32_t epoch;
  struct Big { uintptr_t s, e; uint16_t w, r; int16_t wchain, rchain; } big[BIG_N]; int nbig; bool big_anywhere;
  // the distinct small ranges, each on the list of the one or two 4 KiB pages it touches: what a LARGE range is checked against
  struct Small { uintptr_t s, e, page0; uint16_t w, r; int next[2]; } small[CL_BUF_CMDS * 4]; int nsmall;
  struct Page { uintptr_t key; uint32_t epoch; int head; bool big; } page[PAGE_N];       // big: some large range touches the page
  uintptr_t small_lo, small_hi;                                               // bounding box of the small ranges
};
static_assert(sizeof(Window::Bucket) == 64, "a bucket of four blocks is one cache line");

static void window_reset(Window& W) {
  W.n = 0; W.entries = 0; W.top = 0; W.nchains = 0; W.nbig = 0; W.big_anywhere = false; W.nsmall = 0; W.small_lo = ~(uintptr_t)0; W.small_hi = 0;
  if (++W.epoch == 0) { for (int i = 0; i < HASH_N; i++) W.slot[i].epoch = 0; for (int i = 0; i < PAGE_N; i++) W.page[i].epoch = 0; W.epoch = 1; }
}
static inline Window::Slot* slot_of(Window& W, uintptr_t block, bool create) {
  const uintptr_t four = block >> 2;
  uint32_t h = (uint32_t)((four * 0x9E3779B97F4A7C15ull) >> 48) & (HASH_N - 1);
  for (int probe = 0; probe < HASH_N / 2; probe++, h = (h + 1) & (HASH_N - 1)) {
    Window::Bucket& bk = W.slot[h];
    if (bk.epoch != W.epoch) {
      if (!create) return nullptr;
      bk.key = four; bk.epoch = W.epoch;
      for (int q = 0; q < 4; q++) { Window::Slot& sl = bk.sub[q]; sl.w = sl.r = 0; sl.wchain = sl.rchain = -1; sl.wbase = sl.rbase = 0; }
      return &bk.sub[block & 3];
    }
    if (bk.key == four) return &bk.sub[block & 3];
  }
  return nullptr;
}
static inline uint16_t base16(uintptr_t start) { return (uint16_t)(start >> 2); }
static inline Window::Page* page_of(Window& W, uintptr_t pg, bool create) {
  uint32_t h = (uint32_t)((pg * 0x9E3779B97F4A7C15ull) >> 50) & (PAGE_N - 1);
  for (int probe = 0; probe < PAGE_N; probe++, h = (h + 1) & (PAGE_N - 1)) {
    Window::Page& pe = W.page[h];
    if (pe.epoch != W.epoch) { if (!create) return nullptr; pe.key = pg; pe.epoch = W.epoch; pe.head = -1; pe.big = false; return &pe; }
    if (pe.key == pg) return &pe;
  }
  return nullptr;
}
// What a command must follow: the highest level among the earlier commands of the window it conflicts with, and whether all of
// its conflicts AT that level are with one chain through identically based ranges (then it may join that chain).
struct Conflict {
  int lv = 0, chain = -1; bool one_chain = false;
  void see(int v, int ch, bool same_base) {
    if (v <= 0) return;
    if (v > lv) { lv = v; chain = ch; one_chain = same_base && ch >= 0; }
    else if (v == lv && (!same_base || ch != chain)) one_chain = false;
  }
};
static void conflicts_of(Window& W, const Extent& x, Conflict& c) {
  const bool small = x.e - x.s <= SMALL_BYTES;
  bool scan_big = !small || W.big_anywhere;
  if (!scan_big && W.nbig > 0) {                              // a small range meets a large one only on a page a large one touches
    const Window::Page* pa = page_of(W, x.s >> 12, false);
    scan_big = pa && pa->big;
    if (!scan_big && ((x.e - 1) >> 12) != (x.s >> 12)) { const Window::Page* pb = page_of(W, (x.e - 1) >> 12, false); scan_big = pb && pb->big; }
  }
  if (scan_big)
    for (int i = 0; i < W.nbig; i++) {
      const Window::Big& b = W.big[i];
      if (b.s < x.e && x.s < b.e) {
        const bool same = b.s == x.s && b.e == x.e;
        c.see(b.w, b.wchain, same);
        if (x.w) c.see(b.r, b.rchain, same);
      }
    }
  if (small) {
    for (uintptr_t blk = x.s >> 8; blk <= (x.e - 1) >> 8; blk++) {
      const Window::Slot* sl = slot_of(W, blk, false);
      if (!sl) continue;
      c.see(sl->w, sl->wchain, sl->wbase == base16(x.s));
      if (x.w) c.see(sl->r, sl->rchain, sl->rbase == base16(x.s));
    }
  } else if (x.s < W.small_hi && W.small_lo < x.e) {         // a large range over memory that small ranges of this window touch
    auto meet = [&](const Window::Small& m) { if (m.s < x.e && x.s < m.e) c.see(x.w ? (m.w > m.r ? m.w : m.r) : m.w, -1, false); };
    const uintptr_t pa = (x.s > W.small_lo ? x.s : W.small_lo) >> 12, pb = ((x.e < W.small_hi ? x.e : W.small_hi) - 1) >> 12;
    if (pb - pa >= (uintptr_t)PAGE_SCAN_MAX) { for (int i = 0; i < W.nsmall; i++) meet(W.small[i]); }
    else
      for (uintptr_t pg = pa; pg <= pb; pg++) {
        const Window::Page* pe = page_of(W, pg, false);
        if (!pe) continue;
        for (int i = pe->head; i >= 0;) { const Window::Small& m = W.small[i]; meet(m); i = m.next[m.page0 == pg ? 0 : 1]; }
      }
  }
}
static bool note_extent(Window& W, const Extent& x, int level, int chain) {
  if (x.e - x.s <= SMALL_BYTES) {
    for (uintptr_t blk = x.s >> 8; blk <= (x.e - 1) >> 8; blk++) {
      Window::Slot* sl = slot_of(W, blk, true);
      if (!sl) return false;
      if (x.w) {
        if (level > sl->w) { sl->w = (uint16_t)level; sl->wchain = (int16_t)chain; sl->wbase = base16(x.s); }
        else if (level == sl->w && (sl->wchain != chain || sl->wbase != base16(x.s))) sl->wchain = -1;       // two chains (or two alignments) at one level
      } else {
        if (level > sl->r) { sl->r = (uint16_t)level; sl->rchain = (int16_t)chain; sl->rbase = base16(x.s); }
        else if (level == sl->r && (sl->rchain != chain || sl->rbase != base16(x.s))) sl->rchain = -1;
      }
    }
    const uintptr_t pa = x.s >> 12, pb = (x.e - 1) >> 12;
    Window::Page* pe = page_of(W, pa, true);
    if (!pe) return false;
    int at = pe->head;
    while (at >= 0 && !(W.small[at].s == x.s && W.small[at].e == x.e)) at = W.small[at].next[W.small[at].page0 == pa ? 0 : 1];
    if (at < 0) {                                             // a range not seen in this window: on the list of each page it touches
      Window::Page* pf = pb != pa ? page_of(W, pb, true) : nullptr;
      if (pb != pa && !pf) return false;
      at = W.nsmall++;
      Window::Small& m = W.small[at];
      m.s = x.s; m.e = x.e; m.page0 = pa; m.w = m.r = 0; m.next[0] = pe->head; m.next[1] = -1;
      pe->head = at;
      if (pf) { m.next[1] = pf->head; pf->head = at; }
    }
    Window::Small& m = W.small[at];
    if (x.w) { if (level > m.w) m.w = (uint16_t)level; } else if (level > m.r) m.r = (uint16_t)level;
    if (x.s < W.small_lo) W.small_lo = x.s;
    if (x.e > W.small_hi) W.small_hi = x.e;
    return true;
  }
  for (int i = 0; i < W.nbig; i++) {
    Window::Big& b = W.big[i];
    if (b.s == x.s && b.e == x.e) {
      if (x.w) { if (level > b.w) { b.w = (uint16_t)level; b.wchain = (int16_t)chain; } else if (level == b.w && b.wchain != chain) b.wchain = -1; }
      else { if (level > b.r) { b.r = (uint16_t)level; b.rchain = (int16_t)chain; } else if (level == b.r && b.rchain != chain) b.rchain = -1; }
      return true;
    }
  }
  if (W.nbig == BIG_N) return false;
  const uintptr_t pa = x.s >> 12, pb = (x.e - 1) >> 12;
  if (pb - pa >= (uintptr_t)PAGE_SCAN_MAX) W.big_anywhere = true;
  else for (uintptr_t pg = pa; pg <= pb; pg++) { Window::Page* pe = page_of(W, pg, true); if (!pe) return false; pe->big = true; }
  Window::Big& b = W.big[W.nbig++];
  b.s = x.s; b.e = x.e; b.w = x.w ? (uint16_t)level : 0; b.r = x.w ? 0 : (uint16_t)level;
  b.wchain = x.w ? (int16_t)chain : -1; b.rchain = x.w ? -1 : (int16_t)chain;
  return true;
}

// Where a command goes: its level (one more than the highest level of an earlier command it must follow, or that very level when
// it joins the chain it follows) and its chain (-1: none).  Notes the command's ranges in the window.  false: a table of the
// window is full (nothing of this command is kept as long as the caller then resets the window and places it again).
static bool window_place(Window& W, const LhCmd& c, bool chains, int& lv, int& chain) {
  Extent x[4];
  const int k = cmd_extents(c, x);
  // cf: what the command must follow through operands that map onto wavefronts as the chain's do (all operands of an element-wise
  // command; what a matrix command writes, which cmd_extents lists first); cf_in: through what a matrix command reads
  Conflict cf, cf_in;
  const int cls = cmd_class(c);
  for (int i = 0; i < k; i++) conflicts_of(W, x[i], (cls >= 2 && i > 0) ? cf_in : cf);
  const int row = cls == 4 ? c.i1 : 0;             // rank-1 updates own rows: the same buffer cut into rows of another length is another mapping
  if (cls && chains && cf.one_chain && W.chain_class[cf.chain] == cls && W.chain_row[cf.chain] == row && cf_in.lv < cf.lv) { lv = cf.lv; chain = cf.chain; }      // joins the chain it follows
  else { lv = (cf.lv > cf_in.lv ? cf.lv : cf_in.lv) + 1; chain = -1; if (cls) { chain = W.nchains++; W.chain_class[chain] = (uint8_t)cls; W.chain_row[chain] = row; } }
  for (int i = 0; i < k; i++) if (!note_extent(W, x[i], lv, (cls >= 2 && i > 0) ? -1 : chain)) return false;
  W.cmd[W.n] = c; W.level[W.n] = (uint16_t)lv; W.chain[W.n] = (int16_t)chain; W.n++;
  if (lv > W.top) W.top = lv;
  return true;
}
static Window* window_new() {
  Window* w = new Window();
  for (int i = 0; i < HASH_N; i++) w->slot[i].epoch = 0;
  for (int i = 0; i < PAGE_N; i++) w->page[i].epoch = 0;
  w->epoch = 0;
  window_reset(*w);
  return w;
}
}  // namespace
