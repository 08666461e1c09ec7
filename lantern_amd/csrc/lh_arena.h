// The device arena's bookkeeping: a bump pointer over one allocation, 256-byte blocks, and what has to be cleared so that a
// block from lh_malloc reads zero (the property Tensor.zeros relies on, TensorDifferentiation.scala:1075-1076; the
// reference clears the used span on every rewind, TensorDslCublas.scala:22-25).  Host arithmetic only: lh_runtime.hip acts
// on the grants (it launches the fills), tests/host_cpp/defer_check.cpp uses the same code over host memory.
//   - [top, zero_end) is known to read zero: small blocks are cleared a window of `zero_ahead` bytes at a time, so a run of
//     them costs one fill, not one each; a pop or a rewind forgets the window (what lay above the new top may have been written);
//   - a block of more than `lazy_min` bytes is either cleared when handed out or, when the caller may put the clearing off
//     (`may_defer`), handed out as it is and reported as `lazy` for the deferred-work bookkeeping to note.
#pragma once
#include <stddef.h>

namespace lh {
struct ArenaState { size_t bytes = 0, top = 0, peak = 0, zero_end = 0; };
struct ArenaGrant {
  bool ok = false;              // false: the arena is exhausted (nothing changed)
  size_t offset = 0, need = 0;  // the block: [offset, offset + need)
  bool lazy = false;            // handed out uncleared: the caller notes it as a zero block nobody has touched
  size_t zero_from = 0, zero_to = 0;   // clear [zero_from, zero_to) now (empty when equal)
};
static inline size_t arena_round(size_t bytes) { size_t need = (bytes + 255) & ~(size_t)255; return need ? need : 256; }
static inline ArenaGrant arena_bump(ArenaState& a, size_t bytes, bool zero, bool may_defer, size_t zero_ahead, size_t lazy_min) {
  ArenaGrant g;
  g.need = arena_round(bytes);
  if (g.need < bytes || a.top + g.need > a.bytes || a.top + g.need < a.top) return g;
  g.ok = true; g.offset = a.top;
  if (zero && g.need > lazy_min && may_defer) {
    g.lazy = true;
  } else if (zero && a.top + g.need > a.zero_end) {
    g.zero_from = a.zero_end > a.top ? a.zero_end : a.top;
    g.zero_to = a.top + g.need;
    if (g.need < zero_ahead) g.zero_to = a.top + zero_ahead < a.bytes ? a.top + zero_ahead : a.bytes;
    a.zero_end = g.zero_to;
  }
  a.top += g.need;
  if (a.top > a.peak) a.peak = a.top;
  return g;
}
static inline bool arena_pop(ArenaState& a, size_t bytes) {
  const size_t need = arena_round(bytes);
  if (need > a.top) return false;
  a.top -= need;
  a.zero_end = a.top;            // what was handed out above the new top may have been written
  return true;
}
static inline bool arena_rewind(ArenaState& a, size_t mark) {
  if (mark > a.top || (mark & 255) != 0) return false;
  a.top = mark;
  a.zero_end = mark;
  return true;
}
}  // namespace lh
