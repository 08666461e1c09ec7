// Lifetime, error path, device arena, transfers and timing events.
// Reference behaviour being replaced: CUB:18-25, 113-131 (handles + arena + rewind),
// API:453-473 (myGpuMalloc / myGpuFree), CUB:37-107 (toGPU / toCPU).
#include "lh_common.h"
#include "lh_arena.h"
#include <stdarg.h>
#include <string.h>
#include <vector>

namespace lh {
hipStream_t g_stream_raw = nullptr;
hipStream_t g_stream_cur = nullptr;
// Side stream: work whose results nothing needs before the optimizer (filter gradients) runs beside the main chain.
static hipStream_t g_side_stream = nullptr;
static bool g_side_dirty = false;            // the side stream holds work the main stream has not waited for
static int g_side_enabled = getenv("LH_NO_SIDE_STREAM") == nullptr;
constexpr int SIDE_EVENTS = 16;              // fork and join events, used round-robin
static hipEvent_t g_side_ev[SIDE_EVENTS];
static unsigned g_side_ev_next = 0;
static int64_t g_side_forks = 0;
static hipEvent_t side_event() { return g_side_ev[g_side_ev_next++ % SIDE_EVENTS]; }
void quiet_other_stream() {
  if (g_stream_cur == g_stream_raw) { if (g_side_dirty) (void)hipStreamSynchronize(g_side_stream); }
  else (void)hipStreamSynchronize(g_stream_raw);
}
void side_wait_for_main() {
  if (!g_side_stream) return;
  hipEvent_t ev = side_event();
  LH_HIP(hipEventRecord(ev, g_stream_raw));
  LH_HIP(hipStreamWaitEvent(g_side_stream, ev, 0));
}
// Scratch memory for kernels on the side stream.  Scratch from the top of the arena is safe on the main stream only (the stream
// orders the next user of the same memory behind the kernel that was given it); the side stream's kernels run in their own
// order among themselves, so they share one block of their own, which grows on demand.
static char* g_side_scratch = nullptr; static size_t g_side_scratch_bytes = 0;
void* side_scratch(size_t bytes) {
  if (bytes <= g_side_scratch_bytes) return g_side_scratch;
  if (hipDeviceSynchronize() != hipSuccess) { LH_FAIL("side scratch: the device did not come to rest"); return nullptr; }
  if (g_side_scratch) (void)hipFree(g_side_scratch);
  g_side_scratch = nullptr; g_side_scratch_bytes = 0;
  const size_t want = ((bytes + (bytes >> 2)) + ((size_t)1 << 20) - 1) & ~(((size_t)1 << 20) - 1);
  void* p = nullptr;
  if (hipMalloc(&p, want) != hipSuccess || p == nullptr) { LH_FAIL("side scratch: cannot allocate %zu bytes", want); return nullptr; }
  g_side_scratch = (char*)p; g_side_scratch_bytes = want;
  return p;
}
static int* g_fix_cnt = nullptr;
int* fix_counters() { return g_fix_cnt; }
void* persistent_alloc(size_t bytes) {
  void* p = nullptr;
  if (hipMalloc(&p, bytes) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
  return p;
}
void persistent_free(void* p) { if (p) (void)hipFree(p); }
bool side_work_begin() {
  if (!g_side_stream || !g_side_enabled || g_prof_mask != 0 || g_capturing || g_rec_on || g_stream_cur != g_stream_raw) return false;
  side_wait_for_main();
  g_stream_cur = g_side_stream; g_side_dirty = true;
  return true;
}
void side_work_end() { g_stream_cur = g_stream_raw; }
void* scratch_take(size_t bytes, bool& side) { side = g_stream_cur != g_stream_raw; return side ? side_scratch(bytes) : lh_malloc_uninit(bytes); }
void scratch_give(size_t bytes, bool side) { if (!side) lh_free_top(bytes); }
static void side_scratch_release() { if (g_side_scratch) (void)hipFree(g_side_scratch); g_side_scratch = nullptr; g_side_scratch_bytes = 0; }
void side_join() {
  if (!g_side_dirty) return;
  g_side_dirty = false;
  hipEvent_t ev = side_event();
  LH_HIP(hipEventRecord(ev, g_side_stream));
  LH_HIP(hipStreamWaitEvent(g_stream_raw, ev, 0));
}
bool g_tune_enabled = getenv("LH_NO_TUNE") == nullptr;
bool g_capturing = false;
int64_t g_plans_measured = 0, g_plans_remembered = 0;
bool g_deterministic = getenv("LH_DETERMINISTIC") != nullptr;
double g_tune_min_flop = getenv("LH_TUNE_MIN_FLOP") ? atof(getenv("LH_TUNE_MIN_FLOP")) : 1e7;
unsigned long long* g_capture_advance = nullptr;
unsigned long long g_capture_drawn = 0;
static unsigned long long* g_advance_pool = nullptr;   // one counter per graph
constexpr int MAX_GRAPHS = 256;
int g_error_mode = 0;
int g_num_cu = 256;
static char g_err[1024] = "";
static char* g_heap = nullptr;
static ArenaState g_arena;                     // bump pointer, peak, and the window above the top that is known to read zero (lh_arena.h)
static const size_t ZERO_AHEAD = 1u << 20;     // small zero-filled blocks are cleared this much at a time
static const size_t LAZY_MIN = 16u << 10;      // blocks of more than this may be cleared on demand instead (the networks on 32x32 images are made of blocks of 0.1 to 1 MiB)

bool fail(const char* file, int line, const char* fmt, ...) {
  char msg[768];
  va_list ap; va_start(ap, fmt); vsnprintf(msg, sizeof msg, fmt, ap); va_end(ap);
  const char* base = strrchr(file, '/'); base = base ? base + 1 : file;
  if (g_error_mode == 0) { fprintf(stderr, "lantern_hip error at %s:%d: %s\n", base, line, msg); fflush(stderr); exit(1); }
  if (g_err[0] == 0) snprintf(g_err, sizeof g_err, "%s:%d: %s", base, line, msg);
  return true;
}
bool failed() { return g_err[0] != 0; }

// ---- event profiler ---------------------------------------------------------------------
unsigned g_prof_mask = 0;
double g_work[CAT_COUNT];
int g_kernel_cat = CAT_GEMM;
struct ProfRec { hipEvent_t a, b; int cat; };
static std::vector<ProfRec> g_prof_recs;
static std::vector<hipEvent_t> g_prof_pool;
static hipEvent_t prof_event() {
  if (!g_prof_pool.empty()) { hipEvent_t e = g_prof_pool.back(); g_prof_pool.pop_back(); return e; }
  hipEvent_t e = nullptr;
  if (hipEventCreate(&e) != hipSuccess) return nullptr;
  return e;
}
void prof_begin(int cat) {
  ProfRec r; r.a = prof_event(); r.b = nullptr; r.cat = cat;
  if (g_rec_pending) rec_flush();
  if (r.a) (void)hipEventRecord(r.a, g_stream_cur);      // not ordered_stream(): timing a call must not bring deferred work forward
  g_prof_recs.push_back(r);
}
void prof_end(int cat) {
  for (size_t i = g_prof_recs.size(); i-- > 0;) {
    if (g_prof_recs[i].cat == cat && g_prof_recs[i].b == nullptr) {
      g_prof_recs[i].b = prof_event();
      if (g_rec_pending) rec_flush();
      if (g_prof_recs[i].b) (void)hipEventRecord(g_prof_recs[i].b, g_stream_cur);
      return;
    }
  }
}

static std::vector<hipGraphExec_t> g_graphs;
__global__ void k_set_u64(unsigned long long* p, unsigned long long keep, unsigned long long add) { *p = (keep ? *p : 0ull) + add; }
__global__ void k_zero16(uint4* p, size_t n16) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x, st = (size_t)gridDim.x * blockDim.x;
  for (; i < n16; i += st) p[i] = make_uint4(0, 0, 0, 0);
}
static void zero_async(void* p, size_t bytes) {  // bytes is a multiple of 256
  size_t n16 = bytes / 16;
  if (n16 == 0) return;
  if (rec_ok((int64_t)n16)) { rec_cmd(CL_ZERO16, (int)n16, 0, 0, 0.f, 0.f, 0.f, 0.f, p, nullptr, nullptr, nullptr); return; }
  int grid = stream_grid((int64_t)n16, 256 * 4);
  hipLaunchKernelGGL(k_zero16, dim3(grid), dim3(256), 0, g_stream, (uint4*)p, n16);
}
void zero_bytes_async(void* p, size_t bytes) { ProfScope prof_(CAT_FILL); zero_async(p, bytes); }
}  // namespace lh
using namespace lh;

extern "C" {

void lh_set_error_mode(int mode) { g_error_mode = mode; }
void lh_set_tuning(int on) { g_tune_enabled = on != 0; }
void lh_tune_counters(int64_t* measured, int64_t* remembered) { if (measured) *measured = g_plans_measured; if (remembered) *remembered = g_plans_remembered; }
void lh_set_deterministic(int on) { LZ_ENTER(); side_join(); g_deterministic = on != 0; }
int lh_get_deterministic(void) { return g_deterministic ? 1 : 0; }
const char* lh_last_error(void) { return g_err; }
void lh_clear_error(void) { g_err[0] = 0; }

void lh_setup(size_t heap_bytes) {
  LH_REQUIRE(g_heap == nullptr, "lh_setup called twice without lh_cleanup");
  LH_REQUIRE(heap_bytes >= 4096, "heap of %zu bytes is too small", heap_bytes);
  int dev = 0;
  LH_HIP(hipSetDevice(dev));
  hipDeviceProp_t prop;
  LH_HIP(hipGetDeviceProperties(&prop, dev));
  g_num_cu = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
  LH_HIP(hipStreamCreateWithFlags(&g_stream_raw, hipStreamNonBlocking));
  LH_HIP(hipStreamCreateWithFlags(&g_side_stream, hipStreamNonBlocking));     // same (default) priority as the main stream
  for (auto& e : g_side_ev) LH_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
  g_stream_cur = g_stream_raw; g_side_dirty = false;
  heap_bytes = (heap_bytes + 255) & ~(size_t)255;
  LH_HIP(hipMalloc((void**)&g_heap, heap_bytes));
  g_arena = ArenaState(); g_arena.bytes = heap_bytes;
  lazy::reset();
  LH_HIP(hipMalloc((void**)&g_advance_pool, MAX_GRAPHS * sizeof(unsigned long long)));
  LH_HIP(hipMalloc((void**)&g_fix_cnt, 4096 * sizeof(int)));          // FIX_MAX_TILES arrival counters (lh_igemm.h), zero between launches
  LH_HIP(hipMemset(g_fix_cnt, 0, 4096 * sizeof(int)));
  if (!multi_tensor_setup()) return;
}

static void stage_release();
static void copy_release();
void lh_cleanup(void) {
  lazy::reset();                 // whatever was deferred concerns memory that is about to go
  g_stream_cur = g_stream_raw;
  if (g_side_stream) { (void)hipStreamSynchronize(g_side_stream); (void)hipStreamDestroy(g_side_stream); for (auto& e : g_side_ev) (void)hipEventDestroy(e); }
  g_side_stream = nullptr; g_side_dirty = false;
  if (g_stream_raw) (void)hipStreamSynchronize(g_stream);
  cmdlist_release();
  side_scratch_release();
  stage_release();
  copy_release();
  multi_tensor_release();
  for (auto& e : g_graphs) if (e) { (void)hipGraphExecDestroy(e); e = nullptr; }
  g_graphs.clear(); g_capturing = false;
  if (g_advance_pool) (void)hipFree(g_advance_pool);
  g_advance_pool = nullptr; g_capture_advance = nullptr;
  if (g_fix_cnt) (void)hipFree(g_fix_cnt);
  g_fix_cnt = nullptr;
  if (g_heap) (void)hipFree(g_heap);
  if (g_stream_raw) (void)hipStreamDestroy(g_stream_raw);
  g_heap = nullptr; g_stream_raw = nullptr; g_stream_cur = nullptr; g_arena = ArenaState();
}

void lh_sync(void) {
  LH_NOT_CAPTURING("lh_sync");
  LZ_ENTER();                    // what is parked counts as enqueued; untouched zero blocks and unread results stay as they are
  side_join();
  lh_copy_join();
  LH_HIP(hipStreamSynchronize(g_stream)); LH_CHECK_LAUNCH();
  (void)cmdlist_report_timeout();      // the wait is over: a barrier that gave up in a command-list launch is reported now, not at the next hand-over
}

static void* bump(size_t bytes, bool zero) {
  if (!g_heap) { LH_FAIL("lh_malloc before lh_setup"); return nullptr; }
  if (zero && g_stream_cur != g_stream_raw) { LH_FAIL("lh_malloc between lh_side_begin and lh_side_end: zeroed memory is handed out in main-stream order only"); return nullptr; }
  const ArenaGrant g = arena_bump(g_arena, bytes, zero, lazy::defer_zero(), ZERO_AHEAD, LAZY_MIN);
  if (!g.ok) {
    // API:462-464 aborts on overflow; here it takes the library's error path.
    LH_FAIL("device arena exhausted: %zu used + %zu requested > %zu", g_arena.top, g.need, g_arena.bytes);
    return nullptr;
  }
  void* p = g_heap + g.offset;
  if (g.lazy) {
    lazy::note_zero_block(p, g.need);      // cleared when somebody reads it, never if its first user overwrites it
  } else if (g.zero_to > g.zero_from) {
    lazy::Scope lz_scope_;                 // the fill below is ordered before anything that can touch the block: parked launches stay parked
    ProfScope prof_(CAT_FILL);
    zero_async(g_heap + g.zero_from, g.zero_to - g.zero_from);
  }
  return p;
}
void* lh_malloc(size_t bytes) { return bump(bytes, true); }
void* lh_malloc_uninit(size_t bytes) { return bump(bytes, false); }
void lh_free_top(size_t bytes) {
  const size_t need = arena_round(bytes);
  LH_REQUIRE(need <= g_arena.top, "lh_free_top(%zu) below the arena base", bytes);
  if (lazy::g_busy) {
    if (lazy::g_depth == 0) { LZ_ENTER(); }       // a caller's pop (myGpuFree): nothing parked may still want the block
    lazy::arena_released(g_heap + g_arena.top - need);
  }
  (void)arena_pop(g_arena, bytes);
}
size_t lh_mark(void) { return g_arena.top; }
void lh_rewind(size_t mark) {
  LH_REQUIRE(mark <= g_arena.top && (mark & 255) == 0, "lh_rewind(%zu): not a mark at or below the top (%zu)", mark, g_arena.top);
  LZ_SCOPE();
  if (lazy::g_busy) lazy::on_rewind(g_heap + mark);     // zero fills and unread results of what is released are simply dropped
  side_join();      // what is handed out again must not be in use on the side stream
  (void)arena_rewind(g_arena, mark);
}
size_t lh_heap_used(void) { return g_arena.top; }
size_t lh_heap_peak(void) { return g_arena.peak; }

// Small uploads (a tree's labels, a batch's targets) go through a ring of pinned staging slots and do not wait for the
// device: the caller's buffer is free again when the call returns (it was copied into the slot), and the stream orders
// the transfer before everything issued afterwards.  A slot is reused after the event recorded behind its transfer.
constexpr size_t STAGE_BYTES = 64 << 10;
constexpr int STAGE_SLOTS = 32;
static char* g_stage = nullptr;                 // STAGE_SLOTS * STAGE_BYTES of pinned host memory
static hipEvent_t g_stage_ev[STAGE_SLOTS];
static bool g_stage_used[STAGE_SLOTS];
static unsigned g_stage_next = 0;
static bool stage_init() {
  if (g_stage) return true;
  if (hipHostMalloc((void**)&g_stage, STAGE_SLOTS * STAGE_BYTES, hipHostMallocDefault) != hipSuccess) { g_stage = nullptr; (void)hipGetLastError(); return false; }
  for (int i = 0; i < STAGE_SLOTS; i++) {
    g_stage_used[i] = false;
    if (hipEventCreateWithFlags(&g_stage_ev[i], hipEventDisableTiming) != hipSuccess) { (void)hipHostFree(g_stage); g_stage = nullptr; return false; }
  }
  return true;
}
static void stage_release() {
  if (!g_stage) return;
  for (int i = 0; i < STAGE_SLOTS; i++) (void)hipEventDestroy(g_stage_ev[i]);
  (void)hipHostFree(g_stage);
  g_stage = nullptr;
}

void lh_h2d(void* dst, const void* h_src, size_t bytes) {
  LH_NOT_CAPTURING("lh_h2d");
  LZ_ENTER();
  side_join();
  if (bytes == 0) return;
  lazy::wr(dst, bytes);
  if (bytes <= STAGE_BYTES && stage_init()) {
    const int slot = (int)(g_stage_next++ % STAGE_SLOTS);
    if (g_stage_used[slot]) LH_HIP(hipEventSynchronize(g_stage_ev[slot]));       // long since complete unless 32 uploads are in flight
    char* buf = g_stage + (size_t)slot * STAGE_BYTES;
    memcpy(buf, h_src, bytes);
    LH_HIP(hipMemcpyAsync(dst, buf, bytes, hipMemcpyHostToDevice, g_stream));
    LH_HIP(hipEventRecord(g_stage_ev[slot], g_stream));
    g_stage_used[slot] = true;
    return;
  }
  // Pageable source: the copy is staged before the call returns, so the host buffer may be reused.
  LH_HIP(hipMemcpyAsync(dst, h_src, bytes, hipMemcpyHostToDevice, g_stream));
  LH_HIP(hipStreamSynchronize(g_stream));
}
void lh_d2h(void* h_dst, const void* src, size_t bytes) {
  LH_NOT_CAPTURING("lh_d2h");
  LZ_ENTER();
  lazy::rd(src, bytes);
  side_join();
  lh_copy_join();    // an upload still on the copy stream may be what is read back
  LH_HIP(hipMemcpyAsync(h_dst, src, bytes, hipMemcpyDeviceToHost, g_stream));
  LH_HIP(hipStreamSynchronize(g_stream));
  (void)cmdlist_report_timeout();
}
// ---- transfers that do not stall the step: pinned host memory, a copy stream for uploads, read-backs without a wait ----
static hipStream_t g_copy_stream = nullptr;
static hipEvent_t g_copy_ev[4];
static unsigned g_copy_ev_next = 0;
static bool g_copy_dirty = false;              // the copy stream holds uploads the main stream has not waited for
static bool copy_init() {
  if (g_copy_stream) return true;
  if (hipStreamCreateWithFlags(&g_copy_stream, hipStreamNonBlocking) != hipSuccess) { g_copy_stream = nullptr; return false; }   // default priority
  for (auto& e : g_copy_ev) if (hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess) return false;
  return true;
}
static void copy_release() {
  if (!g_copy_stream) return;
  (void)hipStreamSynchronize(g_copy_stream);
  for (auto& e : g_copy_ev) (void)hipEventDestroy(e);
  (void)hipStreamDestroy(g_copy_stream);
  g_copy_stream = nullptr; g_copy_dirty = false;
}
void* lh_host_alloc(size_t bytes) {
  void* p = nullptr;
  if (hipHostMalloc(&p, bytes ? bytes : 1, hipHostMallocDefault) != hipSuccess) { (void)hipGetLastError(); LH_FAIL("lh_host_alloc(%zu): no pinned host memory", bytes); return nullptr; }
  return p;
}
void lh_host_free(void* p) { if (p) (void)hipHostFree(p); }
void lh_h2d_async(void* dst, const void* h_src_pinned, size_t bytes) {
  LH_NOT_CAPTURING("lh_h2d_async");
  LH_REQUIRE(g_stream_raw != nullptr, "lh_h2d_async before lh_setup");
  LH_REQUIRE(g_stream_cur == g_stream_raw, "lh_h2d_async between lh_side_begin and lh_side_end");
  if (bytes == 0) return;
  LZ_ENTER();
  lazy::wr(dst, bytes);
  LH_REQUIRE(copy_init(), "lh_h2d_async: cannot create the copy stream");
  // after everything issued so far (the last reader of dst), beside everything issued from now on
  hipEvent_t ev = g_copy_ev[g_copy_ev_next++ % 4];
  LH_HIP(hipEventRecord(ev, g_stream));
  LH_HIP(hipStreamWaitEvent(g_copy_stream, ev, 0));
  LH_HIP(hipMemcpyAsync(dst, h_src_pinned, bytes, hipMemcpyHostToDevice, g_copy_stream));
  g_copy_dirty = true;
}
void lh_copy_join(void) {
  if (!g_copy_dirty) return;
  LH_NOT_CAPTURING("lh_copy_join with an upload pending");
  g_copy_dirty = false;
  hipEvent_t ev = g_copy_ev[g_copy_ev_next++ % 4];
  LH_HIP(hipEventRecord(ev, g_copy_stream));
  LH_HIP(hipStreamWaitEvent(g_stream_raw, ev, 0));
}
void lh_d2h_async(void* h_dst_pinned, const void* src, size_t bytes) {
  LH_NOT_CAPTURING("lh_d2h_async");
  if (bytes == 0) return;
  LZ_ENTER();
  lazy::rd(src, bytes);
  LH_HIP(hipMemcpyAsync(h_dst_pinned, src, bytes, hipMemcpyDeviceToHost, g_stream));
}

void lh_d2d(void* dst, const void* src, size_t bytes) {
  LZ_ENTER();
  lazy::rd(src, bytes); lazy::wr(dst, bytes);
  if ((bytes & 3) == 0 && bytes > 0 && rec_ok((int64_t)(bytes / 4))) { rec_cmd(CL_COPY, (int)(bytes / 4), 0, 0, 0.f, 0.f, 0.f, 0.f, dst, src, nullptr, nullptr); return; }
  LH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, g_stream));
}

// ---- HIP graphs: a launch-bound step recorded once and replayed ----------------------------------------------
// ---- side stream ---------------------------------------------------------------------------------------------
void lh_side_begin(void) {
  LH_REQUIRE(g_stream_raw != nullptr, "lh_side_begin before lh_setup");
  LH_REQUIRE(g_stream_cur == g_stream_raw, "lh_side_begin: already on the side stream");
  LZ_SCOPE();                    // what is parked stays parked: whoever launches it from the side stream does so on the main stream and lets the side stream wait
  // In line (no concurrency) when switched off, while kernels are timed one by one, or while the stream is recorded.
  // (Deterministic mode keeps the side stream: which stream a kernel runs on changes no sum's order; two filter gradients of
  // one filter stay ordered by the joins, and the slices of a cut reduction are added up in slice order by a pass of their own.)
  if (!g_side_enabled || g_prof_mask != 0 || g_capturing || g_rec_on) return;
  hipEvent_t ev = side_event();
  LH_HIP(hipEventRecord(ev, g_stream));              // (flushes recorded commands first)
  LH_HIP(hipStreamWaitEvent(g_side_stream, ev, 0));
  g_stream_cur = g_side_stream; g_side_dirty = true; g_side_forks++;
}
void lh_side_end(void) { g_stream_cur = g_stream_raw; }
void lh_side_join(void) { LH_REQUIRE(g_stream_cur == g_stream_raw, "lh_side_join between lh_side_begin and lh_side_end"); side_join(); }
void lh_set_side_stream(int on) { g_side_enabled = on != 0; }
int64_t lh_side_forks(void) { return g_side_forks; }

void lh_capture_begin(void) {
  { LZ_SCOPE(); lazy::flush_all(); }          // the recording starts from memory that is what the program thinks it is
  side_join();
  lh_copy_join();
  LH_REQUIRE(g_stream_raw != nullptr, "lh_capture_begin before lh_setup");
  LH_REQUIRE(!g_capturing, "lh_capture_begin: already capturing");
  LH_REQUIRE(!g_rec_on, "lh_capture_begin: the command list is recording (its buffers cannot be replayed)");
  LH_REQUIRE(g_prof_mask == 0, "lh_capture_begin: per-category timing is on");
  LH_REQUIRE((int)g_graphs.size() < MAX_GRAPHS, "lh_capture_begin: %d graphs exist already", MAX_GRAPHS);
  g_capture_advance = g_advance_pool + g_graphs.size(); g_capture_drawn = 0;
  hipLaunchKernelGGL(k_set_u64, dim3(1), dim3(1), 0, g_stream, g_capture_advance, 0ull, 0ull);
  LH_CHECK_LAUNCH();
  LH_HIP(hipStreamBeginCapture(g_stream_raw, hipStreamCaptureModeThreadLocal));
  g_capturing = true;
  g_arena.zero_end = g_arena.top;       // a zero fill done eagerly says nothing about replays: every block handed out while recording records its own fill
}
int lh_capture_end(void) {
  if (!g_capturing) { LH_FAIL("lh_capture_end without lh_capture_begin"); return -1; }
  { LZ_SCOPE(); lazy::flush_all(); }          // everything the recorded calls stand for is in the graph
  if (g_capture_drawn) hipLaunchKernelGGL(k_set_u64, dim3(1), dim3(1), 0, g_stream_raw, g_capture_advance, 1ull, g_capture_drawn);
  g_capturing = false;
  g_arena.zero_end = g_arena.top;       // fills recorded into the graph have not run
  hipGraph_t graph = nullptr;
  hipError_t e = hipStreamEndCapture(g_stream_raw, &graph);
  if (e != hipSuccess || graph == nullptr) {
    (void)hipGetLastError();      // the capture is over; its error must not be reported by the next launch
    LH_FAIL("hipStreamEndCapture: %s (an entry point that waits for the device was called during capture?); lh_cleanup and lh_setup give a fresh stream", hipGetErrorString(e));
    return -1;
  }
  hipGraphExec_t exec = nullptr;
  e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (e != hipSuccess) { LH_FAIL("hipGraphInstantiate: %s", hipGetErrorString(e)); return -1; }
  g_graphs.push_back(exec);
  return (int)g_graphs.size() - 1;
}
void lh_graph_launch(int id) {
  lazy::flush_undeclared();         // a replay reads and writes whatever its recording did (parameters included): everything deferred is brought up to date, no kept copy survives
  LH_REQUIRE(id >= 0 && id < (int)g_graphs.size() && g_graphs[id] != nullptr, "lh_graph_launch: no graph %d", id);
  LH_HIP(hipGraphLaunch(g_graphs[id], g_stream));
}
void lh_graph_destroy(int id) {
  LH_REQUIRE(id >= 0 && id < (int)g_graphs.size() && g_graphs[id] != nullptr, "lh_graph_destroy: no graph %d", id);
  LH_NOT_CAPTURING("lh_graph_destroy");
  (void)hipStreamSynchronize(g_stream);
  (void)hipGraphExecDestroy(g_graphs[id]);
  g_graphs[id] = nullptr;
}

void lh_work_collect(double* h_bytes, int ncat) {
  for (int c = 0; c < ncat; c++) h_bytes[c] = c < CAT_COUNT ? g_work[c] : 0.0;
  for (int c = 0; c < CAT_COUNT; c++) g_work[c] = 0.0;
}
void lh_prof_enable(unsigned mask) { LZ_ENTER(); side_join(); g_prof_mask = mask; }
void lh_prof_collect(double* h_ms, int64_t* h_calls, int ncat) {
  for (int c = 0; c < ncat; c++) { h_ms[c] = 0.0; h_calls[c] = 0; }
  if (g_stream_raw) (void)hipStreamSynchronize(g_stream);
  for (auto& r : g_prof_recs) {
    float ms = 0.f;
    if (r.a && r.b && hipEventElapsedTime(&ms, r.a, r.b) == hipSuccess && r.cat < ncat) { h_ms[r.cat] += ms; h_calls[r.cat] += 1; }
    if (r.a) g_prof_pool.push_back(r.a);
    if (r.b) g_prof_pool.push_back(r.b);
  }
  g_prof_recs.clear();
}

void* lh_event_create(void) {
  hipEvent_t ev = nullptr;
  if (hipEventCreate(&ev) != hipSuccess) { LH_FAIL("hipEventCreate failed"); return nullptr; }
  return (void*)ev;
}
void lh_event_record(void* ev) { LZ_ENTER(); LH_HIP(hipEventRecord((hipEvent_t)ev, g_stream)); }
float lh_event_elapsed_ms(void* start, void* stop) {
  float ms = -1.0f;
  if (g_capturing) { LH_FAIL("lh_event_elapsed_ms waits for the device, which a graph being recorded cannot do"); return ms; }
  if (hipEventSynchronize((hipEvent_t)stop) != hipSuccess || hipEventElapsedTime(&ms, (hipEvent_t)start, (hipEvent_t)stop) != hipSuccess) {
    LH_FAIL("event timing failed"); return -1.0f;
  }
  return ms;
}
void lh_event_destroy(void* ev) { (void)hipEventDestroy((hipEvent_t)ev); }

}  // extern "C"
