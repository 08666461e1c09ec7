// Shared host-side plumbing for the lantern_hip library: stream, error path, launch helpers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include "../../include/lantern_hip.h"
#include "lh_cmd.h"

namespace lh {

extern hipStream_t g_stream_raw;  // the library's stream
// Where entry points enqueue now: g_stream_raw, or the side stream between lh_side_begin and lh_side_end.
extern hipStream_t g_stream_cur;
void side_join();                 // the main stream waits for what the side stream was given (no-op when it is idle)
void* persistent_alloc(size_t bytes);      // device memory of its own, outside the arena (waits for the device); nullptr when there is none
void persistent_free(void* p);
bool side_work_begin();                    // library-internal fork: the side stream waits for the main stream and becomes current; false: not now
void side_work_end();
void build_filter_layout(int kind, const int* prm, const float* w, float* dst);      // lh_conv.hip: the copy kernel of a layout, on the current stream
void build_filter_layouts(int n, const int* kinds, const int* const* prms, const float* const* ws, float* const* dsts);      // the same for n layouts, batched into few launches
int* fix_counters();                       // FIX_MAX_TILES zeroed ints in device memory (lh_setup): the arrival counters of igemm_launch_shared_tail, left zero by every launch
void* side_scratch(size_t bytes); // a block for the kernels of the side stream (one user at a time, in that stream's order); nullptr after a reported failure
// Scratch memory for a launch: the top of the arena on the main stream (stream order puts the next user of the same memory
// behind this launch), the side stream's own block on the side stream.  One block per entry point at a time.
void* scratch_take(size_t bytes, bool& side);
void scratch_give(size_t bytes, bool side);
void quiet_other_stream();        // host-side wait for the stream that is NOT current, so that a timing run has the device to itself
// Small operations recorded by the command list (lh_cmdlist.hip) but not launched yet.  Anything that is about to use
// the stream goes through `g_stream`, which launches the recorded commands first, so program order is kept.
extern int g_rec_pending;
void rec_flush();
void cmdlist_release();           // frees the command buffers (lh_cleanup)
bool cmdlist_report_timeout();    // true (and an error reported) if an interpreter launch gave up at a barrier since the last look
bool multi_tensor_setup();        // the multi-tensor optimizers' device table: reserved by lh_setup, freed by lh_cleanup
void multi_tensor_release();
// Deferred work (lh_defer.hip): launches parked until the next call shows whether it fuses with them, zero fills of arena
// blocks nobody has touched yet, and results of fused launches that the program could read but no kernel has written.
// An entry point that states what it reads and writes (lazy::Scope + rd / wr / acc / rw below) is served exactly; any
// other entry point reaches ordered_stream() at depth 0, which first brings everything deferred up to date.
constexpr int LAYOUT_PRM = 10;                       // parameters that name a filter layout (see lazy::layout_lookup)
enum { LAYOUT_KRSC = 0, LAYOUT_CTK = 1, LAYOUT_CKRS = 2 };
namespace lazy {
extern bool g_busy;               // something is parked, pending or unwritten
extern int g_depth;               // > 0 inside an entry point that declares its operands, and while deferred work is launched
void flush_undeclared();
}
static inline hipStream_t ordered_stream() {
  if (g_rec_pending) rec_flush();
  if (lazy::g_busy && lazy::g_depth == 0) lazy::flush_undeclared();
  return g_stream_cur;
}
#define g_stream (::lh::ordered_stream())     // every kernel is enqueued here
extern int g_error_mode;         // 0 = print and exit, 1 = record and return
extern int g_num_cu;             // compute units of the device in use
extern bool g_tune_enabled;      // launch plans are measured on first use (lh_set_tuning; off with LH_NO_TUNE in the environment)
extern bool g_capturing;         // between lh_capture_begin and lh_capture_end: work is recorded into a HIP graph, nothing may wait on the stream
// Deterministic mode (lh_set_deterministic): no result depends on the order in which blocks finish or on a measured launch
// plan.  Reductions that are cut across blocks write their partial sums to scratch memory and a second kernel adds them in a
// fixed order (instead of fp32 atomic adds); stream-K and every measured plan are off (the built-in rules decide), and the
// side stream runs in line.
extern bool g_deterministic;
// A remembered launch plan may be used / a plan may be measured now.  While a graph is recorded nothing can be timed, but
// what was measured before is still what gets launched.
extern int64_t g_plans_measured, g_plans_remembered;     // launch plans timed so far / launches that used a remembered plan (lh_tune_counters)
#define g_tune_lookup (::lh::g_tune_enabled && !::lh::g_deterministic)
#define g_tune_measure (g_tune_lookup && !::lh::g_capturing)
// C[m,n] (row stride ldc) = beta*C + partial[0] + partial[1] + ... + partial[slices-1], each partial a dense [m,n] block,
// added in that order by one thread per element.
void reduce_slices(float* C, int ldc, int m, int n, const float* partial, int slices, float beta);
extern double g_tune_min_flop;   // products below this many flop keep the built-in launch rule (a timing run costs more than it can win)
// Dropout draws from a counter-based stream whose position the caller passes per launch.  A replayed graph repeats its
// launch arguments, so a captured dropout adds *g_capture_advance (device memory; 0 for the first replay, advanced at the
// end of every replay by the g_capture_drawn positions the recorded step used) to the position it was recorded with.
// Entry points that wait for the device refuse to run while a graph is recorded (the wait would invalidate the capture).
#define LH_NOT_CAPTURING(what) LH_REQUIRE(!::lh::g_capturing, "%s waits for the device, which a graph being recorded cannot do (lh_capture_end first)", what)
extern unsigned long long* g_capture_advance;
extern unsigned long long g_capture_drawn;

// Records (mode 1) or prints and exits (mode 0).  Returns true so callers can `return` on it.
bool fail(const char* file, int line, const char* fmt, ...);
bool failed();

#define LH_FAIL(...) ::lh::fail(__FILE__, __LINE__, __VA_ARGS__)
#define LH_HIP(expr)                                                              \
  do {                                                                            \
    hipError_t e_ = (expr);                                                       \
    if (e_ != hipSuccess) { LH_FAIL("%s: %s", #expr, hipGetErrorString(e_)); return; } \
  } while (0)
#define LH_REQUIRE(cond, ...)                                                     \
  do { if (!(cond)) { LH_FAIL(__VA_ARGS__); return; } } while (0)
#define LH_CHECK_LAUNCH()                                                         \
  do {                                                                            \
    hipError_t e_ = hipGetLastError();                                            \
    if (e_ != hipSuccess) { LH_FAIL("kernel launch: %s", hipGetErrorString(e_)); return; } \
  } while (0)

// ---- per-category timing with HIP events on g_stream (off unless lh_prof_enable was called) ----
enum {
  CAT_CONV_FWD = 0, CAT_CONV_BWD_DATA, CAT_CONV_BWD_FILTER, CAT_GEMM, CAT_BN_FWD, CAT_BN_BWD,
  CAT_ELEMENTWISE, CAT_POOL, CAT_REDUCE, CAT_OPTIM, CAT_FILL, CAT_RNN, CAT_CMDLIST, CAT_COUNT
};
extern unsigned g_prof_mask;
void prof_begin(int cat);
void prof_end(int cat);
struct ProfScope {
  int cat; bool on;
  explicit ProfScope(int c) : cat(c), on((g_prof_mask >> c) & 1u) { if (on) prof_begin(cat); }
  ~ProfScope() { if (on) prof_end(cat); }
};

// Algorithmic bytes of the HBM-bound kernels launched, per category (lh_work_collect): the kernels that run are chosen here
// (fused or not, one pass or two), so the byte counts a roofline figure needs are kept here too.
extern double g_work[CAT_COUNT];
static inline void work_add(int cat, double bytes) { g_work[cat] += bytes; }

// Category the matrix kernels launched below an entry point are timed under: the events then bracket the
// k_igemm launch itself, not the small layout / fill kernels around it.
extern int g_kernel_cat;
struct KernelCat {
  int saved;
  explicit KernelCat(int c) : saved(g_kernel_cat) { g_kernel_cat = c; }
  ~KernelCat() { g_kernel_cat = saved; }
};

// Batch-norm statistics from the per-piece (sum, sum of squares) a convolution epilogue left behind:
// columns [0, col1) in pieces of g_main columns (slots 0 .. slots_main-1), columns [col1, ncols) in pieces of
// g_rem columns after them; partial[c][slot] = (sum, sum of squares) as float2.  Writes mean, 1/sqrt(var+eps), updates running stats.
void bn_finalize_conv_partials(const float* partial, int C, int ncols, int col1, int g_main, int slots_main, int g_rem,
                               float* save_mean, float* save_invstd, float* run_mean, float* run_var, float eps, float factor);
// The same pieces consumed by the normalisation itself: every block of the apply pass adds up its channel's pieces (as
// k_bn_finalize_conv does), so the separate statistics launch between the convolution and the apply pass disappears.
// out = bn(y) [relu] or relu(bn(y) + shortcut); the block of batch slice 0 stores the saved and running statistics.
struct ConvPieces { const float* partial; int ncols, col1, g_main, slots_main, g_rem, slots; float eps, factor; float* save_mean; float* save_invstd; float* run_mean; float* run_var; };
void bn_apply_from_pieces(const float* y, const ConvPieces& pieces, const float* gamma, const float* beta, const float* shortcut, float* out, int relu,
                          int N, int C, int HW);

static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- deferred work: declarations an entry point makes about its operands (all sizes in bytes) -----------------------------
namespace lazy {
extern bool g_enabled;            // lh_set_fusion (LH_NO_FUSION in the environment): off = every call runs as issued, lh_malloc clears at once
extern bool g_replay;             // deferred work is being launched: entry points run as called and declare nothing
struct Scope { Scope() { g_depth++; } ~Scope() { g_depth--; } };
static inline bool active() { return g_enabled && !g_replay; }
void flush_parked();                               // launch what is parked (unfused)
void flush_all();                                  // parked launches, pending zero fills and unwritten results: all brought up to date
void rd(const void* p, size_t bytes);              // the range is about to be read
void wr(const void* p, size_t bytes);              // the range is about to be overwritten as a whole
bool acc(const void* p, size_t bytes);             // the range is about to be added into; true: it is a zero block nobody has cleared or touched, so overwrite it instead
void rw(const void* p, size_t bytes);              // read and written in place
static inline void rd_f(const void* p, int64_t n) { if (g_busy && p && n > 0) rd(p, (size_t)n * 4); }
static inline void wr_f(const void* p, int64_t n) { if (g_busy && p && n > 0) wr(p, (size_t)n * 4); }
static inline void rw_f(const void* p, int64_t n) { if (g_busy && p && n > 0) rw(p, (size_t)n * 4); }
static inline bool acc_f(const void* p, int64_t n) { return g_busy && p && n > 0 ? acc(p, (size_t)n * 4) : false; }
// an output that may be one of the inputs (in-place forms): then it is read and written, and whatever was still to be produced
// from its old contents is produced first
static inline void out_f(const void* p, int64_t n, bool aliases_an_input) { if (aliases_an_input) rw_f(p, n); else wr_f(p, n); }
// accumulate with a beta the caller passed: 1 on a block nobody has touched becomes 0; 0 is a plain overwrite
static inline float beta_f(const void* p, int64_t n, float beta) {
  if (!g_busy || !p || n <= 0) return beta;
  if (beta == 0.f) { wr(p, (size_t)n * 4); return 0.f; }
  return acc(p, (size_t)n * 4) && beta == 1.f ? 0.f : beta;
}
// arena bookkeeping (lh_runtime.hip)
void note_zero_block(void* p, size_t bytes);       // lh_malloc handed out [p, p + bytes) without clearing it
void arena_released(char* from);                   // the arena above `from` is released (rewind, pop): nothing there can be read again
bool defer_zero();                                 // lh_malloc may hand out large blocks uncleared now
// parking; each returns true when the call has been taken over (parked or fused) and the entry point has nothing left to do
bool park_conv_fwd(const float* x, const float* w, const float* bias, float* y, int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW);
bool park_bn_train_fwd(const float* x, const float* gamma, const float* beta, float* run_mean, float* run_var, float* y,
                       float* save_mean, float* save_invstd, int N, int C, int HW, float eps, float factor);
bool park_add(const float* a, const float* b, float* out, int64_t n);
bool take_relu_inplace(float* y, int64_t n);
bool park_relu_grad_inplace(const float* y, float* d, int64_t n);
bool park_add_grad(float* ad, float* bd, const float* outd, int64_t n);
bool take_relu_grad_bias(const float* dy, float* db, int N, int K, int PQ);
bool take_bn_bwd(const float* x, const float* dy, const float* gamma, const float* save_mean, const float* save_invstd,
                 float* dx, float beta_dx, float* dgamma, float* dbeta, int N, int C, int HW);
bool gather_update(int mode, float* x, float* d, float* v, float lr, float mu, float clip, int nesterov, int64_t n);
// filter layouts (kept copies of a filter in the order a convolution kernel reads it; lh_defer.hip).  Returns the copy, or
// nullptr when the caller has to use scratch memory as before; `build`: the copy has to be written first, by the caller, on
// the current stream (build_filter_layout).
float* layout_lookup(const float* w, size_t wbytes, int kind, const int* prm, size_t bytes, bool& build);
void forget_forward_records();                     // parameters are about to change: what the backward pass would recompute from them is no longer valid
void on_rewind(char* new_top);
void reset();                                      // forget everything deferred without launching anything (lh_setup, lh_cleanup)
}
// An entry point that declares its operands opens with LZ_ENTER(): from here to its end nothing is brought up to date behind
// its back, and whatever was parked (and is not continued by this call) is launched first.
#define LZ_SCOPE() ::lh::lazy::Scope lz_scope_
#define LZ_ENTER() ::lh::lazy::Scope lz_scope_; do { if (::lh::lazy::g_busy && !::lh::lazy::g_replay) ::lh::lazy::flush_parked(); } while (0)
// kernels the deferred work needs from other files
void mask_relu(float* dst, const float* src, const float* y, int64_t n);                     // dst = y > 0 ? src : 0
void add_plain(const float* a, const float* b, float* out, int64_t n);
void relu_grad_inplace_now(const float* y, float* d, int64_t n);
void conv2d_fwd_relu_now(const float* x, const float* w, const float* bias, float* y, int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW);
void conv_bwd_bias_mask_now(const float* y, float* dy, float* db, int N, int K, int PQ);     // dy = y > 0 ? dy : 0 in place; db[k] += its sum over n, p, q
void multi_update_now(int mode, int count, float* const* hx, float* const* hd, float* const* hv, const int64_t* hn, float lr, float mu, float clip, int nesterov);
void zero_bytes_async(void* p, size_t bytes);      // bytes a multiple of 256

// ---- command list: small operations recorded on the host and executed in order by one workgroup -------------
// While recording is on (lh_cmdlist_begin), an entry point whose operands are small enough appends a command instead
// of launching a kernel; a tree-structured model of 150-element vectors issues thousands of such operations per
// step, and the host's launch rate is what bounds it.
extern int g_rec_on;
bool rec_push(const LhCmd& c);                     // appends a command (launches a full buffer first); false on error
static inline bool rec_ok(int64_t n, int64_t limit = REC_MAX_ELEMS) { return g_rec_on && n <= limit; }
static inline bool rec_cmd(int op, int i0, int i1, int i2, float f0, float f1, float f2, float f3,
                             const void* p0, const void* p1, const void* p2, const void* p3) {
  LhCmd c;
  c.op = op; c.i0 = i0; c.i1 = i1; c.i2 = i2; c.f0 = f0; c.f1 = f1; c.f2 = f2; c.f3 = f3;
  c.p0 = (void*)p0; c.p1 = (void*)p1; c.p2 = (void*)p2; c.p3 = (void*)p3;
  return rec_push(c);
}

// Grid for a grid-stride streaming kernel: enough blocks to cover n at `per_block`
// elements each, capped at a few waves of blocks per CU.
static inline int stream_grid(int64_t n, int per_block) {
  int64_t g = cdiv(n, per_block);
  int64_t cap = (int64_t)g_num_cu * 16;
  if (g > cap) g = cap;
  if (g < 1) g = 1;
  return (int)g;
}

}  // namespace lh

// ---- device helpers (absent when a host compiler builds the host-side logic on its own for the sanitizer checks) ----
#ifdef __HIPCC__
__device__ __forceinline__ float lh_wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return v;
}
__device__ __forceinline__ float lh_wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_down(v, off, 64));
  return v;
}
// Block-wide sum for blockDim.x a multiple of 64 (<= 1024); result valid in every thread.
__device__ __forceinline__ float lh_block_sum(float v, float* smem /* >= 17 floats */) {
  v = lh_wave_sum(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  if (wave == 0) {
    float t = lane < nw ? smem[lane] : 0.0f;
    t = lh_wave_sum(t);
    if (lane == 0) smem[16] = t;
  }
  __syncthreads();
  return smem[16];
}
__device__ __forceinline__ float lh_block_max(float v, float* smem) {
  v = lh_wave_max(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  if (wave == 0) {
    float t = lane < nw ? smem[lane] : -3.402823466e+38f;
    t = lh_wave_max(t);
    if (lane == 0) smem[16] = t;
  }
  __syncthreads();
  return smem[16];
}
#endif  // __HIPCC__
