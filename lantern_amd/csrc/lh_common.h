// Shared host-side plumbing for the lantern_hip library: stream, error path, launch helpers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include "../../include/lantern_hip.h"

namespace lh {

extern hipStream_t g_stream;     // every kernel is enqueued here
extern int g_error_mode;         // 0 = print and exit, 1 = record and return
extern int g_num_cu;             // compute units of the device in use

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
  CAT_ELEMENTWISE, CAT_POOL, CAT_REDUCE, CAT_OPTIM, CAT_FILL, CAT_RNN, CAT_COUNT
};
extern unsigned g_prof_mask;
void prof_begin(int cat);
void prof_end(int cat);
struct ProfScope {
  int cat; bool on;
  explicit ProfScope(int c) : cat(c), on((g_prof_mask >> c) & 1u) { if (on) prof_begin(cat); }
  ~ProfScope() { if (on) prof_end(cat); }
};

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

static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

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

// ---- device helpers -------------------------------------------------------
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
