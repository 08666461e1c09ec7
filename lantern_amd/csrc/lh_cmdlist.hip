// Command list: small operations recorded on the host and executed by a few 1024-thread workgroups in one launch per buffer.
//
// A model built from 150-element vectors (the sentiment TreeLSTM: ~3600 operator calls per tree) is bound by the host's
// kernel-launch rate (about 3 us per launch), not by the device.  Between lh_cmdlist_begin() and lh_cmdlist_end() every entry
// point whose operands are small appends a 64-byte command instead of launching; the commands of a buffer are handed to
// k_cmdlist when the buffer is full, when recording ends, or when any other entry point is about to use the stream
// (lh::ordered_stream), so the program order of all operations is kept.
//
// A dependent command costs a memory round trip (load, store, visibility), a microsecond or more, whatever its size.  So the host
// works out, per buffer, which commands depend on which (byte ranges read and written: a command that writes a range comes after
// every earlier command that touches it, one that reads it after every earlier writer) and gives each command a LEVEL, one more
// than the highest level it depends on.  The buffer is executed level by level: commands of one level have no dependence on each
// other and are spread over the workgroups and their wavefronts, so their round trips overlap; one barrier over all workgroups
// per level makes a level's stores visible to the next.  Independent work of a program (the ten gate products of a tree node, the
// two subtrees of a node) thus runs side by side without the program saying so.  Commands that depend only on each other, lane by
// lane (or row by row of what they write), share a level (a chain); long element-wise chains run as programs over LDS.  Each workgroup gets its own list of the commands it has a part in: the walk over
// a list is scalar work, and a compute unit has one scalar unit for its 16 wavefronts.
// The arithmetic of each command follows the stand-alone kernel of the same operation; no command uses atomics, so the result does
// not depend on how many workgroups run it.
#include "lh_common.h"
using namespace lh;

namespace lh {
int g_rec_on = 0;
int g_rec_pending = 0;
}

namespace {
constexpr int CL_THREADS = 1024;
constexpr int CL_CHUNK = 256;                 // commands staged in LDS at a time
constexpr int CL_NBUF = 16;
constexpr int CL_MAX_GROUPS = 64;
// Two op words per entry of a workgroup's list.  Word 0: operation | CL_SPLIT | start << 12 | barriers << 24; word 1: pieces.
constexpr int CL_OP_MASK = 0xff;
constexpr int CL_SYNC = 0xfe;                 // the workgroup's wavefronts meet: what the entries before it put into LDS is there for all
constexpr int CL_CHAIN = 0xfc;                // an element-wise chain as a program: i0 commands of 16 bytes each in the entries behind this one
constexpr int CL_PRELOAD = 0xfd;              // up to four vectors into LDS slots (p0..p3; i0, i2: their lengths, 16 bits each; i1: their slots): what a
                                              // chain program works on
constexpr int CL_NSLOT_MAX = 128, CL_SLOT_ELEMS = 256;   // LDS slots of a workgroup at most (as many as the device's LDS allows), floats in each
constexpr int CL_NOP = 0xff;                  // an entry that only carries barriers (a workgroup with nothing to do in some levels)
constexpr int CL_SPLIT = 0x200;               // a matrix command: its pieces are dealt round the wavefronts of all workgroups
constexpr int CL_START_SHIFT = 12;            // 12 bits: where the command's work starts: a wavefront 0..15 of the workgroup or, for a split
                                              // command, one of the wavefronts of all workgroups taken together
constexpr int CL_BARRIERS_SHIFT = 24;         // 8 bits: barriers over all workgroups to pass before the entry (levels completed since the last one)
constexpr int CL_WBLOCK = 4;                  // wavefronts of all workgroups are numbered in blocks of 4 of one workgroup, the blocks dealt
                                              // round the workgroups: the pieces of a 150-row product fall to 4 workgroups, not to 15
constexpr long CL_SPIN_LIMIT = 4000000L;      // polls of a grid barrier before a workgroup gives up: a few seconds, where a real wait is one level of commands (microseconds)

static bool g_slots = true;           // LH_CMDLIST_SLOTS=0 in the environment: chains read and write memory only
static bool g_chains = true;          // LH_CMDLIST_CHAINS=0 in the environment: every dependent command opens a new level
// A buffer as the device sees it: a directory (first entry and number of entries of each workgroup's list), the lists' commands
// (64 bytes an entry; a command is copied into the list of every workgroup that has a part in it), then their op words.
constexpr int CL_CAP = 6 * CL_BUF_CMDS;       // entries a buffer holds
constexpr size_t CL_DIR_BYTES = CL_MAX_GROUPS * sizeof(uint2);
constexpr size_t CL_BUF_BYTES = CL_DIR_BYTES + (sizeof(LhCmd) + sizeof(uint2)) * (size_t)(CL_CAP + CL_CHUNK);
static_assert(CL_DIR_BYTES % 64 == 0, "the commands start on a 64-byte boundary");
struct Ring {
  char* host[CL_NBUF]; hipEvent_t done[CL_NBUF]; bool busy[CL_NBUF];
  char* mirror;                      // device copy of the buffer being executed (launches are in stream order: one is enough)
  int cur; bool ready;
  int64_t recorded, launches, levels;
  unsigned long long* sync;          // device: [0] arrivals at grid barriers, [1] a workgroup gave up waiting
  unsigned long long sync_base;      // arrivals once everything launched so far has run
  int groups;                        // workgroups per launch
  int nslot;                         // LDS slots of a workgroup for chain programs
  unsigned* host_flag; unsigned* host_flag_dev;       // pinned word a workgroup sets when its barrier wait ran out
};
static Ring g_ring = {};

typedef __attribute__((address_space(1))) float gfloat;       // device (global) memory, as opposed to a generic address
typedef __attribute__((address_space(1))) int gint;
__device__ __forceinline__ float cl_bop(int op, float a, float b) {
  switch (op) { case LH_ADD: return a + b; case LH_SUB: return a - b; case LH_MUL: return a * b; default: return a / b; }
}
__device__ __forceinline__ float cl_unary(int op, float v, float lo, float hi) {
  switch (op) {
    case LH_RELU: return v < 0.f ? 0.f : v;
    case LH_TANH: return tanhf(v);
    case LH_SIGMOID: return 1.0f / (expf(-v) + 1.0f);
    case LH_EXP: return expf(v);
    case LH_LOG: return logf(v);
    case LH_SQRT: return sqrtf(v);
    case LH_SQUARE: return v * v;
    default: return v < lo ? lo : (v > hi ? hi : v);        // LH_HARDTANH
  }
}
// dx (+)= g(x | y, dy) exactly as lh_unary_grad's kernels
__device__ __forceinline__ float cl_unary_grad(int op, int inplace, float d, float xv, float yv, float g, float lo, float hi) {
  switch (op) {
    case LH_RELU: return inplace ? (yv > 0.f ? d : 0.f) : d + (xv < 0.f ? 0.f : g);
    case LH_HARDTANH: return inplace ? ((yv > lo && yv < hi) ? d : 0.f) : d + ((xv < lo || xv > hi) ? 0.f : g);
    case LH_TANH: return d + (1.0f - yv * yv) * g;
    case LH_SIGMOID: return d + ((1.0f - yv) * yv) * g;
    case LH_EXP: return d + g * yv;
    case LH_LOG: return d + g / xv;
    case LH_SQRT: return d + g / yv / 2.0f;
    default: return d + g * xv * 2.0f;                         // LH_SQUARE
  }
}
__device__ __forceinline__ float cl_wave_sum_all(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float cl_wave_max_all(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// Matrix operands are read and written through buffer descriptors: a 32-bit byte offset per lane instead of a 64-bit
// address computed per element (one workgroup's vector ALUs, not memory, bound these commands), constant column steps folded
// into the instruction, and anything past the operand's last byte reads as zero or is not stored, so rows past the matrix
// need no test.  The descriptor's base must be wave-uniform: the pointer comes out of LDS and is made so explicitly.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t cl_rsrc(const gfloat* p, int64_t bytes) {
  const uint64_t a = (uint64_t)(uintptr_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a), hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
  return __builtin_amdgcn_make_buffer_rsrc((void*)(((uint64_t)hi << 32) | lo), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ float cl_ld(__amdgpu_buffer_rsrc_t r, uint32_t off) { return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, (int)off, 0, 0)); }
__device__ __forceinline__ void cl_st(__amdgpu_buffer_rsrc_t r, uint32_t off, float v) { __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), r, (int)off, 0, 0); }
constexpr uint32_t CL_OOB = 0x80000000u;       // an offset no operand reaches (operands are far below 2 GiB)
// Sum over the 64 lanes, the same value in every lane: DPP inside rows of 16, one swizzle, two lane reads.
__device__ __forceinline__ float cl_wave_sum_dpp(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));    // quad_perm [1,0,3,2]
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));    // quad_perm [2,3,0,1]
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));   // row_half_mirror
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));   // row_mirror
  v += __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401F));                      // lane ^ 16
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0)) + __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
}

// Data pointers carry no __restrict__ and no const: a command may read what the command before it wrote.
// `gw` of `GW`: which of the wavefronts that share the command this one is.  An element-wise command belongs to one workgroup
// (GW = 16, gw counted from the wavefront the host let it start on); the matrix commands are cut into pieces over the wavefronts
// of all workgroups (one compute unit draws only some 25 GB/s from memory, whatever its wavefronts do; a 150 x 150 matrix spread
// over 16 units takes one memory round trip): piece k goes to wavefront (start + k) mod GW, neighbouring wavefronts sit in
// different workgroups, and the pieces of the commands of one level follow each other round the wavefronts, so a wavefront
// rarely holds pieces of two of them and their memory round trips overlap instead of queueing.
__device__ __forceinline__ void cl_run(const LhCmd& c, const int opc, const int gw, const int GW, float* S, uint64_t* SP) {
  constexpr int NW = CL_THREADS / 64;
  const int lane = threadIdx.x & 63, wave = gw, t = wave * 64 + lane;
  const int ST = GW * 64;                               // threads that share the command
  // Operands are device memory, and the pointers say so: an access through a generic pointer counts as an LDS operation too until it
  // completes, so the wait for the next op word (an LDS read) would wait for every store of the command before it.
  gfloat* p0 = (gfloat*)(uintptr_t)c.p0; gfloat* p1 = (gfloat*)(uintptr_t)c.p1; gfloat* p2 = (gfloat*)(uintptr_t)c.p2; gfloat* p3 = (gfloat*)(uintptr_t)c.p3;
  switch (opc) {
    case CL_ZERO16: {            // 16 bytes a thread
      typedef __attribute__((ext_vector_type(4))) unsigned int vec4;
      typedef __attribute__((address_space(1))) vec4 gvec4;
      gvec4* p = (gvec4*)(uintptr_t)c.p0; const int n = c.i0; const vec4 z = {0u, 0u, 0u, 0u};
      for (int i = t; i < n; i += ST) p[i] = z;
      break;
    }
    case CL_FILL: { const int n = c.i0; const float v = c.f0; for (int i = t; i < n; i += ST) p0[i] = v; break; }
    case CL_COPY: { const int n = c.i0; for (int i = t; i < n; i += ST) p0[i] = p1[i]; break; }
    case CL_GEAM: { const int n = c.i0; const float al = c.f0, be = c.f1; for (int i = t; i < n; i += ST) p0[i] = p1[i] * al + p2[i] * be; break; }
    case CL_SCALAR: { const int n = c.i0, op = c.i1; const float sc = c.f0; for (int i = t; i < n; i += ST) p0[i] = cl_bop(op, p1[i], sc); break; }
    case CL_BIN: { const int n = c.i0, op = c.i1; for (int i = t; i < n; i += ST) p0[i] = cl_bop(op, p1[i], p2[i]); break; }
    case CL_ACC: { const int n = c.i0; for (int i = t; i < n; i += ST) p0[i] = p0[i] + p1[i]; break; }
    case CL_ACCNEG: { const int n = c.i0; for (int i = t; i < n; i += ST) p0[i] = p0[i] + (0.0f - p1[i]); break; }
    case CL_ACCMUL: { const int n = c.i0; for (int i = t; i < n; i += ST) p0[i] = p0[i] + p1[i] * p2[i]; break; }
    case CL_UNARY: { const int n = c.i0, op = c.i1; const float lo = c.f0, hi = c.f1; for (int i = t; i < n; i += ST) p0[i] = cl_unary(op, p1[i], lo, hi); break; }
    case CL_UNARY_GRAD: {        // p0 = dx, p1 = x, p2 = y, p3 = dy
      const int n = c.i0, op = c.i1, inplace = c.i2; const float lo = c.f0, hi = c.f1;
      const bool need_x = (op == LH_RELU || op == LH_HARDTANH) ? !inplace : (op == LH_LOG || op == LH_SQUARE);
      const bool need_y = (op == LH_RELU || op == LH_HARDTANH) ? inplace != 0 : !(op == LH_LOG || op == LH_SQUARE);
      const bool need_g = !((op == LH_RELU || op == LH_HARDTANH) && inplace);
      for (int i = t; i < n; i += ST)
        p0[i] = cl_unary_grad(op, inplace, p0[i], need_x ? p1[i] : 0.f, need_y ? p2[i] : 0.f, need_g ? p3[i] : 0.f, lo, hi);
      break;
    }
    case CL_PRELOAD: {           // element t of up to four vectors into their slots (all loads in flight together), and where the vectors live
      const uint32_t n01 = (uint32_t)c.i0, n23 = (uint32_t)c.i2, sl = (uint32_t)c.i1;
      const int n0 = n01 & 0xffff, n1 = n01 >> 16, n2 = n23 & 0xffff, n3 = n23 >> 16;
      const float v0 = t < n0 ? p0[t] : 0.f, v1 = t < n1 ? p1[t] : 0.f, v2 = t < n2 ? p2[t] : 0.f, v3 = t < n3 ? p3[t] : 0.f;
      if (t < n0) S[(sl & 0xff) * CL_SLOT_ELEMS + t] = v0;
      if (t < n1) S[((sl >> 8) & 0xff) * CL_SLOT_ELEMS + t] = v1;
      if (t < n2) S[((sl >> 16) & 0xff) * CL_SLOT_ELEMS + t] = v2;
      if (t < n3) S[(sl >> 24) * CL_SLOT_ELEMS + t] = v3;
      if (t == 0) {
        if (n0) SP[sl & 0xff] = (uint64_t)(uintptr_t)c.p0;
        if (n1) SP[(sl >> 8) & 0xff] = (uint64_t)(uintptr_t)c.p1;
        if (n2) SP[(sl >> 16) & 0xff] = (uint64_t)(uintptr_t)c.p2;
        if (n3) SP[sl >> 24] = (uint64_t)(uintptr_t)c.p3;
      }
      break;
    }
    case CL_SYNC: __syncthreads(); break;
    case CL_CHAIN: {             // c.i0 packed commands in the entries behind this one (the same staged chunk): LDS to LDS, results also to memory
      const int count = c.i0;
      const uint4* prog = reinterpret_cast<const uint4*>(&c + 1);
      uint4 ahead = prog[0];
      for (int m = 0; m < count; m++) {
        const uint32_t w0 = __builtin_amdgcn_readfirstlane(ahead.x), w1 = __builtin_amdgcn_readfirstlane(ahead.y);
        const float f0 = __uint_as_float(__builtin_amdgcn_readfirstlane(ahead.z)), f1 = __uint_as_float(__builtin_amdgcn_readfirstlane(ahead.w));
        ahead = prog[m + 1];                                   // the entry after the last packed command exists (the list's op words follow the commands)
        const int mop = w0 & 0xff, n = (int)(w1 >> 16), sub = (int)(w1 >> 8) & 0x7f, inplace = (int)(w1 >> 15) & 1;
        if (t >= n) continue;
        float* d = S + ((w0 >> 8) & 0xff) * CL_SLOT_ELEMS + t;
        const float* a = S + ((w0 >> 16) & 0xff) * CL_SLOT_ELEMS + t;
        const float* b = S + (w0 >> 24) * CL_SLOT_ELEMS + t;
        const float* g = S + (w1 & 0xff) * CL_SLOT_ELEMS + t;
        float r;
        switch (mop) {
          case CL_FILL: r = f0; break;
          case CL_COPY: r = *a; break;
          case CL_GEAM: r = *a * f0 + *b * f1; break;
          case CL_SCALAR: r = cl_bop(sub, *a, f0); break;
          case CL_BIN: r = cl_bop(sub, *a, *b); break;
          case CL_ACC: r = *d + *a; break;
          case CL_ACCNEG: r = *d + (0.0f - *a); break;
          case CL_ACCMUL: r = *d + *a * *b; break;
          case CL_UNARY: r = cl_unary(sub, *a, f0, f1); break;
          default: {             // CL_UNARY_GRAD: d = dx, a = x, b = y, g = dy
            const bool rh = sub == LH_RELU || sub == LH_HARDTANH;
            const bool need_x = rh ? !inplace : (sub == LH_LOG || sub == LH_SQUARE), need_y = rh ? inplace != 0 : !(sub == LH_LOG || sub == LH_SQUARE), need_g = !(rh && inplace);
            r = cl_unary_grad(sub, inplace, *d, need_x ? *a : 0.f, need_y ? *b : 0.f, need_g ? *g : 0.f, f0, f1);
            break;
          }
        }
        *d = r;
        ((gfloat*)(uintptr_t)SP[(w0 >> 8) & 0xff])[t] = r;
      }
      break;
    }
    case CL_GEMV_N: {            // y[m] = alpha * A[m,n] x[n] + beta * y   (p0 = y, p1 = A, p2 = x; i2 = lda): a wavefront takes
      // up to ten rows at a time and a lane four columns of each, all loads issued before the first product
      const int m = c.i0, n = c.i1, lda = c.i2; const float al = c.f0, be = c.f1;
      const __amdgpu_buffer_rsrc_t rA = cl_rsrc(p1, ((int64_t)(m - 1) * lda + n) * 4), rX = cl_rsrc(p2, (int64_t)n * 4);
      constexpr int RB = 10;
      for (int r0 = gw * RB; r0 < m; r0 += GW * RB) {
        float acc[RB];
#pragma unroll
        for (int u = 0; u < RB; u++) acc[u] = 0.f;
        const float yold = (be != 0.f && lane < RB && r0 + lane < m) ? p0[r0 + lane] : 0.f;  // asked for with the matrix, not after it
        for (int j0 = 0; j0 < n; j0 += 256) {
          float xv[4], av[RB][4];
          const uint32_t co = (uint32_t)(j0 + lane) * 4u;
#pragma unroll
          for (int q = 0; q < 4; q++) xv[q] = cl_ld(rX, co + q * 256u);                  // zero past n
#pragma unroll
          for (int u = 0; u < RB; u++) {
            const uint32_t ro = (uint32_t)(r0 + u) * (uint32_t)lda * 4u + co;            // rows past m lie past the operand's end
#pragma unroll
            for (int q = 0; q < 4; q++) av[u][q] = cl_ld(rA, ro + q * 256u);
          }
          if (j0 + 256 > n) {                                                            // columns past n hold the next row's values
#pragma unroll
            for (int q = 0; q < 4; q++) if (j0 + q * 64 + lane >= n) {
#pragma unroll
              for (int u = 0; u < RB; u++) av[u][q] = 0.f;
            }
          }
#pragma unroll
          for (int u = 0; u < RB; u++)
#pragma unroll
            for (int q = 0; q < 4; q++) acc[u] += av[u][q] * xv[q];
        }
        float sv = 0.f;
#pragma unroll
        for (int u = 0; u < RB; u++) { const float tot = cl_wave_sum_dpp(acc[u]); sv = lane == u ? tot : sv; }
        if (lane < RB && r0 + lane < m) p0[r0 + lane] = al * sv + (be == 0.f ? 0.f : be * yold);
      }
      break;
    }
    case CL_GEMV_T: {            // y[n] = alpha * A[m,n]^T x[m] + beta * y  (p0 = y, p1 = A, p2 = x): a wavefront takes 8 columns
      // (the four wavefronts of a block, side by side in one compute unit, a 128-byte line of every row); lane l holds column
      // l mod 8 of the rows congruent to l / 8 mod 8, up to 20 of them in flight together: 160 rows in one memory round trip.  The
      // eight row classes meet by lane exchange: no LDS, no atomics, and the order of the sum is fixed.
      const int m = c.i0, n = c.i1, lda = c.i2; const float al = c.f0, be = c.f1;
      const __amdgpu_buffer_rsrc_t rA = cl_rsrc(p1, ((int64_t)(m - 1) * lda + n) * 4), rX = cl_rsrc(p2, (int64_t)m * 4);
      const int cj = lane & 7, rg = lane >> 3;
      constexpr int RU = 20;
      for (int j0 = gw * 8; j0 < n; j0 += GW * 8) {
        const int j = j0 + cj;
        const uint32_t co = j < n ? (uint32_t)j * 4u : CL_OOB;
        const float yold = (be != 0.f && rg == 0 && j < n) ? p0[j] : 0.f;               // asked for with the matrix, not after it
        float acc = 0.f;
        for (int i0 = 0; i0 < m; i0 += 8 * RU) {
          float xv[RU], av[RU];
#pragma unroll
          for (int u = 0; u < RU; u++) {
            const uint32_t i = (uint32_t)(i0 + u * 8 + rg);
            xv[u] = cl_ld(rX, i * 4u);                                                   // zero past m
            av[u] = cl_ld(rA, i * (uint32_t)lda * 4u + co);                              // rows past m lie past the operand's end
          }
#pragma unroll
          for (int u = 0; u < RU; u++) acc += av[u] * xv[u];
        }
        acc += __shfl_xor(acc, 8, 64);
        acc += __shfl_xor(acc, 16, 64);
        acc += __shfl_xor(acc, 32, 64);
        if (rg == 0 && j < n) p0[j] = al * acc + (be == 0.f ? 0.f : be * yold);
      }
      break;
    }
    case CL_GER: {               // A[m,n] += u[m] (x) v[n]   (p0 = A, p1 = u, p2 = v): a wavefront takes five rows at a time, a lane
      // four columns of each, all loads in flight together
      const int m = c.i0, n = c.i1;
      const __amdgpu_buffer_rsrc_t rA = cl_rsrc(p0, (int64_t)m * n * 4), rU = cl_rsrc(p1, (int64_t)m * 4), rV = cl_rsrc(p2, (int64_t)n * 4);
      for (int j0 = 0; j0 < n; j0 += 256) {
        float vv[4]; uint32_t co[4];
#pragma unroll
        for (int q = 0; q < 4; q++) { const int j = j0 + q * 64 + lane; co[q] = j < n ? (uint32_t)j * 4u : CL_OOB; vv[q] = cl_ld(rV, co[q]); }
        for (int i0 = gw * 5; i0 < m; i0 += 5 * GW) {
          float uu[5], av[5][4];
#pragma unroll
          for (int u = 0; u < 5; u++) {
            const uint32_t i = (uint32_t)(i0 + u);
            uu[u] = cl_ld(rU, i * 4u);
            const uint32_t ro = i * (uint32_t)n * 4u;
#pragma unroll
            for (int q = 0; q < 4; q++) av[u][q] = cl_ld(rA, ro + co[q]);
          }
#pragma unroll
          for (int u = 0; u < 5; u++) {
            const uint32_t ro = (uint32_t)(i0 + u) * (uint32_t)n * 4u;
#pragma unroll
            for (int q = 0; q < 4; q++) cl_st(rA, ro + co[q], av[u][q] + vv[q] * uu[u]);   // nothing is stored past the operand or the row
          }
        }
      }
      break;
    }
    case CL_DOT: {               // out[0] = x . y   (p0 = out, p1 = x, p2 = y)
      const int n = c.i0;
      float acc = 0.f;
      for (int i = t; i < n; i += ST) acc += p1[i] * p2[i];
      acc = cl_wave_sum_all(acc);
      __shared__ float red[NW];
      if (lane == 0) red[wave] = acc;
      __syncthreads();
      if (wave == 0) { float v = lane < NW ? red[lane] : 0.f; v = cl_wave_sum_all(v); if (lane == 0) p0[0] = v; }
      __syncthreads();           // `red` is free again: the next command of the level may follow without a barrier
      break;
    }
    case CL_AXPY_DEV: {          // y += s[0] * x   (p0 = y, p1 = s, p2 = x)
      const int n = c.i0;
      const float a = *(volatile gfloat*)p1;                 // written by an earlier command: a vector load, not the scalar cache
      for (int i = t; i < n; i += ST) p0[i] = p0[i] + a * p2[i];
      break;
    }
    case CL_SOFTMAX: {           // rows of length cc, a wavefront per row   (p0 = y, p1 = x; i2 = log form)
      const int rows = c.i0, cc = c.i1, is_log = c.i2;
      for (int r = wave; r < rows; r += NW) {
        const gfloat* xp = p1 + (int64_t)r * cc; gfloat* yp = p0 + (int64_t)r * cc;
        float mx = -3.402823466e+38f;
        for (int j = lane; j < cc; j += 64) mx = fmaxf(mx, xp[j]);
        mx = cl_wave_max_all(mx);
        float sum = 0.f;
        for (int j = lane; j < cc; j += 64) sum += expf(xp[j] - mx);
        sum = cl_wave_sum_all(sum);
        if (is_log) { const float ls = mx + logf(sum); for (int j = lane; j < cc; j += 64) yp[j] = xp[j] - ls; }
        else { for (int j = lane; j < cc; j += 64) yp[j] = expf(xp[j] - mx) / sum; }
      }
      break;
    }
    case CL_SOFTMAX_GRAD: {      // p0 = dx (accumulates), p1 = y, p2 = dy; rows of length cc
      const int rows = c.i0, cc = c.i1, is_log = c.i2;
      for (int r = wave; r < rows; r += NW) {
        const int64_t base = (int64_t)r * cc;
        float acc = 0.f;
        for (int j = lane; j < cc; j += 64) acc += is_log ? p2[base + j] : p2[base + j] * p1[base + j];
        acc = cl_wave_sum_all(acc);
        for (int j = lane; j < cc; j += 64) {
          const int64_t i = base + j;
          p0[i] += is_log ? p2[i] - expf(p1[i]) * acc : p1[i] * (p2[i] - acc);
        }
      }
      break;
    }
    case CL_NLL: {               // y[b] = -x[b*stride + target[b]]   (p0 = y, p1 = x, p2 = target)
      const int batch = c.i0, stride = c.i1; const gint* tg = (const gint*)(uintptr_t)c.p2;
      for (int b = t; b < batch; b += ST) p0[b] = -1.0f * p1[(int64_t)b * stride + tg[b]];
      break;
    }
    case CL_NLL_GRAD: {          // dx[b*stride + target[b]] += -dy[b]   (p0 = dx, p1 = dy, p2 = target)
      const int batch = c.i0, stride = c.i1; const gint* tg = (const gint*)(uintptr_t)c.p2;
      for (int b = t; b < batch; b += ST) p0[(int64_t)b * stride + tg[b]] += -1.0f * p1[b];
      break;
    }
    case CL_ADAGRAD: {           // p0 = x, p1 = d, p2 = m
      const int n = c.i0; const float lr = c.f0, clip = c.f1;
      for (int i = t; i < n; i += ST) {
        float g = p1[i];
        if (g > clip) g = clip;
        if (g < -clip) g = -clip;
        const float mm = p2[i] + g * g;
        p2[i] = mm;
        p0[i] -= lr * g / sqrtf(mm + 1e-8f);
        p1[i] = 0.f;
      }
      break;
    }
    case CL_SGD: {               // p0 = x, p1 = d
      const int n = c.i0; const float lr = c.f0;
      for (int i = t; i < n; i += ST) { p0[i] = p0[i] * 1.0f + p1[i] * (-lr); p1[i] = 0.f; }
      break;
    }
    default: break;
  }
}

// One barrier over all workgroups of the launch: everything a workgroup stored before it is visible to every workgroup
// after it (release and acquire at device scope: the workgroups sit on different XCDs with their own L2).  `sync[0]` counts
// arrivals over the life of the library (64 bits; `target` is the count this barrier completes at), `sync[1]` is set by a
// workgroup whose wait ran out, which makes every workgroup leave the kernel: a lost workgroup cannot hang the device.
__device__ __forceinline__ bool cl_grid_barrier(unsigned long long* sync, unsigned long long target, int* lds_flag, unsigned* host_flag) {
  __syncthreads();                                       // every wavefront's stores are issued before wavefront 0 releases them
  if (threadIdx.x == 0) {
    __hip_atomic_fetch_add(sync, 1ull, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    long spins = 0;
    int gave_up = 0;
    while (__hip_atomic_load(sync, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
      if (++spins > CL_SPIN_LIMIT || __hip_atomic_load(sync + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0ull) {
        __hip_atomic_store(sync + 1, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *(volatile unsigned*)host_flag = 1u;              // pinned host memory: the host sees it without waiting for the stream
        gave_up = 1;
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    *lds_flag = gave_up;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");   // the caches this workgroup reads through drop what other workgroups have since replaced
  }
  __syncthreads();
  return *lds_flag == 0;
}

// dir, ops, cmds: the device copy of a buffer.  Each workgroup has its own list, in execution order: level by level, an entry saying
// how many barriers over all workgroups come before it (every list passes the same number of barriers in all).  A list is staged
// in LDS 256 entries at a time (the next chunk is fetched while the current one runs).  Every wavefront of the workgroup walks the
// op words (8 bytes an entry, read one ahead and made wave-uniform: the walk is scalar work, and the one scalar unit of a compute
// unit serves all 16 wavefronts, which is why a list holds only what its workgroup has a part in) and reads the 64-byte command
// only when a piece of it is its own.
__global__ void __launch_bounds__(CL_THREADS) k_cmdlist(const uint2* dir, const uint2* ops_all, const LhCmd* cmds_all, unsigned long long* sync,
                                                        unsigned long long sync_base, unsigned* host_flag, unsigned long long* trace) {
  __shared__ uint4 stage[CL_CHUNK * 4];                 // 256 commands of 64 bytes
  __shared__ uint2 sop[CL_CHUNK + 1];
  extern __shared__ float slots[];                      // Ring::nslot slots of CL_SLOT_ELEMS floats
  __shared__ uint64_t slot_ptr[CL_NSLOT_MAX];
  __shared__ int gave_up;
  constexpr int NW = CL_THREADS / 64;
  const int t = threadIdx.x, grp = blockIdx.x, ngrp = gridDim.x;
  const int w0 = __builtin_amdgcn_readfirstlane(t >> 6);
  const int all_w = ngrp * NW, my_w = ((w0 / CL_WBLOCK) * ngrp + grp) * CL_WBLOCK + w0 % CL_WBLOCK;      // this wavefront among all of the launch
  const uint32_t first = __builtin_amdgcn_readfirstlane(dir[grp].x);
  const int n = __builtin_amdgcn_readfirstlane((int)dir[grp].y);
  const uint2* ops = ops_all + first;
  const uint4* src = reinterpret_cast<const uint4*>(cmds_all + first);
  const int total16 = n * 4;
  unsigned long long arrived = sync_base;
  int tr_k = 0;
  if (trace && grp == 0 && t == 0) trace[tr_k++] = wall_clock64();
  uint4 next = make_uint4(0, 0, 0, 0);
  uint2 next_op = make_uint2(0, 0);
  if (t < total16) next = src[t];
  if (t < CL_CHUNK) next_op = ops[t];                   // op words are allocated a chunk past the last list
  for (int base = 0; base < n; base += CL_CHUNK) {
    stage[t] = next;
    if (t < CL_CHUNK) sop[t] = next_op;
    const int nb = base + CL_CHUNK;
    if (nb < n) {
      if (nb * 4 + t < total16) next = src[nb * 4 + t];
      if (t < CL_CHUNK) next_op = ops[nb + t];
    }
    __syncthreads();
    const int cnt = n - base < CL_CHUNK ? n - base : CL_CHUNK;
    const LhCmd* list = reinterpret_cast<const LhCmd*>(stage);
    uint2 ahead = sop[0];
    for (int i = 0; i < cnt; i++) {
      const uint32_t op = __builtin_amdgcn_readfirstlane(ahead.x);
      const int pieces = (int)__builtin_amdgcn_readfirstlane(ahead.y);
      ahead = sop[i + 1];
      for (int b = (int)(op >> CL_BARRIERS_SHIFT); b > 0; b--) {      // levels completed: their stores become visible
        if (ngrp == 1) __syncthreads();
        else { arrived += (unsigned long long)ngrp; if (!cl_grid_barrier(sync, arrived, &gave_up, host_flag)) return; }
        if (trace && grp == 0 && t == 0) trace[tr_k++] = wall_clock64();
      }
      const int start = (int)(op >> CL_START_SHIFT) & 0xfff;
      int gw, GW;
      if (op & CL_SPLIT) {
        gw = my_w - start; if (gw < 0) gw += all_w;
        GW = all_w;
      } else {
        gw = (w0 + NW - start) & (NW - 1);
        GW = NW;
      }
      if (gw >= pieces) continue;                       // no part of this command falls to this wavefront
      cl_run(list[i], (int)(op & CL_OP_MASK), gw, GW, slots, slot_ptr);
    }
    __syncthreads();                                    // the staged commands are no longer read
  }
  if (trace && grp == 0 && t == 0) trace[tr_k++] = wall_clock64();
}

static bool ring_init() {
  if (g_ring.ready) return true;
  for (int i = 0; i < CL_NBUF; i++) {
    if (hipHostMalloc((void**)&g_ring.host[i], CL_BUF_BYTES, hipHostMallocDefault) != hipSuccess) { LH_FAIL("command list: pinned buffer allocation failed"); return false; }
    if (hipEventCreateWithFlags(&g_ring.done[i], hipEventDisableTiming) != hipSuccess) { LH_FAIL("command list: event creation failed"); return false; }
    g_ring.busy[i] = false;
  }
  if (hipMalloc((void**)&g_ring.mirror, CL_BUF_BYTES) != hipSuccess) { LH_FAIL("command list: cannot allocate the device copy of a buffer"); return false; }
  if (hipMalloc((void**)&g_ring.sync, 2 * sizeof(unsigned long long)) != hipSuccess || hipMemset(g_ring.sync, 0, 2 * sizeof(unsigned long long)) != hipSuccess) {
    LH_FAIL("command list: cannot allocate the barrier words"); return false;
  }
  g_ring.sync_base = 0;
  if (hipHostMalloc((void**)&g_ring.host_flag, 64, hipHostMallocDefault) != hipSuccess || hipHostGetDevicePointer((void**)&g_ring.host_flag_dev, g_ring.host_flag, 0) != hipSuccess) {
    LH_FAIL("command list: cannot allocate the pinned flag"); return false;
  }
  *g_ring.host_flag = 0;
  // Workgroups per launch.  More of them draw a level's matrices faster (a compute unit gets some 25 GB/s) and make the barrier
  // dearer; on the sentiment TreeLSTM 4 / 8 / 16 / 24 / 32 / 48 / 64 workgroups give 593 / 803 / 981 / 1058 / 1105 / 1114 / 1095
  // trees a second.  LH_CMDLIST_GROUPS overrides.
  int groups = 32;
  if (const char* e = getenv("LH_CMDLIST_GROUPS")) groups = atoi(e);
  if (const char* e = getenv("LH_CMDLIST_CHAINS")) g_chains = atoi(e) != 0;
  if (const char* e = getenv("LH_CMDLIST_SLOTS")) g_slots = atoi(e) != 0;
  if (groups < 1) groups = 1;
  if (groups > CL_MAX_GROUPS) groups = CL_MAX_GROUPS;
  if (groups > g_num_cu / 4) groups = g_num_cu / 4 > 0 ? g_num_cu / 4 : 1;       // all workgroups of a launch must be resident together
  g_ring.groups = groups;
  // LDS for the operand slots of chain programs: all the device gives a workgroup beyond the kernel's fixed 20 KB, 128 slots at most
  g_ring.nslot = 44;
  {
    int lds = 0, dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) == hipSuccess && lds > 0) {
      int want = (lds - 20 * 1024) / (CL_SLOT_ELEMS * 4);
      if (want > CL_NSLOT_MAX) want = CL_NSLOT_MAX;
      if (want > 44 && hipFuncSetAttribute(reinterpret_cast<const void*>(&k_cmdlist), hipFuncAttributeMaxDynamicSharedMemorySize, want * CL_SLOT_ELEMS * 4) == hipSuccess) g_ring.nslot = want;
      else (void)hipGetLastError();
    }
    if (const char* e = getenv("LH_CMDLIST_NSLOT")) { const int v = atoi(e); if (v >= 0 && v <= g_ring.nslot) g_ring.nslot = v; }
  }
  g_ring.cur = 0; g_ring.ready = true;
  return true;
}
}  // namespace

#include "lh_cmdlist_levels.h"
namespace { static Window* g_win = nullptr; }

static inline void memcpy_host(void* d, const void* s_, size_t nbytes) { __builtin_memcpy(d, s_, nbytes); }
namespace lh {
static long long g_stat_slot_chains = 0, g_stat_slots = 0, g_stat_chain_ptrs = 0;
static unsigned long long g_tsc_push = 0, g_tsc_flush = 0, g_tsc_wait = 0;      // host cycles spent recording (LH_CMDLIST_VERBOSE prints them)
// Hands the recorded buffer to the device: commands in level order (recording order within a level), the first of each
// level flagged for a barrier, each with the wavefront its elements start on.
// An interpreter launch whose barrier wait ran out leaves a flag in pinned host memory.  Whoever looks next (the next
// hand-over, lh_cmdlist_end, lh_sync, lh_d2h) reports it, with the barrier counters and the window put back so that the
// library stays usable; the results of that buffer are incomplete.
bool cmdlist_report_timeout() {
  Ring& r = g_ring;
  if (r.host_flag == nullptr || *(volatile unsigned*)r.host_flag == 0) return false;
  (void)hipStreamSynchronize(g_stream_raw);
  (void)hipMemset(r.sync, 0, 2 * sizeof(unsigned long long));
  *r.host_flag = 0; r.sync_base = 0;
  if (g_win) window_reset(*g_win);
  g_rec_pending = 0;
  LH_FAIL("command list: a barrier between workgroups timed out; the commands of that buffer did not all run");
  return true;
}
void rec_flush() {
  if (cmdlist_report_timeout()) return;
  if (g_rec_pending <= 0 || g_win == nullptr) return;
  const unsigned long long f0 = __builtin_ia32_rdtsc();
  Window& W = *g_win;
  const int n = W.n;
  g_rec_pending = 0;                                  // before any use of the stream below
  Ring& r = g_ring;
  const int groups = r.groups, all_w = groups * (CL_THREADS / 64);
  static int start[CL_BUF_CMDS + 2], order[CL_BUF_CMDS];
  for (int l = 0; l <= W.top + 1; l++) start[l] = 0;
  for (int i = 0; i < n; i++) start[W.level[i] + 1]++;
  for (int l = 1; l <= W.top + 1; l++) start[l] += start[l - 1];
  for (int i = 0; i < n; i++) order[start[W.level[i]]++] = i;
  static int rot_of_level[CL_BUF_CMDS + 2], owner_of_level[CL_BUF_CMDS + 2], split_of_level[CL_BUF_CMDS + 2];
  for (int l = 0; l <= W.top; l++) { rot_of_level[l] = 0; owner_of_level[l] = 0; split_of_level[l] = 0; }
  static int chain_place[CL_BUF_CMDS + 1];
  for (int ch = 0; ch < W.nchains; ch++) chain_place[ch] = -1;
  // Pass 1: where each command runs.
  struct Place { uint32_t op, pieces; int g0, gn; };
  static Place place[CL_BUF_CMDS];
  for (int k = 0; k < n; k++) {
    const int i = order[k], l = W.level[i];
    const LhCmd& c = W.cmd[i];
    // a command that one workgroup runs alone goes to the next workgroup in turn, its first elements to the next free wavefront
    // there; the pieces of a split command start where those of the level's previous split command ended
    int owner = 0, at;
    const bool split = cmd_splits(c);
    const int waves = c.op == CL_DOT ? 0xffff : (cmd_waves(c) < 0xffff ? cmd_waves(c) : 0xffff);
    if (split && W.chain[i] >= 0 && chain_place[W.chain[i]] >= 0) {     // a later matrix command of a chain: the wavefronts of its first one
      at = chain_place[W.chain[i]];
    } else if (split) {
      at = split_of_level[l] % all_w;
      split_of_level[l] += waves;
      if (W.chain[i] >= 0) chain_place[W.chain[i]] = at;
    } else if (W.chain[i] >= 0 && chain_place[W.chain[i]] >= 0) {          // a later command of a chain: where its first one runs
      owner = chain_place[W.chain[i]] >> 4; at = chain_place[W.chain[i]] & 15;
    } else {
      owner = owner_of_level[l] % groups;
      at = rot_of_level[l] & 15;
      owner_of_level[l]++;
      if (owner_of_level[l] % groups == 0) rot_of_level[l] = (rot_of_level[l] + waves) & 15;
      if (W.chain[i] >= 0) chain_place[W.chain[i]] = (owner << 4) | at;
    }
    Place& pl = place[k];
    pl.op = (uint32_t)c.op | (split ? (uint32_t)CL_SPLIT : 0u) | ((uint32_t)at << CL_START_SHIFT);
    pl.pieces = (uint32_t)waves;
    if (split) {
      const int span = waves < all_w ? waves : all_w, b0 = at / CL_WBLOCK, b1 = (at + span - 1) / CL_WBLOCK;
      pl.g0 = b0 % groups; pl.gn = b1 - b0 + 1 < groups ? b1 - b0 + 1 : groups;
    } else { pl.g0 = owner; pl.gn = 1; }
  }
  const int barriers = W.top > 1 ? W.top - 1 : 0;
  // Chain programs.  The commands of an element-wise chain run one after the other on the same few wavefronts, and what one such
  // command costs is not memory but the interpreter: some 280 dependent instructions of one wavefront, 0.7 us.  A chain of at least
  // PROGRAM_MIN_CHAIN commands, all of kinds that write one result, none longer than an LDS slot, whose distinct operand addresses
  // all get a slot of its workgroup (Ring::nslot per workgroup and level), becomes ONE entry of kind CL_CHAIN followed by its
  // commands packed 16 bytes each (operation, slots, length, two scalars).  The workgroup loads every slotted vector, and notes its
  // address, before its first entry of the level (entries of kind CL_PRELOAD on different wavefronts, then one CL_SYNC); the chain's
  // wavefronts then run the packed commands from LDS to LDS, writing every result through to memory.
  struct ChainProg { int count, nptr, head, owner, level, pieces, base, next, first_k, last_k; bool ok, programmed, emitted; };
  struct ChainPtr { const void* p; int maxn, idx, next; };
  static ChainProg cs[CL_BUF_CMDS + 1];
  static ChainPtr cp[CL_BUF_CMDS * 4];
  static uint32_t ptr_index[CL_BUF_CMDS];                      // per command (by position in `order`): the chain-local index of each pointer, a byte each
  static int next_in_chain[CL_BUF_CMDS];
  static uint8_t slots_used[CL_BUF_CMDS + 2][CL_MAX_GROUPS];
  static int16_t bucket[CL_BUF_CMDS + 2][CL_MAX_GROUPS];       // the programmed chains of a (level, workgroup), linked through ChainProg::next
  constexpr int PROGRAM_MIN_CHAIN = 6, SEGMENT = 128;          // commands of one CL_CHAIN entry at most (32 entries of payload behind it)
  const bool use_programs = g_chains && g_slots;
  for (int ch = 0; ch < W.nchains; ch++) { cs[ch].count = 0; cs[ch].programmed = false; cs[ch].emitted = false; }
  if (use_programs) {
    int ncp = 0;
    for (int l = 0; l <= W.top; l++) for (int g = 0; g < groups; g++) { slots_used[l][g] = 0; bucket[l][g] = -1; }
    for (int k = 0; k < n; k++) {
      const int i = order[k], ch = W.chain[i];
      if (ch < 0 || W.chain_class[ch] != 1) continue;
      const LhCmd& c = W.cmd[i];
      ChainProg& C = cs[ch];
      if (C.count == 0) { C.nptr = 0; C.head = -1; C.owner = place[k].g0; C.level = W.level[i]; C.pieces = 1; C.ok = true; C.first_k = k; }
      else next_in_chain[C.last_k] = k;
      C.last_k = k; next_in_chain[k] = -1;
      C.count++;
      if (c.op == CL_ADAGRAD || c.op == CL_SGD || c.i0 > CL_SLOT_ELEMS) C.ok = false;
      if (!C.ok) continue;
      if ((int)place[k].pieces > C.pieces) C.pieces = (int)place[k].pieces;
      const void* ptrs[4] = {c.p0, c.p1, c.p2, c.p3};
      uint32_t word = 0;
      for (int q = 0; q < 4; q++) {
        uint32_t idx = 0xff;
        if (ptrs[q]) {
          int e = C.head;
          while (e >= 0 && cp[e].p != ptrs[q]) e = cp[e].next;
          if (e < 0 && C.nptr < r.nslot) { e = ncp++; cp[e].p = ptrs[q]; cp[e].maxn = 0; cp[e].idx = C.nptr++; cp[e].next = C.head; C.head = e; }
          if (e < 0) C.ok = false;                              // more distinct operands than a workgroup has slots
          else { if (c.i0 > cp[e].maxn) cp[e].maxn = c.i0; idx = (uint32_t)cp[e].idx; }
        }
        word |= idx << (8 * q);
      }
      ptr_index[k] = word;
    }
    for (int ch = 0; ch < W.nchains; ch++) {
      ChainProg& C = cs[ch];
      if (C.count < PROGRAM_MIN_CHAIN || !C.ok || W.chain_class[ch] != 1) continue;
      uint8_t& used = slots_used[C.level][C.owner];
      if (C.nptr > r.nslot - used) continue;                  // the workgroup's slots of this level are taken: the chain runs command by command
      C.base = used; used = (uint8_t)(used + C.nptr);
      C.programmed = true;
      g_stat_slot_chains++; g_stat_slots += C.nptr; g_stat_chain_ptrs += C.count;
      C.next = bucket[C.level][C.owner]; bucket[C.level][C.owner] = (int16_t)ch;
    }
  }
  // Pass 2: the entries in the order they are made, each tagged with its workgroup; then every workgroup's entries are gathered
  // into its list in the buffer.
  struct Rec { LhCmd cmd; uint32_t op, pieces; int g; };
  static Rec* recs = nullptr;
  if (!recs) recs = new Rec[CL_CAP + CL_BUF_CMDS];
  int nrec = 0;
  int list_at[CL_MAX_GROUPS], list_n[CL_MAX_GROUPS], passed[CL_MAX_GROUPS], at_level[CL_MAX_GROUPS], total = 0;
  auto put1 = [&](int g, uint32_t op, uint32_t pieces, const void* cmd64) {        // one entry on workgroup g's list
    if (nrec < CL_CAP + CL_BUF_CMDS) { Rec& rc = recs[nrec]; rc.g = g; rc.op = op; rc.pieces = pieces; if (cmd64) memcpy_host(&rc.cmd, cmd64, sizeof(LhCmd)); }
    nrec++;
    list_n[g]++;
  };
  auto put = [&](int g, uint32_t op, uint32_t pieces, const void* cmd64, int l) {  // ... that belongs to level l: the barriers passed since come with it
    int need = l - 1 - passed[g];
    passed[g] = l - 1;
    for (; need > 255; need -= 255) put1(g, (uint32_t)CL_NOP | (255u << CL_BARRIERS_SHIFT), 0u, nullptr);
    put1(g, op | ((uint32_t)need << CL_BARRIERS_SHIFT), pieces, cmd64);
  };
  // the first entry of workgroup g at level l is about to be put: the level's preloads come before it
  auto open_level = [&](int g, int l) {
    at_level[g] = l;
    if (!use_programs || bucket[l][g] < 0) return;
    int rot = 0;
    for (int ch = bucket[l][g]; ch >= 0; ch = cs[ch].next) {
      const ChainProg& C = cs[ch];
      LhCmd pc = LhCmd{}; int filled = 0;
      for (int e = C.head; e >= 0; e = cp[e].next) {
        const uint32_t nn = (uint32_t)cp[e].maxn, sl = (uint32_t)(C.base + cp[e].idx);
        switch (filled) {
          case 0: pc = LhCmd{}; pc.op = CL_PRELOAD; pc.p0 = (void*)cp[e].p; pc.i0 = (int32_t)nn; pc.i1 = (int32_t)sl; break;
          case 1: pc.p1 = (void*)cp[e].p; pc.i0 = (int32_t)((uint32_t)pc.i0 | (nn << 16)); pc.i1 = (int32_t)((uint32_t)pc.i1 | (sl << 8)); break;
          case 2: pc.p2 = (void*)cp[e].p; pc.i2 = (int32_t)nn; pc.i1 = (int32_t)((uint32_t)pc.i1 | (sl << 16)); break;
          default: pc.p3 = (void*)cp[e].p; pc.i2 = (int32_t)((uint32_t)pc.i2 | (nn << 16)); pc.i1 = (int32_t)((uint32_t)pc.i1 | (sl << 24)); break;
        }
        if (++filled == 4 || cp[e].next < 0) {
          put(g, (uint32_t)CL_PRELOAD | ((uint32_t)(rot & 15) << CL_START_SHIFT), (uint32_t)C.pieces, &pc, l);
          rot += C.pieces; filled = 0;
        }
      }
    }
    LhCmd sync = LhCmd{}; sync.op = CL_SYNC;
    put(g, (uint32_t)CL_SYNC, 0xffffu, &sync, l);
  };
  // a programmed chain, at the place of its first command: CL_CHAIN entries of up to SEGMENT commands, each followed by its packed commands
  auto put_chain = [&](int g, int ch, int l, uint32_t place_op) {
    ChainProg& C = cs[ch];
    int k = C.first_k;
    while (k >= 0) {
      int seg = 0;
      for (int kk = k; kk >= 0 && seg < SEGMENT; kk = next_in_chain[kk]) seg++;
      const int payload = (seg + 3) / 4;
      if (passed[g] < l - 1) put(g, (uint32_t)CL_NOP, 0u, nullptr, l);                   // the barriers before the chain, on an entry of their own
      // the entry and its payload sit in one staged chunk of the list
      while ((list_n[g] % CL_CHUNK) + 1 + payload > CL_CHUNK) put1(g, (uint32_t)CL_NOP, 0u, nullptr);
      LhCmd head = LhCmd{}; head.op = CL_CHAIN; head.i0 = seg;
      put1(g, (uint32_t)CL_CHAIN | (place_op & (0xfffu << CL_START_SHIFT)), (uint32_t)C.pieces, &head);
      uint32_t pack[16]; int filled = 0;
      for (int m = 0; m < seg; m++, k = next_in_chain[k]) {
        const LhCmd& c = W.cmd[order[k]];
        uint32_t sl[4];
        for (int q = 0; q < 4; q++) { const uint32_t idx = (ptr_index[k] >> (8 * q)) & 0xffu; sl[q] = idx == 0xffu ? 0u : (uint32_t)C.base + idx; }
        union { float f; uint32_t u; } f0, f1; f0.f = c.f0; f1.f = c.f1;
        uint32_t* w = pack + 4 * filled;
        w[0] = (uint32_t)c.op | (sl[0] << 8) | (sl[1] << 16) | (sl[2] << 24);
        w[1] = sl[3] | (((uint32_t)c.i1 & 0x7fu) << 8) | ((c.i2 ? 1u : 0u) << 15) | ((uint32_t)c.i0 << 16);
        w[2] = f0.u; w[3] = f1.u;
        if (++filled == 4 || m + 1 == seg) { for (int z = 4 * filled; z < 16; z++) pack[z] = 0; put1(g, (uint32_t)CL_NOP, 0u, pack); filled = 0; }
      }
    }
    C.emitted = true;
  };
  auto emit_all = [&]() {
    for (int g = 0; g < groups; g++) { list_n[g] = 0; passed[g] = 0; at_level[g] = 0; }
    for (int ch = 0; ch < W.nchains; ch++) cs[ch].emitted = false;
    for (int k = 0; k < n; k++) {
      const int i = order[k], l = W.level[i], ch = W.chain[i];
      const Place& pl = place[k];
      for (int j = 0; j < pl.gn; j++) {
        const int g = (pl.g0 + j) % groups;
        if (at_level[g] != l) open_level(g, l);
        if (ch >= 0 && cs[ch].programmed) { if (!cs[ch].emitted) put_chain(g, ch, l, pl.op); }
        else put(g, pl.op, pl.pieces, &W.cmd[i], l);
      }
    }
    for (int g = 0; g < groups; g++) if (passed[g] < barriers) put(g, (uint32_t)CL_NOP, 0u, nullptr, barriers + 1);
  };
  emit_all();
  for (int g = 0; g < groups; g++) { list_at[g] = total; total += list_n[g]; }
  if (total > CL_CAP || nrec != total) { window_reset(W); LH_FAIL("command list: %d entries exceed a buffer (%d)", nrec, CL_CAP); return; }
  uint2* dir = reinterpret_cast<uint2*>(r.host[r.cur]);
  LhCmd* out = reinterpret_cast<LhCmd*>(r.host[r.cur] + CL_DIR_BYTES);
  uint2* ops = reinterpret_cast<uint2*>(out + total);
  for (int g = 0; g < groups; g++) { dir[g] = make_uint2((uint32_t)list_at[g], (uint32_t)list_n[g]); list_n[g] = 0; }
  for (int q = 0; q < nrec; q++) {
    const Rec& rc = recs[q];
    const int at = list_at[rc.g] + list_n[rc.g]++;
    ops[at] = make_uint2(rc.op, rc.pieces);
    memcpy_host(&out[at], &rc.cmd, sizeof(LhCmd));
  }
  g_ring.levels += W.top;
  // LH_CMDLIST_TRACE=<launch>: workgroup 0 notes the time of every barrier of that launch and the next one; the host prints how long
  // each level took and what it held (a diagnostic: the launch is waited for)
  static unsigned long long* trace_buf = nullptr; static int trace_from = -1;
  if (trace_from == -1) { const char* e = getenv("LH_CMDLIST_TRACE"); trace_from = e ? atoi(e) : -2; if (e && hipHostMalloc((void**)&trace_buf, 8 * (CL_BUF_CMDS + 2), hipHostMallocDefault) != hipSuccess) trace_from = -2; }
  const bool tracing = trace_from >= 0 && r.launches >= trace_from && r.launches < trace_from + 2;
  static int tr_counts[CL_BUF_CMDS + 1][7], tr_len[CL_BUF_CMDS + 1];       // per level: element-wise, gemv, gemv_t, ger, other, chains, longest chain
  const int tr_levels = W.top;
  if (tracing) {
    for (int l = 0; l <= tr_levels; l++) for (int k = 0; k < 7; k++) tr_counts[l][k] = 0;
    for (int c = 0; c <= W.nchains; c++) tr_len[c] = 0;
    for (int i = 0; i < n; i++) {
      const int l = W.level[i], o = W.cmd[i].op;
      tr_counts[l][o == CL_GEMV_N ? 1 : o == CL_GEMV_T ? 2 : o == CL_GER ? 3 : cmd_lanewise(W.cmd[i]) ? 0 : 4]++;
      if (W.chain[i] >= 0) { const int L = ++tr_len[W.chain[i]]; if (L == 1) tr_counts[l][5]++; if (L > tr_counts[l][6]) tr_counts[l][6] = L; }
    }
  }
  window_reset(W);
  ProfScope prof_(CAT_CMDLIST);
  hipError_t e = hipMemcpyAsync(r.mirror, r.host[r.cur], CL_DIR_BYTES + (sizeof(LhCmd) + sizeof(uint2)) * (size_t)total, hipMemcpyHostToDevice, g_stream_raw);
  if (e != hipSuccess) { LH_FAIL("command list copy: %s", hipGetErrorString(e)); return; }
  hipLaunchKernelGGL(k_cmdlist, dim3(groups), dim3(CL_THREADS), (size_t)r.nslot * CL_SLOT_ELEMS * 4, g_stream_raw, reinterpret_cast<const uint2*>(r.mirror),
                     reinterpret_cast<const uint2*>(r.mirror + CL_DIR_BYTES + sizeof(LhCmd) * (size_t)total), reinterpret_cast<const LhCmd*>(r.mirror + CL_DIR_BYTES),
                     r.sync, r.sync_base, r.host_flag_dev, tracing ? trace_buf : nullptr);
  if (tracing) {
    (void)hipStreamSynchronize(g_stream_raw);
    fprintf(stderr, "command list launch %lld: %d commands, %d levels, %.1f us\n", (long long)r.launches, n, tr_levels, (trace_buf[tr_levels] - trace_buf[0]) * 0.01);
    for (int l = 1; l <= tr_levels; l++)
      fprintf(stderr, "  level %3d: %6.2f us  element-wise %3d gemv %3d gemv_t %3d ger %3d other %3d chains %3d longest %3d\n", l, (trace_buf[l] - trace_buf[l - 1]) * 0.01,
              tr_counts[l][0], tr_counts[l][1], tr_counts[l][2], tr_counts[l][3], tr_counts[l][4], tr_counts[l][5], tr_counts[l][6]);
  }
  if (groups > 1) r.sync_base += (unsigned long long)barriers * (unsigned long long)groups;
  e = hipGetLastError();
  if (e == hipSuccess) e = hipEventRecord(r.done[r.cur], g_stream_raw);
  if (e != hipSuccess) { LH_FAIL("command list launch: %s", hipGetErrorString(e)); return; }
  r.busy[r.cur] = true;
  r.launches++;
  r.cur = (r.cur + 1) % CL_NBUF;
  if (r.busy[r.cur]) {                                // the buffer about to be refilled must have been consumed
    const unsigned long long w0 = __builtin_ia32_rdtsc();
    (void)hipEventSynchronize(r.done[r.cur]);
    g_tsc_wait += __builtin_ia32_rdtsc() - w0;
    r.busy[r.cur] = false;
  }
  g_tsc_flush += __builtin_ia32_rdtsc() - f0;
}
// Appends a command: works out its level from the ranges it touches, then notes those ranges.
bool rec_push(const LhCmd& c) {
  if (!g_ring.ready || g_win == nullptr) return false;
  const unsigned long long tsc0 = __builtin_ia32_rdtsc();
  struct Acc { unsigned long long t0; ~Acc() { g_tsc_push += __builtin_ia32_rdtsc() - t0; } } acc_{tsc0};
  Window& W = *g_win;
  // the lists of how many workgroups the command goes on (an upper bound; the barrier-only entries are allowed for below)
  int copies = cmd_lanewise(c) ? 3 : 1;             // an element-wise command may bring a CL_PRELOAD and a CL_SYNC entry with it
  if (cmd_splits(c)) {
    const int all_w = g_ring.groups * (CL_THREADS / 64), span = cmd_waves(c) < all_w ? cmd_waves(c) : all_w;
    copies = (span + CL_WBLOCK - 2) / CL_WBLOCK + 1;
    if (copies > g_ring.groups) copies = g_ring.groups;
  }
  for (int attempt = 0; attempt < 2; attempt++) {
    // (a chain program is padded so that it does not straddle two staged chunks: up to 33 entries per 256, allowed for here)
    if (W.n == CL_BUF_CMDS || W.entries + copies + g_ring.groups * 10 > CL_CAP - CL_BUF_CMDS) { rec_flush(); if (failed()) return false; }
    int lv = 0, chain = -1;
    if (!window_place(W, c, g_chains, lv, chain)) { rec_flush(); if (failed()) return false; continue; }       // a table is full: start a new buffer (which begins with a barrier)
    W.entries += copies;
    g_rec_pending = W.n;
    g_ring.recorded++;
    return true;
  }
  LH_FAIL("command list: a single command overflows the dependence tables");
  return false;
}
void cmdlist_release() {
  g_rec_on = 0; g_rec_pending = 0;
  delete g_win; g_win = nullptr;
  if (!g_ring.ready) return;
  for (int i = 0; i < CL_NBUF; i++) { (void)hipEventDestroy(g_ring.done[i]); (void)hipHostFree(g_ring.host[i]); }
  if (g_ring.sync) (void)hipFree(g_ring.sync);
  if (g_ring.mirror) (void)hipFree(g_ring.mirror);
  if (g_ring.host_flag) (void)hipHostFree(g_ring.host_flag);
  g_ring = Ring{};
}
}  // namespace lh

extern "C" {
void lh_cmdlist_begin(void) {
  LH_REQUIRE(g_stream_raw != nullptr, "lh_cmdlist_begin before lh_setup");
  LH_REQUIRE(!g_capturing, "lh_cmdlist_begin: a graph is being recorded (the command buffers cannot be replayed)");
  LH_REQUIRE(g_stream_cur == g_stream_raw, "lh_cmdlist_begin on the side stream");
  { LZ_SCOPE(); lazy::flush_all(); }     // recorded commands do not pass through the deferred-work bookkeeping: it starts empty and stays empty while recording
  if (!ring_init()) return;
  if (g_win == nullptr) g_win = window_new();
  g_rec_on = 1;
}
void lh_cmdlist_end(void) {
  rec_flush();
  g_rec_on = 0;
  (void)cmdlist_report_timeout();
  if (getenv("LH_CMDLIST_VERBOSE")) fprintf(stderr, "command list: %lld commands in %lld levels, %lld launches\n", (long long)g_ring.recorded, (long long)g_ring.levels, (long long)g_ring.launches);
  if (getenv("LH_CMDLIST_VERBOSE")) fprintf(stderr, "command list: %d operand slots per workgroup\n", g_ring.nslot);
  if (getenv("LH_CMDLIST_VERBOSE")) fprintf(stderr, "command list: %lld chains run as programs, %lld operand slots, %lld commands in them\n", g_stat_slot_chains, g_stat_slots, g_stat_chain_ptrs);
  if (getenv("LH_CMDLIST_VERBOSE")) fprintf(stderr, "command list host cycles: push %.1f M (flush inside %.1f M, of which waiting for a free buffer %.1f M)\n", g_tsc_push * 1e-6, g_tsc_flush * 1e-6, g_tsc_wait * 1e-6);
}
void lh_cmdlist_inject_timeout(void) {
  LH_REQUIRE(g_ring.host_flag != nullptr, "lh_cmdlist_inject_timeout before the first lh_cmdlist_begin");
  *(volatile unsigned*)g_ring.host_flag = 1u;       // what a workgroup whose barrier wait ran out writes
}
void lh_cmdlist_stats(int64_t* recorded, int64_t* launches) {
  if (recorded) *recorded = g_ring.recorded;
  if (launches) *launches = g_ring.launches;
}
}  // extern "C"
