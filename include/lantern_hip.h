/*
 * lantern_hip.h -- C ABI of the MI355X (gfx950) tensor backend for Lantern.
 *
 * One entry point per method of Lantern's `Backend` trait that touches device
 * data (reference: src/main/scala/lantern/TensorDifferentiation.scala:137-379,
 * "TD" below), shaped the way the code generator emits calls for the cuBLAS /
 * cuDNN backend it stands in for ("CUB" = src/main/scala/lantern/
 * TensorDslCublas.scala, "CDN" = .../TensorDslCudnn.scala, "API" =
 * .../DslAPI.scala, "CPU" = .../TensorDslCPU.scala).
 *
 * Contract
 *  - Plain pointers and sizes only.  Every `float*` / `int*` is a DEVICE pointer
 *    unless its name starts with `h_`; shape arrays (`*dims`, `*perm`, `*sizes`)
 *    and pointer tables are HOST arrays read during the call.
 *  - Dense row-major fp32, NCHW.  Every `*_grad` / `*_bwd*` entry ACCUMULATES
 *    (+=) into its gradient outputs unless a `beta` argument says otherwise
 *    (beta = 1 accumulate, beta = 0 overwrite), as the reference's backends do
 *    (cuDNN calls with beta = 1: CDN:681, 756, 829, 1106).
 *  - One caller thread; calls are enqueued on one library-owned stream in
 *    program order and return without waiting.  lh_d2h and lh_sync wait.
 *  - Errors: like the reference's CUDA_CALL macros (API:435-451) a failing call
 *    prints "file:line: message" and exits the process.  A host that prefers
 *    to handle errors calls lh_set_error_mode(1): the failing entry point then
 *    returns early and lh_last_error() holds the message.
 *  - Outputs and gradients are caller-provided, normally from the arena below.
 *    Operators call no hipMalloc: convolution takes its filter-layout scratch
 *    from the top of the arena and pops it before returning (stream order
 *    keeps that safe); batch norm uses a fixed device-resident partials
 *    array; the multi-tensor optimizer entry points keep their pointer
 *    table (up to 65536 tensors) in memory that lh_setup reserved.
 */
#ifndef LANTERN_HIP_H
#define LANTERN_HIP_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* ---- operator codes ---------------------------------------------------- */
enum { LH_ADD = 0, LH_SUB = 1, LH_MUL = 2, LH_DIV = 3 };
enum { LH_RELU = 0, LH_TANH = 1, LH_SIGMOID = 2, LH_EXP = 3, LH_LOG = 4, LH_SQRT = 5, LH_SQUARE = 6, LH_HARDTANH = 7 };

/* ---- lifetime, errors -------------------------------------------------- */
/* Backend.setup/cleanup (TD:139-142; CUB:113-131): one device arena of
 * heap_bytes (the reference hard-codes 8 GiB, API:385; here it is an argument). */
void lh_setup(size_t heap_bytes);
void lh_cleanup(void);
void lh_set_error_mode(int mode);           /* 0 = print and exit (reference), 1 = record and return */
const char* lh_last_error(void);            /* "" when none; cleared by lh_clear_error */
void lh_clear_error(void);
void lh_sync(void);                         /* wait for everything enqueued so far */

/* ---- arena: myGpuMalloc / myGpuFree / getCudaMallocAddr / resetCudaMallocAddr
 *      (API:453-473, CUB:18-25).  Memory returned by lh_malloc reads as zero,
 *      the property Tensor.zeros relies on (TD:1075-1076); blocks are 256-byte
 *      aligned (reference: 16). */
void*  lh_malloc(size_t bytes);
void*  lh_malloc_uninit(size_t bytes);      /* same bump pointer, contents unspecified: for outputs an op overwrites */
void   lh_free_top(size_t bytes);           /* LIFO pop of the most recent block(s) */
size_t lh_mark(void);
void   lh_rewind(size_t mark);
size_t lh_heap_used(void);
size_t lh_heap_peak(void);

/* ---- transfers: toGPU / toCPU / copyFloatArray (CUB:37-107, 128-131) --- */
/* The host buffer may be reused as soon as lh_h2d returns.  Up to 64 KiB it is copied into a pinned staging slot and the
 * transfer is only enqueued (no wait for the device; the stream orders it before later calls); larger uploads wait for
 * the device as the reference's cudaMemcpy does. */
void lh_h2d(void* dst, const void* h_src, size_t bytes);
void lh_d2h(void* h_dst, const void* src, size_t bytes);   /* waits */
void lh_d2d(void* dst, const void* src, size_t bytes);
/* Transfers that do not stall the step.  The reference's training loop uploads every batch with a blocking cudaMemcpy and
 * reads the loss back with another (GPUOPS:64-65; resnet50FromOnnx.scala:172-176): the device idles during the upload and
 * the host cannot issue the next step until the loss has arrived.  Same data movement, overlapped:
 *   lh_host_alloc / lh_host_free   pinned host memory (what the two calls below need on the host side);
 *   lh_h2d_async   the upload runs on a copy stream, after everything issued so far (so the last reader of dst is done)
 *                  and beside everything issued afterwards; dst must not be touched until lh_copy_join(), which makes the
 *                  main stream wait for the uploads issued so far (lh_sync and lh_cleanup join too).  With two device
 *                  buffers the batch of step i+1 travels while step i computes;
 *   lh_d2h_async   enqueues the read-back and returns; the value is in h_dst after the next lh_sync (or any later lh_d2h).
 * None of them can be recorded into a graph. */
void* lh_host_alloc(size_t bytes);
void  lh_host_free(void* p);
void  lh_h2d_async(void* dst, const void* h_src_pinned, size_t bytes);
void  lh_copy_join(void);
void  lh_d2h_async(void* h_dst_pinned, const void* src, size_t bytes);

/* ---- timing helpers for the benchmark (HIP events on the library stream) */
void* lh_event_create(void);
void  lh_event_record(void* ev);
float lh_event_elapsed_ms(void* start, void* stop);        /* waits for stop */
void  lh_event_destroy(void* ev);

/* ---- per-category kernel timing (no counterpart in the reference; a measurement aid for the
 *      benchmark).  Bit c of `mask` turns on HIP-event timing of category c; lh_prof_collect waits,
 *      sums elapsed milliseconds and call counts per category since the last collect. */
enum { LH_CAT_CONV_FWD = 0, LH_CAT_CONV_BWD_DATA, LH_CAT_CONV_BWD_FILTER, LH_CAT_GEMM, LH_CAT_BN_FWD, LH_CAT_BN_BWD,
       LH_CAT_ELEMENTWISE, LH_CAT_POOL, LH_CAT_REDUCE, LH_CAT_OPTIM, LH_CAT_FILL, LH_CAT_COUNT };
void lh_prof_enable(unsigned mask);

/* Side stream: work whose results nothing needs for a while runs beside the main chain of kernels instead of in it.
 * The reference issues every operator on one stream (CUB:171-560), so the filter gradient of a convolution, which only
 * the optimizer reads, delays the input gradient the next backward operator is waiting for.  Entry points called
 * between lh_side_begin() and lh_side_end() are enqueued on a second stream (same priority) that first waits for
 * everything issued before lh_side_begin(); work issued after lh_side_end() does NOT wait for them.  The caller
 * guarantees that, until the next join, later calls neither touch what the side work writes nor write what it reads
 * (for filter gradients: x and dy are dead or read-only for the rest of the backward pass, dw and db are read by the
 * optimizer only).  Joins (the main stream waits for the side work): lh_side_join(), and implicitly lh_sync, lh_h2d,
 * lh_d2h, lh_rewind, lh_clip and every optimizer entry point (lh_sgd, lh_momentum, lh_adagrad, lh_multi_*).
 * lh_malloc is refused on the side stream.  The side stream is bypassed (calls run in line) while per-category timing,
 * the command list or a graph recording is on, after lh_set_side_stream(0), or with LH_NO_SIDE_STREAM in the
 * environment.  lh_side_forks() counts the lh_side_begin() calls that did switch streams. */
void lh_side_begin(void);
void lh_side_end(void);
void lh_side_join(void);
void lh_set_side_stream(int on);
int64_t lh_side_forks(void);

/* HIP graph of a whole step, for programs whose kernels are shorter than their launches (LeNet, SqueezeNet on 32x32
 * images: several hundred launches of a few microseconds per step; the reference pays a launch per operator, CUB:171-560).
 * lh_capture_begin() switches the library's stream to capture: every entry point called until lh_capture_end() is
 * recorded instead of run (entry points that wait for the device -- lh_sync, lh_h2d, lh_d2h -- are errors there, and
 * launch plans are not measured, so run the step a few times first).  lh_capture_end() returns a handle;
 * lh_graph_launch(handle) enqueues the recorded step again.  The step must be replayable as recorded: the same arena
 * addresses (rewind to the same mark before capturing and after), inputs refreshed in place, parameters updated in place
 * by the recorded optimizer.  No memset nodes are recorded: the library clears memory with kernels. */
void lh_capture_begin(void);
int lh_capture_end(void);
void lh_graph_launch(int graph);
void lh_graph_destroy(int graph);

/* Command list for launch-bound programs (the sentiment TreeLSTM, SentimentTreeLSTM.scala:242-318, issues about
 * 3600 operator calls on 150-element vectors per tree; the reference pays one cuBLAS / kernel launch for each,
 * CUB:171-560).  Between lh_cmdlist_begin and lh_cmdlist_end every entry point of this header whose operands are
 * small (element-wise up to 65536 elements, matrix-vector up to 131072 matrix elements: fill, copy, geam, scalar and
 * same-shape broadcast arithmetic with gradients, unary ops with gradients, sgemv, ger, dot_vv, axpy_dev, softmax and
 * nll with gradients over rows, adagrad, sgd, and the arena's zero fill) is recorded instead of launched.  Recorded
 * commands are handed to the device whenever any other entry point is called, when 2048 are pending, and at
 * lh_cmdlist_end / lh_sync / lh_d2h, so program order holds between recorded and launched work.  Within a buffer the
 * library works out from the byte ranges each command reads and writes which commands depend on which, and runs the buffer
 * level by level: commands that do not depend on each other side by side (element-wise commands dealt over 32 workgroups,
 * LH_CMDLIST_GROUPS in the environment overrides; the matrix commands cut by rows or columns over the wavefronts of all of
 * them), a barrier over the workgroups between levels.  The barrier's wait is bounded: if a workgroup never arrives the
 * kernel ends, and the next lh_sync, lh_d2h, hand-over of recorded commands or lh_cmdlist_end reports it.  Results equal those of the stand-alone kernels
 * up to summation order in the reductions; no command uses atomic adds and every sum has a fixed order, so two runs give the
 * same bits whatever the number of workgroups.  Element-wise commands that depend only on each other lane by lane, and matrix
 * commands that write the same rows, share a level (chains; LH_CMDLIST_CHAINS=0 turns them off); chains of six and more element-wise
 * commands run as one entry over operands held in LDS (LH_CMDLIST_SLOTS=0 turns that off, LH_CMDLIST_NSLOT limits the slots).
 * None of these switches changes a result.  LH_CMDLIST_TRACE=<launch> prints, for that launch and the next, how long each level
 * took and what it held; LH_CMDLIST_VERBOSE=1 prints totals at lh_cmdlist_end.  Generated code calls lh_cmdlist_begin() once after
 * lh_setup(). */
void lh_cmdlist_begin(void);
void lh_cmdlist_end(void);
/* A test aid: sets, from the host, the flag a workgroup sets when its barrier wait runs out, so that the reporting and
 * recovery path (the next lh_sync, lh_d2h, hand-over or lh_cmdlist_end reports "timed out" once and leaves the library
 * usable) can be exercised without a kernel that gives up. */
void lh_cmdlist_inject_timeout(void);
/* Commands recorded and interpreter launches since lh_setup (either pointer may be NULL). */
void lh_cmdlist_stats(int64_t* recorded, int64_t* launches);
void lh_prof_collect(double* h_ms, int64_t* h_calls, int ncat);

/* Fusion of adjacent calls (no counterpart in the reference, whose cuDNN backend runs every trait method as its own
 * library call: CDN:833-880, 1025-1109, 1380-1429).  Lantern's generated code issues ONE call per method of the Backend
 * trait: convBBP -> batchNorm -> relu(inPlace) arrive as lh_conv2d_fwd, lh_bn_train_fwd, lh_unary(LH_RELU, y, y)
 * (ONNXLib.scala:847-872), the optimizer as one lh_momentum per parameter (NNModule.scala:296-303), and every buffer,
 * gradients included, comes zero-filled from lh_malloc and is accumulated into (TD:1509-1514).  With fusion on (the
 * default; LH_NO_FUSION=1 in the environment or lh_set_fusion(0) turn it off) the library puts work off until the next
 * call shows what it is part of, so that such a program runs the kernels a hand-fused one would:
 *   - lh_conv2d_fwd, lh_bn_train_fwd, a same-shape lh_bcast_op(LH_ADD), lh_unary_grad(LH_RELU, in place) and the same-shape
 *     lh_bcast_op_grad(LH_ADD) behind it do not launch when called.  If the next call continues one of the chains
 *       conv -> batch norm -> [+ shortcut] -> relu in place,     relu_grad -> [add_grad] -> batch-norm gradient
 *     the chain runs as lh_conv2d_fwd_bn_apply / lh_bn_train_fwd_relu / lh_add_relu / lh_bn_bwd_relu / lh_bn_bwd_add_relu;
 *     any other call (lh_malloc, lh_malloc_uninit and lh_mark excepted) first launches what is waiting, unfused.
 *     Runs of lh_momentum / lh_sgd calls with equal hyper-parameters become one multi-tensor launch.
 *   - a block of more than 16 KiB from lh_malloc is cleared when something first reads it; a call that overwrites it, or
 *     would add into it with beta = 1, writes it without the clearing pass and without reading it; lh_rewind forgets it.
 *   - what a fused chain does not store because programs do not read it (the batch norm's own output under a residual
 *     join; the in-place masking of the gradient buffer by relu_grad) is produced when a call does read it.
 *   - the copies of a filter in the layouts the convolution kernels read (tap-major for the forward pass, transposed per
 *     stride class for the input gradient) are kept, in device memory of their own outside the arena (at most 1 GiB together),
 *     while nothing writes the filter: any call of this header that writes into the filter's range ends them, and so does a
 *     rewind or pop that releases the filter; behind the gathered optimizer launch they are made again on the side stream.
 * Results are those of the calls as issued (the fused kernels give the bits of the sequences they replace wherever two
 * launches of the sequence itself agree bit for bit).  Every entry point of this header takes part; a pointer handed to
 * anything else (another library, a kernel of the caller's) must be preceded by lh_sync() AND lh_flush_deferred().
 * lh_fusion_stats: h_out[0..7] = forward chains fused, backward chains fused, optimizer calls gathered, zero fills avoided,
 * zero fills done, results produced on demand, conv -> bn or bn -> + chains that ended without a relu, filter copies found
 * kept by a convolution call. */
void lh_set_fusion(int on);
int lh_get_fusion(void);
void lh_flush_deferred(void);               /* everything put off is enqueued now (nothing waits) */
void lh_fusion_stats(int64_t* h_out, int n);
/* Algorithmic bytes of the HBM-bound kernels launched since the last call, per LH_CAT_* category (a measurement aid for the
 * benchmark: with fusion on, the caller no longer knows which kernels ran).  h_bytes[c] = bytes the kernels of category c
 * must move at least (every operand read or written once per pass the kernel makes over it). */
void lh_work_collect(double* h_bytes, int ncat);

/* ---- fill / elementwise ------------------------------------------------ */
void lh_fill(float* x, float v, int64_t n);                                    /* fill, fillInPlace: CUB:133-151 */
void lh_fill_with_bias(float* y, const float* bias, int64_t outer, int64_t c, int64_t inner); /* fillWithBias: CPU:39-62 */
void lh_clip(float* x, float bound, int64_t n);                                /* clipAt: CUB:157-161 */
void lh_mask4d(float* x, const int* lengths, int n, int c, int d, int t);      /* mask4D: CUB:710-719 */
/* repeat0 / repeat0_grad (TD:1446-1451; CDN:378-399 with the repeat0 / shift0 kernels of API:625-650): in [rows, inner] ->
 * out [rows - context, context + 1, inner] with out[i0, i1, :] = in[i0 + i1, :] (the Lookahead layer's sliding window).
 * lh_repeat0_grad adds every window's gradient into ind, all rows included (the reference leaves out the last `context` rows,
 * which its only caller fills with zero padding that has no use for a gradient). */
void lh_repeat0(const float* in, float* out, int rows, int context, int64_t inner);
void lh_repeat0_grad(float* ind, const float* outd, int rows, int context, int64_t inner);
/* Cifar10DataLoader's decode (src/main/scala/lantern/TensorDataLoader.scala:109-127) on the device: n records of one label
 * byte + count pixel bytes -> x[n, count] = (float)byte / 255.0f (correctly rounded, the host loop's bits), y[n] = (int)byte.
 * records need no alignment; x and y must not overlap records. */
void lh_cifar_decode(const unsigned char* records, float* x, int* y, int n, int count);
/* relu/tanh/sigmoid/hardTanh/exp/log/sqrt/square (TD:319-335; CDN:1349-1429, CUB:733-800).
 * y may alias x (in place).  lo/hi are used by LH_HARDTANH only. */
void lh_unary(int op, const float* x, float* y, int64_t n, float lo, float hi);
/* inplace != 0: x == y is the activated buffer and dx == dy; the gradient is
 * zeroed where the activation is flat (mask y > 0 for relu, as CDN:1404-1405). */
void lh_unary_grad(int op, const float* x, const float* y, const float* dy, float* dx, int64_t n, int inplace, float lo, float hi);
void lh_scalar_op(int op, const float* x, float* y, float s, int64_t n);       /* tensor (+,-,*,/) scalar: CDN:284-375 */
/* broadcast binary ops, numpy right-aligned rules, rank <= 4, dims padded with
 * leading 1s by the caller (TD:997-1016; CDN:153-216) */
void lh_bcast_op(int op, const float* a, const int* adims, const float* b, const int* bdims, float* out, const int* odims, int rank);
void lh_bcast_op_grad(int op, const float* a, float* ad, const int* adims, int a_is_input,
                      const float* b, float* bd, const int* bdims, int b_is_input,
                      const float* outd, const int* odims, int rank);          /* add/minus/mul/div_grad: CPU:246-337 */
/* a (op)= b with b broadcast, or reduced when a is the smaller one: += -= *= /=,
 * plusBias, plusEqual and their grads (TD:229-270; CPU:265-296; CDN:476-512, 626-649) */
void lh_bcast_update(int op, float* a, const int* adims, const float* b, const int* bdims, int rank);
void lh_geam(const float* x, float alpha, const float* y, float beta, float* out, int64_t n);   /* geam, no transposes: CPU:342-347 */
void lh_trans(const float* x, float* y, int rows, int cols);                   /* trans: CUB:361-374 */
void lh_trans_grad(float* xd, const float* yd, int rows, int cols);
void lh_permute(const float* x, float* y, const int* dims, const int* perm, int rank);          /* CUB:524-560 */
void lh_permute_grad(float* xd, const float* yd, const int* dims, const int* perm, int rank);   /* CUB:562-587, accumulates */

/* ---- reductions / loss ------------------------------------------------- */
void lh_sum_all(const float* x, float* out, int64_t n);                        /* sum: CDN:1579-1581 */
void lh_mean_all(const float* x, float* out, int64_t n);                       /* mean: CDN:1583-1585 */
void lh_add_scalar_from(float* dx, const float* dy1, float scale, int64_t n);  /* sum_grad / mean_grad: CDN:1587-1605 */
void lh_sum_dim(const float* x, float* y, int outer, int dim, int inner);      /* sum(dim): CDN:1607-1621; overwrites y */
void lh_sum_dim_grad(float* dx, const float* dy, int outer, int dim, int inner);/* CDN:1623-1636 */
/* softmax / logSoftmax over the middle axis of an [outer, c, inner] view (CDN:1431-1504) */
void lh_softmax(int is_log, const float* x, float* y, int outer, int c, int inner);
void lh_softmax_grad(int is_log, const float* y, const float* dy, float* dx, int outer, int c, int inner);
void lh_nll(const float* x, const int* target, float* y, int batch, int stride);          /* nllLoss: CUB:802-807 */
void lh_nll_grad(float* dx, const int* target, const float* dy, int batch, int stride);   /* nllLoss_grad: CUB:808-813 */

/* ---- dense: dot family and gemm (CUB:173-359, 589-688) ----------------- */
/* Row-major C[m,n] = alpha * op(A) * op(B) + beta * C; lda/ldb/ldc = row strides. */
void lh_sgemm(int ta, int tb, int m, int n, int k, float alpha, const float* A, int lda,
              const float* B, int ldb, float beta, float* C, int ldc);
void lh_sgemv(int trans, int m, int n, float alpha, const float* A, int lda, const float* x, float beta, float* y);
void lh_ger(int m, int n, const float* u, const float* v, float* A);           /* A[m,n] += u[m] (x) v[n]  (add_cartesian) */
void lh_dot_vv(const float* x, const float* y, float* out, int n);
void lh_axpy_dev(float* y, const float* h_or_d_scalar_on_device, const float* x, int64_t n);   /* y += s[0]*x, s on device (vv-dot grad) */

/* ---- conv2D_batch and its gradient (TD:292-296; CDN:515-880) ----------- */
/* y[n,k,p,q] = bias[k] + sum_{c,r,s} x[n,c,p*sH-pH+r,q*sW-pW+s] * w[k,c,r,s]; bias may be NULL.
 * Launch plans are measured once per convolution shape on first use and remembered for the life of the process: the
 * filter gradient (tile shape, number of slices of its long reduction N*P*Q and how the slices are combined: atomic adds or a second
 * summing kernel; timed on scratch memory) and, on calls
 * whose result overwrites its output, the forward and input-gradient products (tile shape, stream-K workers; a few timed
 * repetitions of the launch itself).  Products below 1e7 flop (LH_TUNE_MIN_FLOP) keep the built-in rule.  Environment:
 * LH_NO_TUNE=1 keeps the built-in rules everywhere, LH_TUNE_VERBOSE=1 prints each choice to stderr, LH_FORCE_M32=1 (a test
 * switch) sends every product of at most 32 rows to the 32-row tile whatever was measured, LH_FORCE_PLAN=n (a test switch) every forward /
 * input-gradient product to launch plan n where the shape allows it, LH_FORCE_STATS_TILE=n (a test switch) every forward product that also leaves
 * batch-norm statistics to tile plan n, LH_NO_PADDED_REDUCTION=1 (a test switch) the filter gradient over maps whose pixel count is not a multiple
 * of 4 to 4-byte loads over the plain numbering of its reduction (by default samples are numbered with their pixel count rounded up to a multiple
 * of 4, which keeps the loads 16 bytes wide; the sums then associate differently, within the usual rounding), LH_NO_SPLIT_GATHER=1 (a test switch)
 * the filter gradient of unpadded filters with rows of 5 taps and more to the gather that decodes every element of x per lane.  lh_set_tuning(0) does the same as LH_NO_TUNE from inside the process (remembered plans stay
 * remembered and are used again after lh_set_tuning(1)). */
void lh_set_tuning(int on);
/* How many launch plans have been measured so far, and how many launches have used a remembered plan (either pointer may be
 * NULL).  While a graph is recorded nothing is measured, but remembered plans are what gets recorded. */
void lh_tune_counters(int64_t* measured, int64_t* remembered);
/* Deterministic mode (no counterpart in the reference, whose CPU backend accumulates in one fixed order: CPU:589-620).  By
 * default, reductions that are cut across blocks (filter gradients, long matrix products with few tiles, stream-K tiles,
 * convolution bias gradients, sums over a long middle axis) combine their pieces with fp32 atomic adds, so two runs on the
 * same inputs differ in the last bits.  With lh_set_deterministic(1) (or LH_DETERMINISTIC=1 in the environment) every such
 * reduction writes its pieces to scratch memory and a second kernel adds them in a fixed order; stream-K is off and every
 * choice that changes the order of a sum follows a built-in rule, not a timing (slice counts and tiles of the filter gradients
 * and of lh_sgemm, the tile of a forward launch that leaves batch-norm statistics).  The measured choice among the forward /
 * input-gradient plans whose tiles are finished by one block each stays: they give the same bits whatever the tile shape.
 * The side stream stays too.  Two runs of the same calls on the same inputs then give the same bits.  Outside the guarantee:
 * lh_maxpool_bwd (the scatter form: three or more overlapping windows add in any order; lh_maxpool_bwd_dense is exact)
 * and lh_ctc_loss (fp64 sums rounded to fp32 once). */
void lh_set_deterministic(int on);
int lh_get_deterministic(void);
void lh_conv2d_fwd(const float* x, const float* w, const float* bias, float* y,
                   int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW);
void lh_conv2d_bwd_data(const float* dy, const float* w, float* dx, float beta,
                        int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW);
void lh_conv2d_bwd_filter(const float* x, const float* dy, float* dw, float* db /* or NULL */, float beta,
                          int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW);

/* ---- pooling (TD:298-302; CPU:848-1038; CDN:882-982) ------------------- */
/* argmax holds the global flat index into x (batch offset included, CPU:908); first maximum wins. */
void lh_maxpool_fwd(const float* x, float* y, int* argmax, int N, int C, int H, int W, int kH, int kW, int sH, int sW, int pad);
void lh_maxpool_bwd(const float* dy, const int* argmax, float* dx, int64_t n_out);
void lh_avgpool_fwd(const float* x, float* y, int N, int C, int H, int W, int kH, int kW, int sH, int sW);
void lh_avgpool_bwd(const float* dy, float* dx, int N, int C, int H, int W, int kH, int kW, int sH, int sW);
/* averagePool2D_batch with padding (CDN:975-982: CUDNN_POOLING_AVERAGE_COUNT_EXCLUDE_PADDING; the reference's CPU backend has
 * no implementation, CPU:1003-1005, 1035-1037): windows over the zero-padded image, divided by the number of elements inside the
 * image; pad < kernel.  lh_avgpool_pad_bwd adds into dx. */
void lh_avgpool_pad_fwd(const float* x, float* y, int N, int C, int H, int W, int kH, int kW, int sH, int sW, int pH, int pW);
void lh_avgpool_pad_bwd(const float* dy, float* dx, int N, int C, int H, int W, int kH, int kW, int sH, int sW, int pH, int pW);

/* ---- batch norm (TD:304-310; CDN:984-1266).  Spatial: x is [N,C,HW];
 *      per-activation (batchNorm1D) is the same call with HW = 1.
 *      save_mean / save_invstd hold mean and 1/sqrt(var+eps); running stats are
 *      updated as (1-factor)*running + factor*batch (unbiased variance). */
void lh_bn_infer(const float* x, const float* gamma, const float* beta, const float* run_mean, const float* run_var,
                 float* y, int N, int C, int HW, float eps);
void lh_bn_train_fwd(const float* x, const float* gamma, const float* beta, float* run_mean, float* run_var, float* y,
                     float* save_mean, float* save_invstd, int N, int C, int HW, float eps, float factor);
void lh_bn_bwd(const float* x, const float* dy, const float* gamma, const float* save_mean, const float* save_invstd,
               float* dx, float beta_dx, float* dgamma, float* dbeta, int N, int C, int HW);

/* ---- recurrent layer and CTC (DeepSpeech2 path) --------------------------------------------------
 * RNNBase over cudnnRNNForwardTraining / BackwardData / BackwardWeights (NNModule.scala:332-417,
 * CDN:1638-1893): one layer, mode 0 = relu, 1 = tanh, optionally bidirectional, zero initial state.
 *   x [T,B,I];  y [T,B,D*H] (D = 2 when bidirectional: forward half, then reverse half) holds the hidden
 *   states and is all the backward pass needs besides x;  w = packed parameters, per direction
 *   W_ih[H,I], W_hh[H,H], b_ih[H], b_hh[H] (NNModule.scala:378-390), forward direction first.
 * lh_rnn_bwd: dx = beta_dx*dx + ... (dx may be NULL), dw += ...; takes T*B*D*H + D*H*H + ... floats of
 * scratch from the top of the arena and releases them before returning.
 * The recurrence runs one kernel per time step; for 16-byte aligned operands and 64 <= H <= 2048 that kernel uses the matrix
 * instructions (LH_RNN_MFMA=0 in the environment keeps the vector form everywhere). */
void lh_rnn_fwd(int mode, const float* x, const float* w, float* y, int T, int B, int I, int H, int bidir);
void lh_rnn_bwd(int mode, const float* x, const float* y, const float* dy, const float* w, float* dx, float beta_dx, float* dw,
                int T, int B, int I, int H, int bidir);
/* The LSTM and GRU modes of RNNBase (NNModule.scala:324-330 over the same cuDNN calls): mode 2 = LSTM (gates i, f, g, o;
 * c' = f*c + i*g, h' = o*tanh(c')), 3 = GRU (gates r, z, n; n = tanh(W_in x + b_in + r*(W_hn h + b_hn)), h' = (1-z)*n + z*h),
 * cuDNN's gate order and formulas.  One layer, zero initial state; x, y, w, dx, dw as for lh_rnn_fwd / lh_rnn_bwd with
 * W_ih[G,I], W_hh[G,H], b_ih[G], b_hh[G] per direction, G = 4H or 3H.  `reserve` (cuDNN's reserve space) is caller memory of
 * lh_rnn_gated_reserve_floats(...) floats that the forward call fills and the backward call consumes (it is overwritten:
 * one backward call per forward call).  Both calls take a few [B, G] blocks (the GRU backward: T*B*G floats) from the top
 * of the arena and release them before returning. */
int64_t lh_rnn_gated_reserve_floats(int mode, int T, int B, int H, int bidir);
void lh_rnn_gated_fwd(int mode, const float* x, const float* w, float* y, float* reserve, int T, int B, int I, int H, int bidir);
void lh_rnn_gated_bwd(int mode, const float* x, const float* y, const float* dy, const float* w, float* reserve, float* dx, float beta_dx,
                      float* dw, int T, int B, int I, int H, int bidir);
/* The same four calls with the initial states of RNNBase.apply(input, hx, cx) (NNModule.scala:392-409; hxData / cxData at
 * CDN:1832-1833): hx [D,B,H] and, for the LSTM, cx [D,B,H] of this layer (NULL = zeros, which is what the calls above pass).
 * They are values only: the reference passes NULL for dhx / dcx (CDN:1843-1844), so no gradient is produced for them. */
void lh_rnn_fwd_init(int mode, const float* x, const float* hx, const float* w, float* y, int T, int B, int I, int H, int bidir);
void lh_rnn_bwd_init(int mode, const float* x, const float* hx, const float* y, const float* dy, const float* w, float* dx, float beta_dx, float* dw,
                     int T, int B, int I, int H, int bidir);
void lh_rnn_gated_fwd_init(int mode, const float* x, const float* hx, const float* cx, const float* w, float* y, float* reserve,
                           int T, int B, int I, int H, int bidir);
void lh_rnn_gated_bwd_init(int mode, const float* x, const float* hx, const float* cx, const float* y, const float* dy, const float* w,
                           float* reserve, float* dx, float beta_dx, float* dw, int T, int B, int I, int H, int bidir);
/* ctcLoss (TD:349; CDN:1895-1938, cudnnCTCLoss): probs [T,B,A] are softmax outputs, class 0 is the blank;
 * h_labels (concatenated), h_label_len [B], h_input_len [B] are HOST arrays as in the cuDNN call;
 * costs[b] = -log p(labels_b | probs).  When dprobs is not NULL the gradient with respect to the
 * pre-softmax activations (probs - posterior, what cuDNN reports) is ADDED to it, unscaled. */
void lh_ctc_loss(const float* probs, float* dprobs, const int* h_labels, const int* h_label_len, const int* h_input_len,
                 float* costs, int T, int B, int A);

/* ---- fusions of adjacent trait calls (no single counterpart in the reference; each gives the
 *      result of the sequence it replaces, in one pass over memory) ------------------------ */
/* batchNormTraining followed by relu(inPlace = true): y = max(bn(x), 0) */
void lh_bn_train_fwd_relu(const float* x, const float* gamma, const float* beta, float* run_mean, float* run_var, float* y,
                          float* save_mean, float* save_invstd, int N, int C, int HW, float eps, float factor);
/* relu_grad(inPlace) followed by batchNorm_grad: dy counts only where y > 0 (dy itself is left untouched).
 * With `bias` (the layer's beta, unchanged since the forward call) the mask is recomputed from x as
 * gamma*(x - mean)*invstd + bias > 0, bit-identical to the y that lh_bn_train_fwd_relu stored, and y
 * is not read (it may be NULL); with bias == NULL the mask is read from y. */
void lh_bn_bwd_relu(const float* x, const float* y, const float* dy, const float* gamma, const float* bias,
                    const float* save_mean, const float* save_invstd,
                    float* dx, float beta_dx, float* dgamma, float* dbeta, int N, int C, int HW);
/* maxPool2D_batch_grad as a gather: every input pixel sums the dy of the windows whose argmax it is
 * (no atomics, dx written once); dx = beta*dx + sum.  Same result as lh_maxpool_bwd. */
void lh_maxpool_bwd_dense(const float* dy, const int* argmax, float* dx, float beta,
                          int N, int C, int H, int W, int kH, int kW, int sH, int sW, int pad);
/* conv2D_batch followed by batchNormTraining of its output: the convolution's epilogue leaves per-channel
 * partial sums, so the statistics cost no pass over y.  lh_conv2d_fwd_bnstats = lh_conv2d_fwd + the
 * mean / 1/sqrt(var+eps) / running-statistics part of lh_bn_train_fwd;  lh_bn_apply is the remaining
 * part (y = gamma*(x-mean)*invstd + beta, then relu when `relu` != 0).  lh_bn_stats computes the same
 * statistics from a tensor (what lh_conv2d_fwd_bnstats falls back to for shapes without the epilogue). */
void lh_conv2d_fwd_bnstats(const float* x, const float* w, const float* bias, float* y,
                           int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW,
                           float* save_mean, float* save_invstd, float* run_mean, float* run_var, float eps, float factor);
void lh_bn_stats(const float* x, float* save_mean, float* save_invstd, float* run_mean, float* run_var,
                 int N, int C, int HW, float eps, float factor);
void lh_bn_apply(const float* x, const float* gamma, const float* beta, const float* save_mean, const float* save_invstd, float* y,
                 int N, int C, int HW, int relu);
/* Both in one call: y = conv(x, w) and out = bn(y) with relu when `relu` != 0, or, with a shortcut, the residual join
 * out = relu(bn(y) + shortcut).  Same results as lh_conv2d_fwd_bnstats followed by lh_bn_apply / lh_bn_apply_add_relu (bit for
 * bit wherever two launches of the convolution itself agree bit for bit); where the convolution's epilogue leaves the partial sums, the normalisation pass adds them up itself (every block for
 * its channel), so no statistics kernel runs between the two. */
void lh_conv2d_fwd_bn_apply(const float* x, const float* w, const float* bias, float* y,
                            int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW,
                            const float* gamma, const float* beta, float* save_mean, float* save_invstd, float* run_mean, float* run_var,
                            float eps, float factor, const float* shortcut, float* out, int relu);

/* The residual join behind a batch norm (ResNet's bn3 -> Add -> Relu; the reference runs cudnnBatchNormalizationForwardTraining,
 * an element-wise add kernel (CUB:397-420) and cudnnActivationForward, CDN:1025-1068, 1380-1400, as three passes):
 *   out = relu(gamma * (x - mean) * invstd + beta + shortcut)     with the statistics in save_mean / save_invstd
 * (from lh_conv2d_fwd_bnstats or lh_bn_stats), one pass.  Its backward, given dout = d loss / d out:
 *   g = dout where out > 0 else 0;   ds = beta_ds * ds + g;   dx = beta_dx * dx + batch-norm backward of g;
 *   dgamma += sum g * xhat;  dbeta += sum g.
 * dout is unspecified after the call: some paths overwrite it with g (two passes with ds accumulating or NULL), the others
 * leave it as it was.  dx may be NULL (no input gradient). */
void lh_bn_apply_add_relu(const float* x, const float* gamma, const float* beta, const float* save_mean, const float* save_invstd,
                          const float* shortcut, float* out, int N, int C, int HW);
void lh_bn_bwd_add_relu(const float* x, const float* out, float* dout, const float* gamma, const float* save_mean, const float* save_invstd,
                        float* dx, float beta_dx, float* ds, float beta_ds, float* dgamma, float* dbeta, int N, int C, int HW);
/* `+` of two same-shape tensors followed by relu(inPlace = true), and the gradient of that pair:
 * g = dy where y > 0 else 0;  ad = abeta*ad + g;  bd = bbeta*bd + g  (ad or bd may be NULL) */
void lh_add_relu(const float* a, const float* b, float* out, int64_t n);
void lh_add_relu_grad(const float* y, const float* dy, float* ad, float abeta, float* bd, float bbeta, int64_t n);

/* ---- dropout (TD:312-313; CPU:1066-1088).  The mask is drawn from a
 *      counter-based generator keyed by (seed, offset + element index), so a
 *      host restatement reproduces it exactly. */
void lh_dropout_fwd(const float* x, float* y, float* mask, int64_t n, float p, uint64_t seed, uint64_t offset);
void lh_dropout_bwd(const float* dy, const float* mask, float* dx, int64_t n);

/* ---- concat along one axis of n tensors (TD:369-370; CUB:825-879) ------ */
void lh_concat(int n, const float* const* h_in_ptrs, const int* sizes, float* out, int outer, int inner);
void lh_concat_grad(int n, float* const* h_ind_ptrs, const int* sizes, const float* outd, int outer, int inner);
/* The same with a host array of n betas: input t's gradient is overwritten (beta 0: a buffer no other consumer has written,
 * which then needs no zero fill) or accumulated (beta 1, what the reference does for all of them); h_beta NULL = all 1. */
void lh_concat_grad_beta(int n, float* const* h_ind_ptrs, const float* h_beta, const int* sizes, const float* outd, int outer, int inner);

/* ---- optimizers (TD:377-378; NN:255-303; API:652-678) ------------------ */
void lh_sgd(float* x, float* d, float lr, int64_t n);          /* x -= lr*d; d = 0  (SGD.step = geam + clear_grad, NN:279-285) */
void lh_momentum(float* x, float* d, float* v, float lr, float mu, float clip, int nesterov, int64_t n);
void lh_adagrad(float* x, float* d, float* m, float lr, float clip, int64_t n);
/* One launch over `count` tensors (pointer tables on the host): the 161-tensor
 * ResNet-50 update in one kernel instead of one launch per tensor. */
void lh_multi_momentum(int count, float* const* h_x, float* const* h_d, float* const* h_v, const int64_t* h_n,
                       float lr, float mu, float clip, int nesterov);
void lh_multi_sgd(int count, float* const* h_x, float* const* h_d, const int64_t* h_n, float lr);
/* lh_multi_momentum for callers that cannot allocate or wait: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  No counterpart in the reference.  Same arguments and the same results, bit for bit.  The pointer
 * table goes into a fixed 160 KiB device array (at most 4096 tensors per call; more is an error) and is written by kernels
 * that carry the entries as launch arguments, so the call allocates nothing, copies nothing from the host and never waits for
 * the device; it may be recorded into a graph.  Every call on a GPU shares that GPU's array: calls that overlap on one GPU
 * (two host threads, two streams) race. */
void lh_multi_momentum_static(int count, float* const* h_x, float* const* h_d, float* const* h_v, const int64_t* h_n,
                              float lr, float mu, float clip, int nesterov);

#ifdef __cplusplus
}
#endif
#endif
