/*
 * TEST INFRASTRUCTURE, NOT PRODUCT.
 *
 * CPU restatement of Lantern's BackendCPU (reference:
 * src/main/scala/lantern/TensorDslCPU.scala) in plain C.  It is the checker
 * the HIP kernels are compared with, and the host-core baseline that the
 * benchmark times.  Only tests, the smoke check and the benchmark's
 * cpu_baseline leg may link or load it; the shipped library never does.
 *
 * Every function names the reference lines it follows.  "ref" paths are
 * relative to the reference checkout; CPU = src/main/scala/lantern/
 * TensorDslCPU.scala, TD = .../TensorDifferentiation.scala,
 * CDN = .../TensorDslCudnn.scala, NN = .../NNModule.scala.
 *
 * Conventions (same as the reference): dense row-major fp32, NCHW; every
 * *_grad function accumulates (+=) into the gradient buffers.
 *
 * Pinning status of each function (what independent evidence fixes it) is
 * given by tests/test_reference_vectors.py (the reference's own vectors) and
 * tests/test_oracle_math.py (closed forms, brute force, library routines); functions without a reference
 * vector are marked "parity unpinned" there and below.
 *   parity unpinned: lc_ctc_loss, lc_rnn_fwd, lc_rnn_bwd, lc_rnn_gated_fwd, lc_rnn_gated_bwd, lc_avgpool_pad_fwd, lc_avgpool_pad_bwd (no asserted vector and no CPU implementation in the
 *   reference; both are checked against torch's CPU routines in tests/test_oracle_math.py).
 */
#ifndef LANTERN_CPU_ORACLE_H
#define LANTERN_CPU_ORACLE_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

enum { LC_ADD = 0, LC_SUB = 1, LC_MUL = 2, LC_DIV = 3 };
enum { LC_RELU = 0, LC_TANH = 1, LC_SIGMOID = 2, LC_EXP = 3, LC_LOG = 4, LC_SQRT = 5, LC_SQUARE = 6, LC_HARDTANH = 7 };

void lc_set_threads(int n);
int  lc_get_threads(void);

/* fill / init */
void lc_fill(float* x, float v, long n);                                           /* CPU:26-37 */
void lc_fill_with_bias(float* y, const float* bias, long outer, long c, long inner);/* CPU:39-62 */
void lc_srand(unsigned seed);                                                      /* TD:66-69 */
void lc_rand_uniform(float* x, long n);                                            /* Tensor.rand: TD Random.rand */
void lc_clip(float* x, float bound, long n);                                       /* CPU:112-119 */

/* BLAS-like (the reference calls OpenBLAS; this is an own row-major kernel) */
void lc_sgemm(int ta, int tb, int m, int n, int k, float alpha, const float* A, int lda,
              const float* B, int ldb, float beta, float* C, int ldc);
void lc_sgemv(int trans, int m, int n, float alpha, const float* A, int lda, const float* x, float beta, float* y);

/* dot family: CPU:135-225 */
void lc_dot_vv(const float* x, const float* y, float* out, int n);
void lc_dot_mv(const float* A, const float* v, float* out, int m, int n);
void lc_dot_mm(const float* A, const float* B, float* out, int m, int k, int n);
void lc_add_cartesian(float* xd, const float* y, const float* outd, int m, int n);  /* xd[m,n] += outd[m] (x) y[n] */
void lc_add_composition(float* xd, const float* Y, const float* outd, int m, int n);/* xd[n] += Y[m,n]^T outd[m] */
void lc_add_dottrans1(float* xd, const float* Y, const float* outd, int d1, int d2, int d3); /* xd[d2,d3] += Y[d1,d2]^T outd[d1,d3] */
void lc_add_dottrans2(float* xd, const float* Y, const float* outd, int d1, int d2, int d3); /* xd[d1,d2] += Y[d1,d3] outd[d2,d3]^T */
void lc_addmul_scalar(float* xd, const float* s, const float* y, long n);           /* xd += s[0]*y (vv-dot grad) */

/* gemm: CPU:379-472 */
void lc_gemm(int tx, int ty, int d1, int d2, int d3, float alpha, const float* x, const float* y, float* out);
void lc_gemm_grad(int tx, int ty, int d1, int d2, int d3, float alpha, const float* x, float* xd, int x_is_input,
                  const float* y, float* yd, int y_is_input, const float* outd);

/* broadcast ops, rank<=4 right-aligned dims (CPU:227-340, TD:997-1016) */
void lc_bcast_op(int op, const float* a, const int* adims, const float* b, const int* bdims, float* out, const int* odims, int rank);
void lc_bcast_op_grad(int op, const float* a, float* ad, const int* adims, int a_is_input,
                      const float* b, float* bd, const int* bdims, int b_is_input,
                      const float* outd, const int* odims, int rank);
void lc_bcast_update(int op, float* a, const int* adims, const float* b, const int* bdims, int rank); /* CPU:265-279 */
void lc_scalar_op(int op, const float* x, float* y, float s, long n);               /* CPU:298-339 */
void lc_geam(const float* x, float alpha, const float* y, float beta, float* out, long n); /* CPU:342-347 */
void lc_trans(const float* x, float* y, int rows, int cols);                        /* CPU:349-362 */
void lc_trans_grad(float* xd, const float* yd, int rows, int cols);                 /* CPU:364-374 */
/* repeat0 (TD:1446-1451; CPU ??? 1214-1215; API:625-650) */
void lc_repeat0(const float* in, float* out, int rows, int context, long inner);
void lc_repeat0_grad(float* ind, const float* outd, int rows, int context, long inner);
void lc_permute(const float* x, float* y, const int* dims, const int* perm, int rank);      /* math; CPU ??? 376 */
void lc_permute_grad(float* xd, const float* yd, const int* dims, const int* perm, int rank);

/* conv: CPU:484-692 */
void lc_conv2d_fwd(const float* x, const float* w, const float* bias, float* y, float* finput,
                   int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW);
void lc_conv2d_bwd(const float* finput, const float* w, const float* dy, float* dx, float* dw, float* db,
                   float* fgrad_scratch, int N, int C, int H, int W, int K, int R, int S, int sH, int sW, int pH, int pW);

/* activations: CPU:711-781 */
void lc_unary(int op, const float* x, float* y, long n, float lo, float hi);
void lc_unary_grad(int op, const float* x, const float* y, const float* dy, float* dx, long n, int inplace, float lo, float hi);

/* softmax / loss: CPU:784-846, 1090-1110 */
void lc_softmax(int is_log, const float* x, float* y, int rows, int cols);
void lc_softmax_grad(int is_log, const float* y, const float* dy, float* dx, int rows, int cols);
void lc_softmax3(int is_log, const float* x, float* y, int outer, int c, int inner);       /* CDN:1431-1504 view */
void lc_softmax3_grad(int is_log, const float* y, const float* dy, float* dx, int outer, int c, int inner);
void lc_nll(const float* x, const int* target, float* y, int batch, int stride);
void lc_nll_grad(float* dx, const int* target, const float* dy, int batch, int stride);

/* pooling: CPU:848-1038; argmax = global flat input index */
void lc_maxpool_fwd(const float* x, float* y, int* idx, int N, int C, int H, int W, int kH, int kW, int sH, int sW, int pad);
void lc_maxpool_bwd(const float* dy, const int* idx, float* dx, long n_out);
void lc_avgpool_fwd(const float* x, float* y, int N, int C, int H, int W, int kH, int kW, int sH, int sW);
/* padded, divisor = elements inside the image (CDN:975-982); parity unpinned against the reference, checked against torch */
void lc_avgpool_pad_fwd(const float* x, float* y, int N, int C, int H, int W, int kH, int kW, int sH, int sW, int pH, int pW);
void lc_avgpool_pad_bwd(const float* dy, float* dx, int N, int C, int H, int W, int kH, int kW, int sH, int sW, int pH, int pW);
void lc_avgpool_bwd(const float* dy, float* dx, int N, int C, int H, int W, int kH, int kW, int sH, int sW);

/* batch norm: forward formula CPU:1040-1056; statistics/backward semantics CDN:1025-1131 */
void lc_bn_infer(const float* x, const float* gamma, const float* beta, const float* rmean, const float* rvar,
                 float* y, int N, int C, int HW, float eps);
void lc_bn_train_fwd(const float* x, const float* gamma, const float* beta, float* rmean, float* rvar, float* y,
                     float* save_mean, float* save_invstd, int N, int C, int HW, float eps, float factor);
void lc_bn_bwd(const float* x, const float* dy, const float* gamma, const float* save_mean, const float* save_invstd,
               float* dx, float* dgamma, float* dbeta, int N, int C, int HW);

/* dropout: CPU:1066-1088 (glibc rand order) and the counter-based variant the device uses */
void lc_dropout_rand(const float* x, float* y, float* mask, long n, float p);
void lc_dropout_ctr(const float* x, float* y, float* mask, long n, float p, uint64_t seed, uint64_t offset);
float lc_ctr_uniform(uint64_t seed, uint64_t index);
void lc_dropout_bwd(const float* dy, const float* mask, float* dx, long n);

/* reductions: CPU:1115-1164 */
void lc_sum_all(const float* x, float* out, long n);
void lc_mean_all(const float* x, float* out, long n);
void lc_add_scalar_from(float* dx, const float* dy1, float scale, long n);          /* sum_grad / mean_grad */
void lc_sum_dim(const float* x, float* y, int outer, int dim, int inner);
void lc_sum_dim_grad(float* dx, const float* dy, int outer, int dim, int inner);

/* concat along dim of n tensors: CPU:1166-1212 */
void lc_concat(int n, const float* const* in, const int* sizes, float* out, int outer, int inner);
void lc_concat_grad(int n, float* const* ind, const int* sizes, const float* outd, int outer, int inner);

void lc_mask4d(float* x, const int* lengths, int n, int c, int d, int t);          /* CPU:694-708 */

/* optimizers: NN:265-303, CPU:1217-1246 */
void lc_sgd(float* x, float* d, float lr, long n);
void lc_momentum(float* x, float* d, float* v, float lr, float mu, float clip, int nesterov, long n);
void lc_adagrad(float* x, float* d, float* m, float lr, float clip, long n);

/* CTC loss (parity unpinned: reference has no asserted vector; CDN:1895-1938 semantics) */
void lc_ctc_loss(const float* probs, float* dprobs, const int* labels, const int* label_len, const int* input_len,
                 float* costs, int T, int B, int A);
void lc_rnn_fwd(int mode, const float* x, const float* w, float* y, int T, int B, int I, int H, int bidir);
/* LSTM (mode 2) / GRU (mode 3), cuDNN formulas; parity unpinned against the reference, checked against torch.nn.LSTM / GRU */
void lc_rnn_gated_fwd(int mode, const float* x, const float* w, float* y, int T, int B, int I, int H, int bidir);
void lc_rnn_gated_bwd(int mode, const float* x, const float* dy, const float* w, float* dx, float* dw, int T, int B, int I, int H, int bidir);
void lc_rnn_bwd(int mode, const float* x, const float* y, const float* dy, const float* w, float* dx, float* dw,
                int T, int B, int I, int H, int bidir);

#ifdef __cplusplus
}
#endif
#endif
