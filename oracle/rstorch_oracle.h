/*
 * CPU restatement of the rstorch f64 training step (Linear / ReLU / Identity /
 * softmax / CrossEntropyLoss / SGD / Sequential).
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker the HIP kernels are
 * compared against and the CPU baseline that benchmarks time; nothing that
 * ships may call it.  Every function cites the reference lines it follows
 * (paths relative to the reference crate root).
 *
 * All matrices are dense row-major f64 with no strides, exactly like the
 * reference's `Array2<f64>` in standard layout.
 *
 * Parity status (what pins each function, beyond "looks like the source"):
 *   rsto_linear_forward / rsto_linear_backward  pinned  (reference KATs in
 *       linear.rs tests; exact rational brute force on tiny shapes; numpy matmul)
 *   rsto_relu_forward / rsto_relu_backward      pinned  (reference KATs; bitwise)
 *   rsto_softmax                                pinned  (reference KAT sums;
 *       shift invariance; power-of-two uniform rows; mpmath on tiny rows)
 *   rsto_cross_entropy_forward / _backward      pinned by closed forms only
 *       (the reference has no test for it): log-sum-exp identity, ln C for
 *       uniform logits, mpmath on tiny inputs, finite differences.
 *   rsto_sgd_step                               pinned  (bit-exact against
 *       numpy's two-rounding `w - lr*g`; reference zero-gradient KAT)
 *   Last-bit summation order of the reference's third-party GEMM
 *   (matrixmultiply, version unpinned by the reference) and of ndarray's
 *   `sum`/`sum_axis`, and the libm `exp`/`ln` roundings: parity unpinned;
 *   they are absorbed by the 1e-10 tolerance.
 */
#ifndef RSTORCH_ORACLE_H
#define RSTORCH_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- layer kinds for the Sequential restatement ---- */
enum { RSTO_IDENTITY = 0, RSTO_LINEAR = 1, RSTO_RELU = 2 };

/* Number of threads the GEMMs may use (1 = faithful to the reference, which is
 * single-threaded; >1 is only for the "all cores" baseline figure). */
void rsto_set_threads(int n);
int rsto_get_threads(void);

/* src/module/linear.rs:43-57 : out[B,N] = x[B,K] . w[N,K]^T, then out += bias[1,N] */
void rsto_linear_forward(const double* x, const double* w, const double* bias, double* out,
                         size_t batch, size_t in_features, size_t out_features);

/* src/module/linear.rs:60-69 : n = batch; gw[N,K] = (g^T . x)/n ; gb[1,N] = colsum(g)/n ;
 * gx[B,K] = g . w (not scaled).  gb and gx may be NULL. */
void rsto_linear_backward(const double* g, const double* x, const double* w, double* gw,
                          double* gb, double* gx, size_t batch, size_t in_features,
                          size_t out_features);

/* src/module/activation/relu.rs:19-22 : out = max(x, 0) with f64::max semantics (NaN -> 0) */
void rsto_relu_forward(const double* x, double* out, size_t n);
/* src/module/activation/relu.rs:25-27 : out = g * (x > 0 ? 1.0 : 0.0)  (a multiply) */
void rsto_relu_backward(const double* g, const double* x, double* out, size_t n);

/* src/module/activation/softmax.rs:36-53 : softmax along `axis` (0 or 1) of x[rows,cols].
 * Returns 0, or -1 if a NaN is met while taking the maximum (the reference panics there). */
int rsto_softmax(const double* x, double* out, size_t rows, size_t cols, int axis);

/* src/module/activation/softmax.rs:62-73 : the Softmax MODULE's backward (a "next" row, not on
 * the training path): jacobian = -(out^T . out) with diagonal d -> d*(1-d), result = grad . jacobian.
 * Pinned by the reference KAT (softmax.rs:105-113, tolerance 0.01) and an independent einsum. */
void rsto_softmax_module_backward(const double* grad, const double* out, double* grad_in,
                                  double* jac, size_t rows, size_t cols);

/* src/loss/cross_entropy.rs:34-42 : prob = softmax(pred, axis 1);
 * loss = -(sum(truth * ln(prob))) / rows.  prob[rows,cols] is written (the reference caches it).
 * Returns 0, or -1 on NaN logits (reference panic). */
int rsto_cross_entropy_forward(const double* pred, const double* truth, double* prob,
                               size_t rows, size_t cols, double* loss);
/* src/loss/cross_entropy.rs:45-47 : grad = -(truth - prob) */
void rsto_cross_entropy_backward(const double* prob, const double* truth, double* grad, size_t n);

/* src/optim/sgd.rs:19-24 : parm = parm - (lr * grad), two roundings, no fused multiply-add */
void rsto_sgd_step(double* parm, const double* grad, size_t n, double lr);

/* src/utils.rs:44-65 : fraction of rows whose first-maximum column matches in pred and truth */
double rsto_accuracy(const double* pred, const double* truth, size_t rows, size_t cols);

/* Exact-ish arbiter for tiny shapes: C[M,N] = sum_k A(i,k) B(k,j) accumulated in long double.
 * a_kc / b_kc select the storage of each operand (1: contraction index contiguous). */
void rsto_gemm_long_double(const double* a, const double* b, double* c, size_t m, size_t n,
                           size_t k, int a_kc, int b_kc);

/* ---- Sequential restatement (src/module/sequential.rs:78-109) ---- */
typedef struct rsto_model rsto_model;

/* kinds[i] in {RSTO_IDENTITY, RSTO_LINEAR, RSTO_RELU}; in/out features are read for LINEAR only.
 * Weights start at zero; fill them through rsto_model_parameter. */
rsto_model* rsto_model_create(const int* kinds, const size_t* in_features,
                              const size_t* out_features, size_t n_layers);
void rsto_model_destroy(rsto_model* m);
/* Parameters in the reference's order: per Linear in layer order, weight then bias
 * (src/module/linear.rs:71-78, src/module/sequential.rs:102-109). */
size_t rsto_model_parameter_count(const rsto_model* m);
int rsto_model_parameter(rsto_model* m, size_t index, double** parm, double** grad, size_t* rows,
                         size_t* cols);
/* forward: returns pointer to the logits [batch, out] owned by the model */
const double* rsto_model_forward(rsto_model* m, const double* x, size_t batch);
/* backward from grad [batch, out_last]; returns the gradient w.r.t. the input (owned) */
const double* rsto_model_backward(rsto_model* m, const double* grad);
/* SGD over every parameter, reference order */
void rsto_model_sgd_step(rsto_model* m, double lr);
/* forward, CE loss, backward, SGD: the body of the README training loop without accuracy
 * (README.md:64-74).  Returns the loss, NaN-free inputs assumed. */
double rsto_model_train_step(rsto_model* m, const double* x, const double* truth, size_t batch,
                             double lr);
/* probabilities / loss gradient of the last train_step (for inspection) */
const double* rsto_model_last_loss_grad(const rsto_model* m);

/* ---- counter-based synthetic data, shared definition with the device fill kernels ---- */
uint64_t rsto_rng_u64(uint64_t seed, uint64_t stream, uint64_t index);
void rsto_fill_uniform(double* dst, size_t n, uint64_t seed, uint64_t stream, double lo, double hi);
void rsto_fill_normal(double* dst, size_t n, uint64_t seed, uint64_t stream, double mean,
                      double std);
void rsto_fill_one_hot(double* dst, size_t rows, size_t cols, uint64_t seed, uint64_t stream);

#ifdef __cplusplus
}
#endif
#endif
