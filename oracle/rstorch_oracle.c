/*
 * CPU restatement of the rstorch f64 training step.  TEST INFRASTRUCTURE ONLY:
 * the checker for the HIP kernels and the timed CPU baseline, never a shipped path.
 * See rstorch_oracle.h for what pins each function.
 *
 * Reference files followed (relative to the reference crate root):
 *   src/module/linear.rs:43-78            Linear forward / backward / parameter order
 *   src/module/activation/relu.rs:19-27   ReLU
 *   src/module/activation/identity.rs:17-24
 *   src/module/activation/softmax.rs:36-53
 *   src/loss/cross_entropy.rs:34-47
 *   src/optim/sgd.rs:19-24
 *   src/module/sequential.rs:78-109
 *   src/utils.rs:44-65
 *
 * The reference's matrix products go through ndarray 0.15.6 `dot`, which calls the
 * `matrixmultiply` crate's dgemm (any 0.3.x; the reference does not pin it).  That crate
 * is a packed, register-blocked BLIS-style kernel; this file restates that published
 * algorithm (pack panels of A and B, MR x NR micro-kernel, k innermost) without
 * claiming its last-bit summation order.
 */
#define _GNU_SOURCE
#include "rstorch_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------------------------
 * GEMM core:  C[M,N] = sum_k A(i,k) * B(k,j)
 *   a_kc: A(i,k) = a[i*lda + k]   else  A(i,k) = a[k*lda + i]
 *   b_kc: B(k,j) = b[j*ldb + k]   else  B(k,j) = b[k*ldb + j]
 * ---------------------------------------------------------------------------------------- */
#define MR 6
#define NR 8
#define KC 256
#define MC 96
#define NC 2048

static int g_threads = 1;

void rsto_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int rsto_get_threads(void) { return g_threads; }

static void* xmalloc(size_t bytes) {
  void* p = NULL;
  if (bytes == 0) bytes = 64;
  if (posix_memalign(&p, 64, bytes) != 0) abort();
  return p;
}

/* micro-kernel: c[MR][NR] (+)= sum_{p<kc} ap[p*MR + i] * bp[p*NR + j], k innermost and
 * sequential, accumulators held in registers as 4-wide vectors. */
typedef double v4d __attribute__((vector_size(32), aligned(8)));

__attribute__((target_clones("fma", "default"), optimize("fp-contract=fast")))
static void micro_kernel(size_t kc, const double* restrict ap, const double* restrict bp,
                         double* restrict c, size_t ldc, size_t mr, size_t nr, int first) {
  const v4d zero = {0.0, 0.0, 0.0, 0.0};
  v4d c00 = zero, c01 = zero, c10 = zero, c11 = zero, c20 = zero, c21 = zero;
  v4d c30 = zero, c31 = zero, c40 = zero, c41 = zero, c50 = zero, c51 = zero;
  for (size_t p = 0; p < kc; ++p) {
    const double* a = ap + p * MR;
    const v4d b0 = *(const v4d*)(bp + p * NR), b1 = *(const v4d*)(bp + p * NR + 4);
    v4d ai;
#define RSTO_ROW(i, lo, hi)              \
  ai = (v4d){a[i], a[i], a[i], a[i]};    \
  lo += ai * b0;                         \
  hi += ai * b1;
    RSTO_ROW(0, c00, c01)
    RSTO_ROW(1, c10, c11)
    RSTO_ROW(2, c20, c21)
    RSTO_ROW(3, c30, c31)
    RSTO_ROW(4, c40, c41)
    RSTO_ROW(5, c50, c51)
#undef RSTO_ROW
  }
  double tmp[MR][NR];
  *(v4d*)&tmp[0][0] = c00; *(v4d*)&tmp[0][4] = c01;
  *(v4d*)&tmp[1][0] = c10; *(v4d*)&tmp[1][4] = c11;
  *(v4d*)&tmp[2][0] = c20; *(v4d*)&tmp[2][4] = c21;
  *(v4d*)&tmp[3][0] = c30; *(v4d*)&tmp[3][4] = c31;
  *(v4d*)&tmp[4][0] = c40; *(v4d*)&tmp[4][4] = c41;
  *(v4d*)&tmp[5][0] = c50; *(v4d*)&tmp[5][4] = c51;
  for (size_t i = 0; i < mr; ++i)
    for (size_t j = 0; j < nr; ++j) {
      if (first)
        c[i * ldc + j] = tmp[i][j];
      else
        c[i * ldc + j] += tmp[i][j];
    }
}

__attribute__((target_clones("fma", "default")))
static void pack_a(const double* a, size_t lda, int a_kc, size_t i0, size_t mc, size_t p0,
                   size_t kc, double* dst) {
  /* panels of MR rows: dst[panel][p][MR] */
  for (size_t ip = 0; ip < mc; ip += MR) {
    size_t mr = mc - ip < MR ? mc - ip : MR;
    for (size_t p = 0; p < kc; ++p) {
      for (size_t i = 0; i < MR; ++i) {
        double v = 0.0;
        if (i < mr) {
          size_t gi = i0 + ip + i, gp = p0 + p;
          v = a_kc ? a[gi * lda + gp] : a[gp * lda + gi];
        }
        dst[p * MR + i] = v;
      }
    }
    dst += kc * MR;
  }
}

/* pack one NR-column panel of B */
__attribute__((target_clones("fma", "default")))
static void pack_b_panel(const double* b, size_t ldb, int b_kc, size_t jcol, size_t nr, size_t p0,
                         size_t kc, double* dst) {
  if (!b_kc) {
    for (size_t p = 0; p < kc; ++p) {
      const double* src = b + (p0 + p) * ldb + jcol;
      for (size_t j = 0; j < NR; ++j) dst[p * NR + j] = j < nr ? src[j] : 0.0;
    }
  } else {
    for (size_t j = 0; j < NR; ++j) {
      if (j < nr) {
        const double* src = b + (jcol + j) * ldb + p0;
        for (size_t p = 0; p < kc; ++p) dst[p * NR + j] = src[p];
      } else {
        for (size_t p = 0; p < kc; ++p) dst[p * NR + j] = 0.0;
      }
    }
  }
}

#define JCHUNK 16 /* NR-panels per task: 128 columns */

static void gemm(const double* a, size_t lda, int a_kc, const double* b, size_t ldb, int b_kc,
                 double* c, size_t ldc, size_t m, size_t n, size_t k) {
  if (m == 0 || n == 0) return;
  if (k == 0) {
    for (size_t i = 0; i < m; ++i) memset(c + i * ldc, 0, n * sizeof(double));
    return;
  }
  double* bpack = (double*)xmalloc(sizeof(double) * KC * (NC + NR));
  for (size_t j0 = 0; j0 < n; j0 += NC) {
    size_t nc = n - j0 < NC ? n - j0 : NC;
    long n_panels = (long)((nc + NR - 1) / NR);
    for (size_t p0 = 0; p0 < k; p0 += KC) {
      size_t kc = k - p0 < KC ? k - p0 : KC;
      int first = (p0 == 0);
      long n_iblocks = (long)((m + MC - 1) / MC);
      long n_jchunks = (n_panels + JCHUNK - 1) / JCHUNK;
      /* The k order inside every output element is the same for any thread count: threads only
       * split the (row block, column chunk) grid. */
#ifdef _OPENMP
#pragma omp parallel num_threads(g_threads) if (g_threads > 1)
#endif
      {
        double* apack = (double*)xmalloc(sizeof(double) * KC * (MC + MR));
#ifdef _OPENMP
#pragma omp for schedule(static)
#endif
        for (long jp = 0; jp < n_panels; ++jp) {
          size_t jcol = (size_t)jp * NR;
          size_t nr = nc - jcol < NR ? nc - jcol : NR;
          pack_b_panel(b, ldb, b_kc, j0 + jcol, nr, p0, kc, bpack + (size_t)jp * kc * NR);
        }
        long packed_ib = -1;
#ifdef _OPENMP
#pragma omp for schedule(dynamic, 1)
#endif
        for (long task = 0; task < n_iblocks * n_jchunks; ++task) {
          long ib = task / n_jchunks, jc = task % n_jchunks;
          size_t i0 = (size_t)ib * MC;
          size_t mc = m - i0 < MC ? m - i0 : MC;
          if (packed_ib != ib) {
            pack_a(a, lda, a_kc, i0, mc, p0, kc, apack);
            packed_ib = ib;
          }
          long jp_end = (jc + 1) * JCHUNK < n_panels ? (jc + 1) * JCHUNK : n_panels;
          for (long jp = jc * JCHUNK; jp < jp_end; ++jp) {
            size_t jcol = (size_t)jp * NR;
            size_t nr = nc - jcol < NR ? nc - jcol : NR;
            const double* bp = bpack + (size_t)jp * kc * NR;
            for (size_t ip = 0; ip < mc; ip += MR) {
              size_t mr = mc - ip < MR ? mc - ip : MR;
              const double* ap = apack + (ip / MR) * kc * MR;
              micro_kernel(kc, ap, bp, c + (i0 + ip) * ldc + j0 + jcol, ldc, mr, nr, first);
            }
          }
        }
        free(apack);
      }
    }
  }
  free(bpack);
}

void rsto_gemm_long_double(const double* a, const double* b, double* c, size_t m, size_t n,
                           size_t k, int a_kc, int b_kc) {
  for (size_t i = 0; i < m; ++i)
    for (size_t j = 0; j < n; ++j) {
      long double s = 0.0L;
      for (size_t p = 0; p < k; ++p) {
        long double av = a_kc ? a[i * k + p] : a[p * m + i];
        long double bv = b_kc ? b[j * k + p] : b[p * n + j];
        s += av * bv;
      }
      c[i * n + j] = (double)s;
    }
}

/* ------------------------------------------------------------------------------------------
 * Linear
 * ---------------------------------------------------------------------------------------- */

/* src/module/linear.rs:43-57 */
void rsto_linear_forward(const double* x, const double* w, const double* bias, double* out,
                         size_t batch, size_t in_features, size_t out_features) {
  /* linear.rs:44  let mut x = input.dot(&self.weight.t()); */
  gemm(x, in_features, 1, w, in_features, 1, out, out_features, batch, out_features, in_features);
  /* linear.rs:51-53  x += bias  (broadcast of the (1,N) row over the batch, after the product) */
  if (bias) {
    for (size_t r = 0; r < batch; ++r) {
      double* row = out + r * out_features;
      for (size_t j = 0; j < out_features; ++j) row[j] += bias[j];
    }
  }
}

/* src/module/linear.rs:60-69 */
void rsto_linear_backward(const double* g, const double* x, const double* w, double* gw,
                          double* gb, double* gx, size_t batch, size_t in_features,
                          size_t out_features) {
  /* linear.rs:62  let n = prev_input.nrows() as f64; */
  const double n = (double)batch;
  /* linear.rs:63  grad_weight = gradient.t().dot(&prev_input) / n   -> (out, in) */
  gemm(g, out_features, 0, x, in_features, 0, gw, in_features, out_features, in_features, batch);
  for (size_t i = 0; i < out_features * in_features; ++i) gw[i] = gw[i] / n;
  /* linear.rs:65-67  grad_bias = (gradient.sum_axis(Axis(0)) / n).insert_axis(Axis(0)) -> (1,out)
   * sum_axis over the outer axis adds the row views one after another. */
  if (gb) {
    for (size_t j = 0; j < out_features; ++j) gb[j] = 0.0;
    for (size_t r = 0; r < batch; ++r) {
      const double* row = g + r * out_features;
      for (size_t j = 0; j < out_features; ++j) gb[j] += row[j];
    }
    for (size_t j = 0; j < out_features; ++j) gb[j] = gb[j] / n;
  }
  /* linear.rs:68  gradient.dot(&self.weight)   -> (batch, in), not divided by n */
  if (gx) gemm(g, out_features, 1, w, in_features, 0, gx, in_features, batch, in_features,
               out_features);
}

/* ------------------------------------------------------------------------------------------
 * ReLU
 * ---------------------------------------------------------------------------------------- */

/* src/module/activation/relu.rs:21  input.mapv(|x| x.max(0.0)) ; f64::max returns the other
 * operand when one is NaN, so NaN maps to 0.0 (C fmax has the same rule). */
void rsto_relu_forward(const double* x, double* out, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = fmax(x[i], 0.0);
}

/* src/module/activation/relu.rs:26  gradient * prev_input.mapv(|x| f64::from(x > 0.0)) */
void rsto_relu_backward(const double* g, const double* x, double* out, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = g[i] * (x[i] > 0.0 ? 1.0 : 0.0);
}

/* ------------------------------------------------------------------------------------------
 * softmax and cross entropy
 * ---------------------------------------------------------------------------------------- */

/* src/module/activation/softmax.rs:36-53.
 * max folds from f64::MIN (the most negative finite double, i.e. -DBL_MAX) with
 * partial_cmp().unwrap(), which panics when either side is NaN -> return -1. */
int rsto_softmax(const double* x, double* out, size_t rows, size_t cols, int axis) {
  if (axis == 1) {
    for (size_t r = 0; r < rows; ++r) {
      const double* xi = x + r * cols;
      double* oi = out + r * cols;
      double mx = -DBL_MAX;
      for (size_t c = 0; c < cols; ++c) {
        if (isnan(xi[c])) return -1;
        if (mx < xi[c]) mx = xi[c]; /* Less -> b ; Equal/Greater -> a */
      }
      double s = 0.0;
      for (size_t c = 0; c < cols; ++c) {
        oi[c] = exp(xi[c] - mx);
        s += oi[c];
      }
      for (size_t c = 0; c < cols; ++c) oi[c] = oi[c] / s;
    }
    return 0;
  }
  /* axis 0: reduce down each column */
  for (size_t c = 0; c < cols; ++c) {
    double mx = -DBL_MAX;
    for (size_t r = 0; r < rows; ++r) {
      double v = x[r * cols + c];
      if (isnan(v)) return -1;
      if (mx < v) mx = v;
    }
    double s = 0.0;
    for (size_t r = 0; r < rows; ++r) {
      double e = exp(x[r * cols + c] - mx);
      out[r * cols + c] = e;
      s += e;
    }
    for (size_t r = 0; r < rows; ++r) out[r * cols + c] = out[r * cols + c] / s;
  }
  return 0;
}

/* src/module/activation/softmax.rs:62-73 (Softmax module backward).  One C x C matrix for the
 * whole batch: jacobian = -(out^T . out); its diagonal entries d = (out^T . out)_ii become
 * d * (1 - d); the result is gradient . jacobian.  `jac` is C*C scratch. */
void rsto_softmax_module_backward(const double* grad, const double* out, double* grad_in,
                                  double* jac, size_t rows, size_t cols) {
  gemm(out, cols, 0, out, cols, 0, jac, cols, cols, cols, rows); /* out^T . out */
  for (size_t i = 0; i < cols; ++i)
    for (size_t j = 0; j < cols; ++j) {
      double v = jac[i * cols + j];
      if (i == j) {
        double el = -v;       /* jacobian = -(...) */
        el = -el;             /* softmax.rs:67  *el = -*el          */
        el = el * (1.0 - el); /* softmax.rs:68  *el = *el * (1 - *el) */
        jac[i * cols + j] = el;
      } else {
        jac[i * cols + j] = -v;
      }
    }
  gemm(grad, cols, 1, jac, cols, 0, grad_in, cols, rows, cols, cols); /* gradient . jacobian */
}

/* src/loss/cross_entropy.rs:34-42.  ln of the probability (not a log-sum-exp form): a
 * probability that underflowed to 0 gives 0 * -inf = NaN when truth is 0 there, as in the
 * reference.  EPSILON (cross_entropy.rs:6) is unused by the reference and here. */
int rsto_cross_entropy_forward(const double* pred, const double* truth, double* prob,
                               size_t rows, size_t cols, double* loss) {
  const double batch_size = (double)rows;
  if (rsto_softmax(pred, prob, rows, cols, 1) != 0) return -1;
  double s = 0.0;
  for (size_t i = 0; i < rows * cols; ++i) s += truth[i] * log(prob[i]);
  *loss = -s / batch_size;
  return 0;
}

/* src/loss/cross_entropy.rs:45-47   -(truth - pred) */
void rsto_cross_entropy_backward(const double* prob, const double* truth, double* grad, size_t n) {
  for (size_t i = 0; i < n; ++i) grad[i] = -(truth[i] - prob[i]);
}

/* ------------------------------------------------------------------------------------------
 * SGD.  src/optim/sgd.rs:23  *parm = parm.clone() - (self.lr * grad.clone())
 * The product is rounded to f64 before the subtraction: keep the compiler from fusing them.
 * ---------------------------------------------------------------------------------------- */
#pragma GCC push_options
#pragma GCC optimize("fp-contract=off")
void rsto_sgd_step(double* parm, const double* grad, size_t n, double lr) {
  for (size_t i = 0; i < n; ++i) {
    volatile double prod = lr * grad[i];
    parm[i] = parm[i] - prod;
  }
}
#pragma GCC pop_options

/* src/utils.rs:44-65.  argmax keeps the first maximum: reduce replaces only on strict `>`. */
double rsto_accuracy(const double* pred, const double* truth, size_t rows, size_t cols) {
  size_t hits = 0;
  for (size_t r = 0; r < rows; ++r) {
    size_t ap = 0, at = 0;
    for (size_t c = 1; c < cols; ++c) {
      if (pred[r * cols + c] > pred[r * cols + ap]) ap = c;
      if (truth[r * cols + c] > truth[r * cols + at]) at = c;
    }
    hits += (ap == at);
  }
  return (double)hits / (double)rows;
}

/* ------------------------------------------------------------------------------------------
 * Sequential
 * ---------------------------------------------------------------------------------------- */
typedef struct {
  int kind;
  size_t in, out;
  double *w, *b, *gw, *gb; /* Linear only */
  double* cache;           /* Linear: input ; ReLU: pre-activation input */
  double* fwd_out;
  double* bwd_out;
  size_t width_in, width_out; /* features flowing through, resolved at forward time */
} rsto_layer;

struct rsto_model {
  size_t n_layers;
  rsto_layer* layers;
  size_t batch;
  size_t cap_batch;
  size_t in_width;
  double* prob;
  double* loss_grad;
  double* x_copy;
};

rsto_model* rsto_model_create(const int* kinds, const size_t* in_features,
                              const size_t* out_features, size_t n_layers) {
  rsto_model* m = (rsto_model*)calloc(1, sizeof(rsto_model));
  m->n_layers = n_layers;
  m->layers = (rsto_layer*)calloc(n_layers ? n_layers : 1, sizeof(rsto_layer));
  for (size_t i = 0; i < n_layers; ++i) {
    rsto_layer* l = &m->layers[i];
    l->kind = kinds[i];
    if (l->kind == RSTO_LINEAR) {
      l->in = in_features[i];
      l->out = out_features[i];
      l->w = (double*)xmalloc(sizeof(double) * l->in * l->out);
      l->gw = (double*)xmalloc(sizeof(double) * l->in * l->out);
      l->b = (double*)xmalloc(sizeof(double) * l->out);
      l->gb = (double*)xmalloc(sizeof(double) * l->out);
      memset(l->w, 0, sizeof(double) * l->in * l->out);
      memset(l->gw, 0, sizeof(double) * l->in * l->out);
      memset(l->b, 0, sizeof(double) * l->out);
      memset(l->gb, 0, sizeof(double) * l->out);
    }
  }
  return m;
}

static void free_buffers(rsto_model* m) {
  for (size_t i = 0; i < m->n_layers; ++i) {
    rsto_layer* l = &m->layers[i];
    free(l->cache);
    free(l->fwd_out);
    free(l->bwd_out);
    l->cache = l->fwd_out = l->bwd_out = NULL;
  }
  free(m->prob);
  free(m->loss_grad);
  free(m->x_copy);
  m->prob = m->loss_grad = m->x_copy = NULL;
}

void rsto_model_destroy(rsto_model* m) {
  if (!m) return;
  free_buffers(m);
  for (size_t i = 0; i < m->n_layers; ++i) {
    rsto_layer* l = &m->layers[i];
    free(l->w);
    free(l->b);
    free(l->gw);
    free(l->gb);
  }
  free(m->layers);
  free(m);
}

size_t rsto_model_parameter_count(const rsto_model* m) {
  size_t n = 0;
  for (size_t i = 0; i < m->n_layers; ++i)
    if (m->layers[i].kind == RSTO_LINEAR) n += 2;
  return n;
}

int rsto_model_parameter(rsto_model* m, size_t index, double** parm, double** grad, size_t* rows,
                         size_t* cols) {
  size_t n = 0;
  for (size_t i = 0; i < m->n_layers; ++i) {
    rsto_layer* l = &m->layers[i];
    if (l->kind != RSTO_LINEAR) continue;
    if (index == n) { /* weight (out, in) */
      *parm = l->w; *grad = l->gw; *rows = l->out; *cols = l->in;
      return 0;
    }
    if (index == n + 1) { /* bias (1, out) */
      *parm = l->b; *grad = l->gb; *rows = 1; *cols = l->out;
      return 0;
    }
    n += 2;
  }
  return -1;
}

static size_t first_linear_in(const rsto_model* m) {
  for (size_t i = 0; i < m->n_layers; ++i)
    if (m->layers[i].kind == RSTO_LINEAR) return m->layers[i].in;
  return 0;
}

static void ensure_buffers(rsto_model* m, size_t batch, size_t in_width) {
  if (batch <= m->cap_batch && in_width == m->in_width) return;
  free_buffers(m);
  size_t width = in_width;
  for (size_t i = 0; i < m->n_layers; ++i) {
    rsto_layer* l = &m->layers[i];
    l->width_in = width;
    if (l->kind == RSTO_LINEAR) width = l->out;
    l->width_out = width;
    if (l->kind != RSTO_IDENTITY) {
      l->cache = (double*)xmalloc(sizeof(double) * batch * l->width_in);
      l->fwd_out = (double*)xmalloc(sizeof(double) * batch * l->width_out);
      l->bwd_out = (double*)xmalloc(sizeof(double) * batch * l->width_in);
    }
  }
  m->prob = (double*)xmalloc(sizeof(double) * batch * width);
  m->loss_grad = (double*)xmalloc(sizeof(double) * batch * width);
  m->x_copy = (double*)xmalloc(sizeof(double) * batch * in_width);
  m->cap_batch = batch;
  m->in_width = in_width;
}

/* src/module/sequential.rs:78-82  fold(input, |input, layer| layer.forward(input)) */
const double* rsto_model_forward(rsto_model* m, const double* x, size_t batch) {
  size_t in_width = first_linear_in(m);
  ensure_buffers(m, batch, in_width);
  m->batch = batch;
  memcpy(m->x_copy, x, sizeof(double) * batch * in_width);
  const double* cur = m->x_copy;
  for (size_t i = 0; i < m->n_layers; ++i) {
    rsto_layer* l = &m->layers[i];
    switch (l->kind) {
      case RSTO_IDENTITY: /* identity.rs:17-19 */
        break;
      case RSTO_LINEAR: /* linear.rs:43-57: compute, then keep the input */
        rsto_linear_forward(cur, l->w, l->b, l->fwd_out, batch, l->in, l->out);
        memcpy(l->cache, cur, sizeof(double) * batch * l->in);
        cur = l->fwd_out;
        break;
      case RSTO_RELU: /* relu.rs:19-22: keep the pre-activation, return max(x, 0) */
        memcpy(l->cache, cur, sizeof(double) * batch * l->width_in);
        rsto_relu_forward(cur, l->fwd_out, batch * l->width_in);
        cur = l->fwd_out;
        break;
    }
  }
  return cur;
}

/* src/module/sequential.rs:85-90  reversed fold over layer.backward */
const double* rsto_model_backward(rsto_model* m, const double* grad) {
  const double* cur = grad;
  size_t batch = m->batch;
  for (size_t ii = m->n_layers; ii-- > 0;) {
    rsto_layer* l = &m->layers[ii];
    switch (l->kind) {
      case RSTO_IDENTITY: /* identity.rs:22-24 */
        break;
      case RSTO_LINEAR:
        rsto_linear_backward(cur, l->cache, l->w, l->gw, l->gb, l->bwd_out, batch, l->in, l->out);
        cur = l->bwd_out;
        break;
      case RSTO_RELU:
        rsto_relu_backward(cur, l->cache, l->bwd_out, batch * l->width_in);
        cur = l->bwd_out;
        break;
    }
  }
  return cur;
}

/* src/optim/sgd.rs:19-24 over src/module/sequential.rs:102-109 */
void rsto_model_sgd_step(rsto_model* m, double lr) {
  for (size_t i = 0; i < m->n_layers; ++i) {
    rsto_layer* l = &m->layers[i];
    if (l->kind != RSTO_LINEAR) continue;
    rsto_sgd_step(l->w, l->gw, l->in * l->out, lr);
    rsto_sgd_step(l->b, l->gb, l->out, lr);
  }
}

/* README.md:64-74 without the accuracy call */
double rsto_model_train_step(rsto_model* m, const double* x, const double* truth, size_t batch,
                             double lr) {
  const double* logits = rsto_model_forward(m, x, batch);
  size_t classes = m->n_layers ? m->layers[m->n_layers - 1].width_out : m->in_width;
  double loss = NAN;
  if (rsto_cross_entropy_forward(logits, truth, m->prob, batch, classes, &loss) != 0) return NAN;
  rsto_cross_entropy_backward(m->prob, truth, m->loss_grad, batch * classes);
  rsto_model_backward(m, m->loss_grad);
  rsto_model_sgd_step(m, lr);
  return loss;
}

const double* rsto_model_last_loss_grad(const rsto_model* m) { return m->loss_grad; }

/* ------------------------------------------------------------------------------------------
 * Counter-based synthetic data: value(seed, stream, index) is a pure function, so the device
 * fill kernels and this file produce the same sequences (uniforms bit-identical; normals
 * up to the last bits of log / sqrt / cos).
 * ---------------------------------------------------------------------------------------- */
static inline uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ULL;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
  return z ^ (z >> 31);
}

uint64_t rsto_rng_u64(uint64_t seed, uint64_t stream, uint64_t index) {
  uint64_t key = mix64(mix64(seed) ^ (stream * 0xD1342543DE82EF95ULL));
  return mix64(key + index * 0x9E3779B97F4A7C15ULL);
}

static inline double u01(uint64_t r) { return (double)(r >> 11) * 0x1.0p-53; }

void rsto_fill_uniform(double* dst, size_t n, uint64_t seed, uint64_t stream, double lo, double hi) {
  for (size_t i = 0; i < n; ++i) dst[i] = lo + (hi - lo) * u01(rsto_rng_u64(seed, stream, i));
}

void rsto_fill_normal(double* dst, size_t n, uint64_t seed, uint64_t stream, double mean,
                      double std) {
  const double two_pi = 6.283185307179586476925286766559;
  for (size_t i = 0; i < n; ++i) {
    uint64_t r1 = rsto_rng_u64(seed, stream, 2 * i), r2 = rsto_rng_u64(seed, stream, 2 * i + 1);
    double u1 = ((double)(r1 >> 11) + 1.0) * 0x1.0p-53; /* (0, 1] */
    double u2 = u01(r2);
    dst[i] = mean + std * (sqrt(-2.0 * log(u1)) * cos(two_pi * u2));
  }
}

void rsto_fill_one_hot(double* dst, size_t rows, size_t cols, uint64_t seed, uint64_t stream) {
  memset(dst, 0, sizeof(double) * rows * cols);
  for (size_t r = 0; r < rows; ++r) {
    size_t label = (size_t)(rsto_rng_u64(seed, stream, r) % (uint64_t)cols);
    dst[r * cols + label] = 1.0;
  }
}
