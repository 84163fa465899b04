// Operator-level C ABI: argument checking and dispatch onto the launch functions.  Each entry
// point names the reference lines it replaces in include/rstorch_hip.h.
#include <climits>
#include <cstring>

#include "common.h"

using namespace rst;

namespace rst {

// enqueues the arg-max agreement count of pred / truth and waits until it is in the pinned hit word;
// `ahead` (if any) runs between the two: launches that the caller wants on the stream before the wait
int engine_accuracy(rst_engine* e, const double* pred, const double* truth, size_t rows, size_t cols,
                    int (*ahead)(void*), void* ahead_arg) {
  bool mirrored = false;
  const unsigned ticket = engine_next_ticket(e);
  RST_TRY(launch_accuracy(e->stream, pred, truth, rows, cols, e->d_hits, e->hd_hits, &mirrored, e->hd_slots,
                          ticket));
  if (ahead) RST_TRY(ahead(ahead_arg));
  if (mirrored) {
    RST_TRY(engine_wait_ticket(e, ticket, 2));
    *e->h_hits = e->h_slots[1].count;  // (the record and the plain word hold the same count; only the record is certain to be there)
    return RST_OK;
  }
  RST_HIP(hipMemcpyAsync(e->h_hits, e->d_hits, sizeof(unsigned long long), hipMemcpyDeviceToHost,
                         e->stream));
  RST_HIP(hipStreamSynchronize(e->stream));
  return RST_OK;
}

namespace {

__global__ void reset_softmax_flag_kernel(int* flags) { flags[2] = 0; }

int check_dim(size_t v, const char* what) {
  if (v > (size_t)INT_MAX) return fail(RST_ERR_UNSUPPORTED, "%s = %zu exceeds 2^31-1", what, v);
  return RST_OK;
}

}  // namespace

namespace {
// where the launch that finishes a loss stores it for the host, and the launch's ticket
int loss_mirror(rst_engine* e, LossMirror* mirror) {
  mirror->loss = e->hd_loss;
  mirror->flags = e->hd_flags;
  // A launch that is being recorded into a graph gets no ticket: every replay would announce the
  // number of the recording.
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  RST_HIP(hipStreamIsCapturing(e->stream, &capture));
  e->loss_ticket = 0;
  e->loss_with_hits = false;
  if (capture == hipStreamCaptureStatusNone) {
    mirror->slots = e->hd_slots;
    mirror->ticket = e->loss_ticket = engine_next_ticket(e);
  }
  return RST_OK;
}
}  // namespace

int engine_head_cross_entropy(rst_engine* e, double* row_loss, const double* h, const double* w,
                              const double* bias, const double* truth, double* logits, double* grad,
                              double* dx, bool mask, size_t rows, size_t cols, size_t in_features,
                              const HiddenLayer* hidden) {
  if (rows == 0 || cols == 0) return fail(RST_ERR_SHAPE, "cross entropy of an empty batch");
  LossMirror mirror;
  RST_TRY(loss_mirror(e, &mirror));
  RST_TRY(launch_head_ce(e->stream, h, w, bias, truth, logits, grad, dx, mask, row_loss, e->d_loss, e->d_flags,
                         rows, cols, in_features, mirror, hidden));
  e->loss_valid = true;
  return RST_OK;
}

int engine_cross_entropy(rst_engine* e, double* row_loss, const double* pred, const double* truth,
                         double* grad_out, double* prob_out, size_t rows, size_t cols,
                         double* host_loss, bool* hits_done) {
  if (rows == 0 || cols == 0) return fail(RST_ERR_SHAPE, "cross entropy of an empty batch");
  unsigned* group_hits = nullptr;
  if (!row_loss) {  // the engine's own scratch; it moves when it grows, so nothing may keep its address
    // (with the hit count: a second stretch of the same scratch for the workgroups' counts)
    RST_TRY(engine_reserve_row_loss(e, hits_done ? 2 * rows : rows));
    row_loss = e->d_row_loss;
    if (hits_done) group_hits = reinterpret_cast<unsigned*>(e->d_row_loss + rows);
  }
  LossMirror mirror;
  RST_TRY(loss_mirror(e, &mirror));
  if (hits_done) {
    mirror.hits = e->hd_hits;
    mirror.group_hits = group_hits;
  }
  RST_TRY(launch_softmax_ce(e->stream, pred, truth, grad_out, prob_out, row_loss, e->d_loss,
                            e->d_flags, rows, cols, mirror, hits_done));
  e->loss_with_hits = hits_done && *hits_done;
  e->loss_valid = true;
  if (host_loss) return rst_loss_value(e, host_loss);
  return RST_OK;
}

}  // namespace rst

extern "C" {

int rst_linear_forward(rst_engine* e, const double* x, const double* weight, const double* bias,
                       double* out, size_t batch, size_t in_features, size_t out_features,
                       int fuse_relu) {
  RST_TRY(engine_activate(e));
  if (batch == 0 || out_features == 0) return RST_OK;
  if (!out || !weight || (!x && in_features))
    return fail(RST_ERR_INVALID_ARGUMENT, "linear_forward: null operand");
  RST_TRY(check_dim(batch, "batch"));
  RST_TRY(check_dim(in_features, "in_features"));
  RST_TRY(check_dim(out_features, "out_features"));
  GemmDesc d{};
  d.A = x; d.B = weight; d.C = out;
  d.M = (int)batch; d.N = (int)out_features; d.K = (int)in_features;
  d.lda = (long)in_features; d.ldb = (long)in_features; d.ldc = (long)out_features;
  d.a_kc = true; d.b_kc = true;
  d.bias = bias;
  if (bias) d.epilogue = fuse_relu ? EPI_BIAS_RELU : EPI_BIAS;
  else d.epilogue = fuse_relu ? EPI_RELU : EPI_NONE;
  d.workspace = e->d_gemm_ws; d.workspace_count = e->gemm_ws_count;
  return launch_gemm(e->stream, d);
}

int rst_linear_backward(rst_engine* e, const double* grad, const double* x, const double* weight,
                        double* grad_weight, double* grad_bias, double* grad_input,
                        const double* relu_mask_source, size_t batch, size_t in_features,
                        size_t out_features) {
  RST_TRY(engine_activate(e));
  if (!grad || !x || !weight || !grad_weight)
    return fail(RST_ERR_INVALID_ARGUMENT, "linear_backward: null operand");
  RST_TRY(check_dim(batch, "batch"));
  RST_TRY(check_dim(in_features, "in_features"));
  RST_TRY(check_dim(out_features, "out_features"));
  const double n = (double)batch;
  GemmDesc dw{};  // grad_weight[out,in] = (grad^T . x) / n
  dw.A = grad; dw.B = x; dw.C = grad_weight;
  dw.M = (int)out_features; dw.N = (int)in_features; dw.K = (int)batch;
  dw.lda = (long)out_features; dw.ldb = (long)in_features; dw.ldc = (long)in_features;
  dw.a_kc = false; dw.b_kc = false;
  dw.epilogue = EPI_DIVIDE; dw.divisor = n;
  // grad_bias[1,out] = colsum(grad) / n rides along in the same launch
  dw.colsum = (in_features > 0 && batch > 0) ? grad_bias : nullptr;
  dw.colsum_div = n;
  dw.workspace = e->d_gemm_ws; dw.workspace_count = e->gemm_ws_count;
  GemmDesc dx{};  // grad_input[batch,in] = grad . weight
  dx.A = grad; dx.B = weight; dx.C = grad_input;
  dx.M = (int)batch; dx.N = (int)in_features; dx.K = (int)out_features;
  dx.lda = (long)out_features; dx.ldb = (long)in_features; dx.ldc = (long)in_features;
  dx.a_kc = true; dx.b_kc = false;
  dx.epilogue = relu_mask_source ? EPI_MASK : EPI_NONE;
  dx.mask = relu_mask_source; dx.ldmask = (long)in_features;
  dx.workspace = e->d_gemm_ws; dx.workspace_count = e->gemm_ws_count;
  // two small products that do not depend on each other: one grid
  const GemmDesc both[2] = {dw, dx};
  if (grad_input && can_group_gemm(dw) && can_group_gemm(dx) &&
      gemm_group_workspace(both, 2) <= e->gemm_ws_count) {
    RST_TRY(launch_gemm_group(e->stream, both, 2));
  } else {
    RST_TRY(launch_gemm(e->stream, dw));
    if (grad_input) RST_TRY(launch_gemm(e->stream, dx));
  }
  if (grad_bias && !dw.colsum)
    RST_TRY(launch_column_mean(e->stream, grad, grad_bias, batch, out_features, n));
  return RST_OK;
}

int rst_relu_forward(rst_engine* e, const double* x, double* out, size_t count) {
  RST_TRY(engine_activate(e));
  if (count && (!x || !out)) return fail(RST_ERR_INVALID_ARGUMENT, "relu_forward: null operand");
  return launch_relu_forward(e->stream, x, out, count);
}

int rst_relu_backward(rst_engine* e, const double* grad, const double* x, double* out,
                      size_t count) {
  RST_TRY(engine_activate(e));
  if (count && (!grad || !x || !out))
    return fail(RST_ERR_INVALID_ARGUMENT, "relu_backward: null operand");
  return launch_relu_backward(e->stream, grad, x, out, count);
}

int rst_softmax_rows(rst_engine* e, const double* x, double* out, size_t rows, size_t cols) {
  RST_TRY(engine_activate(e));
  if (rows == 0 || cols == 0) return RST_OK;
  if (!x || !out) return fail(RST_ERR_INVALID_ARGUMENT, "softmax_rows: null operand");
  hipLaunchKernelGGL(reset_softmax_flag_kernel, dim3(1), dim3(1), 0, e->stream, e->d_flags);
  RST_HIP(hipGetLastError());
  RST_TRY(launch_softmax_ce(e->stream, x, nullptr, nullptr, out, nullptr, nullptr, e->d_flags, rows,
                            cols));
  RST_HIP(hipMemcpyAsync(e->h_flags, e->d_flags, 4 * sizeof(int), hipMemcpyDeviceToHost, e->stream));
  RST_HIP(hipStreamSynchronize(e->stream));
  if (e->h_flags[2] & 1)
    return fail(RST_ERR_NAN, "softmax: NaN in the input (the reference panics in softmax.rs:38)");
  return RST_OK;
}

int rst_softmax_forward(rst_engine* e, const double* x, double* out, size_t rows, size_t cols,
                        int axis) {
  if (axis == 1) return rst_softmax_rows(e, x, out, rows, cols);
  RST_TRY(engine_activate(e));
  if (axis != 0) return fail(RST_ERR_INVALID_ARGUMENT, "softmax axis %d of a 2-D array", axis);
  if (rows == 0 || cols == 0) return RST_OK;
  if (!x || !out) return fail(RST_ERR_INVALID_ARGUMENT, "softmax_forward: null operand");
  hipLaunchKernelGGL(reset_softmax_flag_kernel, dim3(1), dim3(1), 0, e->stream, e->d_flags);
  RST_HIP(hipGetLastError());
  RST_TRY(launch_softmax_columns(e->stream, x, out, e->d_flags, rows, cols));
  RST_HIP(hipMemcpyAsync(e->h_flags, e->d_flags, 4 * sizeof(int), hipMemcpyDeviceToHost, e->stream));
  RST_HIP(hipStreamSynchronize(e->stream));
  if (e->h_flags[2] & 1)
    return fail(RST_ERR_NAN, "softmax: NaN in the input (the reference panics in softmax.rs:38)");
  return RST_OK;
}

int rst_softmax_backward(rst_engine* e, const double* grad, const double* output, double* grad_input,
                         size_t rows, size_t cols) {
  RST_TRY(engine_activate(e));
  if (rows == 0 || cols == 0) return RST_OK;
  if (!grad || !output || !grad_input)
    return fail(RST_ERR_INVALID_ARGUMENT, "softmax_backward: null operand");
  RST_TRY(check_dim(rows, "rows"));
  RST_TRY(check_dim(cols, "cols"));
  double* jac = nullptr;
  RST_TRY(rst_malloc(e, cols * cols, &jac));
  int status = RST_OK;
  {  // jac[C,C] = output^T . output
    GemmDesc d{};
    d.A = output; d.B = output; d.C = jac;
    d.M = (int)cols; d.N = (int)cols; d.K = (int)rows;
    d.lda = (long)cols; d.ldb = (long)cols; d.ldc = (long)cols;
    d.a_kc = false; d.b_kc = false;
    d.epilogue = EPI_NONE;
    d.workspace = e->d_gemm_ws; d.workspace_count = e->gemm_ws_count;
    status = launch_gemm(e->stream, d);
  }
  if (status == RST_OK) status = launch_softmax_jacobian(e->stream, jac, cols);
  if (status == RST_OK) {  // grad_input[B,C] = grad . jac
    GemmDesc d{};
    d.A = grad; d.B = jac; d.C = grad_input;
    d.M = (int)rows; d.N = (int)cols; d.K = (int)cols;
    d.lda = (long)cols; d.ldb = (long)cols; d.ldc = (long)cols;
    d.a_kc = true; d.b_kc = false;
    d.epilogue = EPI_NONE;
    d.workspace = e->d_gemm_ws; d.workspace_count = e->gemm_ws_count;
    status = launch_gemm(e->stream, d);
  }
  (void)rst_free(e, jac);  // stream-ordered reuse: the launches above are already enqueued
  return status;
}

int rst_cross_entropy(rst_engine* e, const double* pred, const double* truth, double* grad_out,
                      double* prob_out, size_t rows, size_t cols, double* host_loss) {
  RST_TRY(engine_activate(e));
  if (!pred || !truth || !grad_out)
    return fail(RST_ERR_INVALID_ARGUMENT, "cross_entropy: null operand");
  return engine_cross_entropy(e, nullptr, pred, truth, grad_out, prob_out, rows, cols, host_loss);
}

int rst_loss_value(rst_engine* e, double* host_loss) {
  RST_TRY(engine_activate(e));
  if (!host_loss) return fail(RST_ERR_INVALID_ARGUMENT, "host_loss is null");
  if (!e->loss_valid) return fail(RST_ERR_STATE, "no loss has been computed on this engine");
  // the kernel that finished the loss stored it, and the NaN flag, in the pinned words as well
  RST_TRY(engine_wait_ticket(e, e->loss_ticket, e->loss_with_hits ? 3 : 1));
  int nan_flag;
  if (e->loss_ticket != 0) {  // announced by ticket: the record is certain to be there
    *host_loss = static_cast<volatile ResultSlot*>(e->h_slots)[0].value;
    nan_flag = (int)static_cast<volatile ResultSlot*>(e->h_slots)[0].flags;
    if (e->loss_with_hits) *e->h_hits = static_cast<volatile ResultSlot*>(e->h_slots)[1].count;
  } else {                    // the stream has drained: the plain words are there
    *host_loss = *static_cast<volatile double*>(e->h_loss);
    nan_flag = static_cast<volatile int*>(e->h_flags)[1];
  }
  if (nan_flag & 1)
    return fail(RST_ERR_NAN, "cross entropy: NaN logits (the reference panics in softmax.rs:38)");
  return RST_OK;
}

int rst_sgd_step_flat(rst_engine* e, double* parm, const double* grad, size_t count, double lr) {
  RST_TRY(engine_activate(e));
  if (count && (!parm || !grad)) return fail(RST_ERR_INVALID_ARGUMENT, "sgd: null operand");
  return launch_sgd_flat(e->stream, parm, grad, count, lr);
}

int rst_sgd_step(rst_engine* e, double* const* host_parm_ptrs, const double* const* host_grad_ptrs,
                 const size_t* host_counts, size_t tensor_count, double lr) {
  RST_TRY(engine_activate(e));
  if (tensor_count == 0) return RST_OK;
  if (!host_parm_ptrs || !host_grad_ptrs || !host_counts)
    return fail(RST_ERR_INVALID_ARGUMENT, "sgd: null table");
  std::vector<SgdTensor> table;
  table.reserve(tensor_count);
  unsigned long long blocks = 0;
  for (size_t i = 0; i < tensor_count; ++i) {
    if (host_counts[i] == 0) continue;
    if (!host_parm_ptrs[i] || !host_grad_ptrs[i])
      return fail(RST_ERR_INVALID_ARGUMENT, "sgd: tensor %zu has a null pointer", i);
    SgdTensor t;
    t.parm = host_parm_ptrs[i];
    t.grad = host_grad_ptrs[i];
    t.count = host_counts[i];
    t.first_block = blocks;
    blocks += sgd_blocks_for(t.count);
    table.push_back(t);
  }
  if (table.empty()) return RST_OK;
  const bool same = table.size() == e->sgd_table_host.size() &&
                    std::memcmp(table.data(), e->sgd_table_host.data(),
                                table.size() * sizeof(SgdTensor)) == 0;
  if (!same) {
    // an earlier launch may still be reading the device table
    RST_HIP(hipStreamSynchronize(e->stream));
    if (table.size() > e->sgd_table_capacity) {
      if (e->d_sgd_table) RST_HIP(hipFree(e->d_sgd_table));
      e->d_sgd_table = nullptr;
      e->sgd_table_capacity = 0;
      size_t cap = table.size() < 64 ? 64 : table.size() * 2;
      RST_HIP(hipMalloc(&e->d_sgd_table, cap * sizeof(SgdTensor)));
      e->sgd_table_capacity = cap;
    }
    RST_HIP(hipMemcpy(e->d_sgd_table, table.data(), table.size() * sizeof(SgdTensor),
                      hipMemcpyHostToDevice));
    e->sgd_table_host = table;
    e->sgd_total_blocks = blocks;
  }
  return launch_sgd_multi(e->stream, e->d_sgd_table, table.size(), blocks, lr);
}

int rst_accuracy(rst_engine* e, const double* pred, const double* truth, size_t rows, size_t cols,
                 double* host_accuracy) {
  RST_TRY(engine_activate(e));
  if (!pred || !truth || !host_accuracy)
    return fail(RST_ERR_INVALID_ARGUMENT, "accuracy: null operand");
  RST_TRY(engine_accuracy(e, pred, truth, rows, cols));
  *host_accuracy = (double)(*static_cast<volatile unsigned long long*>(e->h_hits)) / (double)rows;
  return RST_OK;
}

int rst_cross_entropy_accuracy(rst_engine* e, const double* pred, const double* truth, double* grad_out,
                               size_t rows, size_t cols, double* host_loss, double* host_accuracy) {
  RST_TRY(engine_activate(e));
  if (!pred || !truth || !grad_out || !host_loss || !host_accuracy)
    return fail(RST_ERR_INVALID_ARGUMENT, "cross_entropy_accuracy: null operand");
  bool hits_done = false;
  RST_TRY(engine_cross_entropy(e, nullptr, pred, truth, grad_out, nullptr, rows, cols, nullptr, &hits_done));
  // rows of at most 64 threads are counted by the cross-entropy launches themselves; for wider rows
  // the arg-max kernels follow on the stream, and either way the host waits once
  if (!hits_done) RST_TRY(engine_accuracy(e, pred, truth, rows, cols));
  const int status = rst_loss_value(e, host_loss);
  *host_accuracy = (double)(*static_cast<volatile unsigned long long*>(e->h_hits)) / (double)rows;
  return status;
}

int rst_fill_uniform(rst_engine* e, double* dst, size_t count, uint64_t seed, uint64_t stream,
                     double lo, double hi) {
  RST_TRY(engine_activate(e));
  if (count && !dst) return fail(RST_ERR_INVALID_ARGUMENT, "fill_uniform: null destination");
  return launch_fill_uniform(e->stream, dst, count, seed, stream, lo, hi);
}

int rst_fill_normal(rst_engine* e, double* dst, size_t count, uint64_t seed, uint64_t stream,
                    double mean, double std) {
  RST_TRY(engine_activate(e));
  if (count && !dst) return fail(RST_ERR_INVALID_ARGUMENT, "fill_normal: null destination");
  return launch_fill_normal(e->stream, dst, count, seed, stream, mean, std);
}

int rst_fill_one_hot(rst_engine* e, double* dst, size_t rows, size_t cols, uint64_t seed,
                     uint64_t stream) {
  RST_TRY(engine_activate(e));
  if (rows && cols && !dst) return fail(RST_ERR_INVALID_ARGUMENT, "fill_one_hot: null destination");
  return launch_fill_one_hot(e->stream, dst, rows, cols, seed, stream);
}

}  // extern "C"
