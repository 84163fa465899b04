// Shared declarations of the gfx950 backend: engine state, error plumbing and the internal
// launch functions that the C ABI (ops.hip, model.hip) is built from.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/rstorch_hip.h"

namespace rst {

// ---- error plumbing ------------------------------------------------------------------------
int fail(int status, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int fail_hip(hipError_t err, const char* what, const char* file, int line);
void clear_error();

#define RST_HIP(expr)                                                          \
  do {                                                                         \
    hipError_t rst_hip_err_ = (expr);                                          \
    if (rst_hip_err_ != hipSuccess)                                            \
      return ::rst::fail_hip(rst_hip_err_, #expr, __FILE__, __LINE__);         \
  } while (0)

#define RST_TRY(expr)                      \
  do {                                     \
    int rst_status_ = (expr);              \
    if (rst_status_ != RST_OK) return rst_status_; \
  } while (0)

// ---- epilogues of the contraction kernels ----------------------------------------------------
enum Epilogue {
  EPI_NONE = 0,
  EPI_BIAS = 1,       // C = acc + bias[col]                       (Linear forward)
  EPI_BIAS_RELU = 2,  // C = max(acc + bias[col], 0)               (Linear forward + ReLU)
  EPI_DIVIDE = 3,     // C = acc / divisor                         (weight gradient)
  EPI_MASK = 4,       // C = acc * (mask[row,col] > 0 ? 1 : 0)     (input gradient + ReLU backward)
  EPI_RELU = 5        // C = max(acc, 0)                           (Linear without bias + ReLU)
};

// C[M,N] = sum_k A(i,k) * B(k,j), every matrix dense row-major.
//   a_kc: A(i,k) = A[i*lda + k]  (contraction index contiguous), else A(i,k) = A[k*lda + i]
//   b_kc: B(k,j) = B[j*ldb + k]  (contraction index contiguous), else B(k,j) = B[k*ldb + j]
struct GemmDesc {
  const double* A;
  const double* B;
  double* C;
  int M, N, K;
  long lda, ldb, ldc;
  bool a_kc, b_kc;
  int epilogue;
  const double* bias;  // [N]
  double divisor;
  const double* mask;  // [M, ldmask]
  long ldmask;
  // only with a_kc == false (weight gradient): colsum[i] = (sum_k A(i,k)) / colsum_div, i.e.
  // the bias gradient, computed by the workgroups of the first tile column.  NULL: not wanted.
  double* colsum;
  double colsum_div;
  // only with EPI_DIVIDE (the fused training step): after the gradient is stored, the parameter
  // at the same index gets parm -= lr * grad (two roundings); sgd_bias likewise next to colsum
  double* sgd_parm;
  double* sgd_bias;
  double sgd_lr;
  // scratch for split-K partial products (small outputs with a long contraction); NULL: never split
  double* workspace;
  size_t workspace_count;
};

int launch_gemm(hipStream_t stream, const GemmDesc& d);
// Two independent contractions, the input gradient of one layer (A contraction-contiguous, B
// output-contiguous) and the weight gradient of another (both output-contiguous), in one grid.
// Possible when both run as unsplit 128x128 direct-to-LDS tiles and the first alone would
// under-fill the chip (fewer than 512 tiles).
bool can_pair_gemm(const GemmDesc& input_grad, const GemmDesc& weight_grad);
int launch_gemm_pair(hipStream_t stream, const GemmDesc& input_grad, const GemmDesc& weight_grad);
// Several small weight gradients (both operands output-contiguous, each a launch of 32x32 tiles
// on its own, with or without K slices) in one grid, plus one shared reduction grid for the
// sliced ones; same results as launch_gemm on each, except that from a batch of about 4096 a
// group of weight gradients runs as K-sliced 128x128 tiles whose slices differ from a lone launch's
// (equal within rounding, 1e-13).  The descriptors share one workspace, of which the group as a
// whole takes gemm_group_workspace(d, count) doubles.
bool can_group_gemm(const GemmDesc& d);
size_t gemm_group_workspace(const GemmDesc* d, int count);
int max_gemm_group();
int launch_gemm_group(hipStream_t stream, const GemmDesc* d, int count);

// ---- streaming kernels -----------------------------------------------------------------------
int launch_relu_forward(hipStream_t s, const double* x, double* out, size_t n);
int launch_relu_backward(hipStream_t s, const double* g, const double* x, double* out, size_t n);
int launch_fill(hipStream_t s, double* dst, size_t n, double value);
// out[j] = (sum_r g[r, j]) / divisor, rows added in order inside fixed groups (deterministic)
int launch_column_mean(hipStream_t s, const double* g, double* out, size_t rows, size_t cols,
                       double divisor);
int launch_sgd_flat(hipStream_t s, double* parm, const double* grad, size_t n, double lr);

struct SgdTensor {
  double* parm;
  const double* grad;
  unsigned long long count;
  unsigned long long first_block;  // prefix of blocks, filled by the launcher
};
// table: device copy of `n_tensors` SgdTensor entries followed by a sentinel
int launch_sgd_multi(hipStream_t s, const SgdTensor* device_table, size_t n_tensors,
                     unsigned long long total_blocks, double lr);
unsigned long long sgd_blocks_for(unsigned long long count);

// softmax / cross entropy.  grad_out != NULL: cross entropy (row kernel + a one-workgroup
// reduction; a batch of at most 64 rows that fits one workgroup is finished by the row kernel) -
// row_loss is [rows] scratch, loss[0] receives -(sum)/rows, flags[1] the NaN flag of this call
// (flags[0] is a working word left at zero).  grad_out == NULL: softmax only, prob_out is written
// and flags[2] is set on a NaN input.
// LossMirror: device-visible addresses of pinned host words that receive the loss and flags[1]
// as well (written by the thread that finishes the loss), so that the host can read them after a
// stream synchronisation without a copy in between.  Null members: no mirror.
// slots / ticket: the same thread also writes the result, together with the launch's ticket, into a
// 16-byte record in pinned host memory with ONE 16-byte store (slots[0]: loss and NaN flag, slots[1]:
// hit count): the host can then wait for exactly this result by polling the record instead of
// synchronising the stream, and a record that shows the ticket holds the result whatever order
// separate writes to host memory may arrive in.  hits: when set, a cross entropy whose whole batch
// sits in one workgroup also counts the rows whose first arg-max agrees between logits and truth
// (src/utils.rs:44-65) and stores the count there; launch_softmax_ce reports whether it did.
struct alignas(16) ResultSlot {
  union {
    double value;
    unsigned long long count;
  };
  unsigned flags;
  unsigned ticket;
};
static_assert(sizeof(ResultSlot) == 16, "one 16-byte store");
struct LossMirror {
  double* loss = nullptr;
  int* flags = nullptr;
  ResultSlot* slots = nullptr;
  unsigned ticket = 0;
  unsigned long long* hits = nullptr;
  // device scratch, one word per workgroup of the row kernel, for the hit counts of a cross entropy
  // on several workgroups (added up by the reduction launch); NULL: such a launch does not count
  unsigned* group_hits = nullptr;
};
int launch_softmax_ce(hipStream_t s, const double* z, const double* t, double* grad_out,
                      double* prob_out, double* row_loss, double* loss, int* flags, size_t rows,
                      size_t cols, LossMirror mirror = LossMirror(), bool* hits_done = nullptr);
// The classifier head of a training step in one launch: logits = h.w^T + bias ([rows, cols], h is
// [rows, in_features] with contiguous rows), cross entropy against truth with grad = -(truth - p),
// dx = grad.w (NULL: not wanted; mask: zeroed where h <= 0, the backward of a ReLU that produced h)
// and the loss, finished by the workgroup that arrives last (flags[4..5], one 64-bit word, counts
// arrivals and is left at zero; flags[1], loss and the mirror as for launch_softmax_ce; row_loss is
// [rows] scratch).  Only for shapes
// head_ce_supported accepts: few classes on few inputs, where the weight matrix sits in LDS.
bool head_ce_supported(size_t cols, size_t in_features);
// The Linear in front of the head, run by the same launch when it is small enough for its weights to
// sit in LDS (tail_ce_supported): output = input.weight^T + bias ([rows, in_features] -> the head's
// input, with the ReLU between the two applied when the head's `mask` says there is one);
// input_grad = (the head's dx).weight, zeroed where input <= 0 if mask_input_grad, or NULL.
struct HiddenLayer {
  const double* input;
  const double* weight;  // [head in_features, in_features]
  const double* bias;
  double* output;        // [rows, head in_features]: written here, and the head's `h` is ignored
  double* input_grad;    // [rows, in_features] or NULL
  size_t in_features;
  bool mask_input_grad;
};
bool tail_ce_supported(size_t cols, size_t hidden, size_t in_features, size_t lds_limit);
int launch_head_ce(hipStream_t s, const double* h, const double* w, const double* bias, const double* truth,
                   double* logits, double* grad, double* dx, bool mask, double* row_loss, double* loss,
                   int* flags, size_t rows, size_t cols, size_t in_features, LossMirror mirror = LossMirror(),
                   const HiddenLayer* hidden = nullptr);
int launch_softmax_columns(hipStream_t s, const double* z, double* out, int* flags, size_t rows,
                           size_t cols);
int launch_softmax_jacobian(hipStream_t s, double* jac, size_t cols);
// hits[0] = number of rows whose first arg-max agrees
// hits_mirror: device-visible address of a pinned host word; *mirrored tells whether the count
// was also written there (small inputs, counted by one workgroup without atomics)
// slots / ticket: as in LossMirror; the mirrored count also goes to slots[1]
int launch_accuracy(hipStream_t s, const double* pred, const double* truth, size_t rows,
                    size_t cols, unsigned long long* hits, unsigned long long* hits_mirror = nullptr,
                    bool* mirrored = nullptr, ResultSlot* slots = nullptr, unsigned ticket = 0);

int launch_fill_uniform(hipStream_t s, double* dst, size_t n, uint64_t seed, uint64_t stream,
                        double lo, double hi);
int launch_fill_normal(hipStream_t s, double* dst, size_t n, uint64_t seed, uint64_t stream,
                       double mean, double std);
int launch_fill_one_hot(hipStream_t s, double* dst, size_t rows, size_t cols, uint64_t seed,
                        uint64_t stream);

}  // namespace rst

// ---- engine ------------------------------------------------------------------------------------
struct rst_engine {
  int device = 0;
  hipStream_t stream = nullptr;
  hipDeviceProp_t props;
  // device-side scalars and their pinned host mirrors
  double* d_loss = nullptr;
  int* d_flags = nullptr;
  unsigned long long* d_hits = nullptr;
  double* h_loss = nullptr;  // pinned
  int* h_flags = nullptr;    // pinned
  unsigned long long* h_hits = nullptr;  // pinned
  // the same three words as the device addresses them (kernels store scalar results there)
  double* hd_loss = nullptr;
  int* hd_flags = nullptr;
  unsigned long long* hd_hits = nullptr;
  // results are announced by a ticket: a kernel that finishes a scalar writes it, with the number
  // the launch was given, into a pinned 16-byte record, and the host polls that record (a few
  // microseconds sooner than a stream synchronisation returns).  Tickets are never 0.  loss_ticket:
  // the ticket of the latest loss, 0 when that loss was enqueued without one (recorded into a graph,
  // whose replays would all write the same number); loss_with_hits: that launch also counted hits.
  rst::ResultSlot* h_slots = nullptr;   // pinned: [0] loss, [1] hit count
  rst::ResultSlot* hd_slots = nullptr;  // the same records as the device addresses them
  unsigned tickets_issued = 0;
  unsigned loss_ticket = 0;
  bool loss_with_hits = false;
  bool loss_valid = false;
  // split-K scratch of the contraction kernels (fixed size, allocated with the engine)
  double* d_gemm_ws = nullptr;
  size_t gemm_ws_count = 0;
  // per-row loss scratch
  double* d_row_loss = nullptr;
  size_t row_loss_capacity = 0;
  // rst_malloc / rst_free block cache (bytes -> free blocks) and the live allocations
  std::unordered_map<size_t, std::vector<void*>> free_blocks;
  std::unordered_map<void*, size_t> live_blocks;
  size_t cached_bytes = 0;
  // SGD descriptor table cache
  rst::SgdTensor* d_sgd_table = nullptr;
  size_t sgd_table_capacity = 0;
  std::vector<rst::SgdTensor> sgd_table_host;
  unsigned long long sgd_total_blocks = 0;
};

namespace rst {
int engine_activate(rst_engine* e);
// a fresh ticket (never 0)
unsigned engine_next_ticket(rst_engine* e);
// waits until the kernel that was given `ticket` has written the records named by `slots` (bit 0:
// loss, bit 1: hit count); ticket 0: until the stream has drained
int engine_wait_ticket(rst_engine* e, unsigned ticket, int slots);
int engine_reserve_row_loss(rst_engine* e, size_t rows);
// looks up, once per device, the address of the fixed scratch behind rst_cross_entropy_static
int static_scratch_setup(int device, hipStream_t stream);
// row_loss: [rows] scratch of the caller, or NULL for the engine's own (which is reallocated when
// it grows: only for launches that are not recorded into a graph)
// hits_done != NULL: the arg-max agreement count is wanted as well (into the engine's pinned hit
// word); *hits_done tells whether the cross-entropy launch took it
int engine_cross_entropy(rst_engine* e, double* row_loss, const double* pred, const double* truth,
                         double* grad_out, double* prob_out, size_t rows, size_t cols,
                         double* host_loss, bool* hits_done = nullptr);
// the arg-max agreement count of pred / truth into the engine's pinned hit word: enqueues, runs
// `ahead` (launches the caller wants on the stream before the host waits), waits
int engine_accuracy(rst_engine* e, const double* pred, const double* truth, size_t rows, size_t cols,
                    int (*ahead)(void*) = nullptr, void* ahead_arg = nullptr);
// the fused classifier head (launch_head_ce) with the engine's loss words, mirror and ticket
int engine_head_cross_entropy(rst_engine* e, double* row_loss, const double* h, const double* w,
                              const double* bias, const double* truth, double* logits, double* grad,
                              double* dx, bool mask, size_t rows, size_t cols, size_t in_features,
                              const rst::HiddenLayer* hidden = nullptr);
}  // namespace rst
