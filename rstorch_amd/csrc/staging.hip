// Input staging and parameter export/import: the steps either side of the training step.
//
// rst_stager pipelines host batches into HBM through `depth` slots of pinned host memory and
// device memory on a copy stream of its own (default priority), so the transfer of batch k+1
// overlaps the training step on batch k.  Labels travel as class indices and are expanded on the
// device into the dense one-hot truth that the loss takes (utils::one_hot, src/utils.rs:38-42):
// 4 bytes per row over PCIe instead of 8 * classes.  The reference assembles a batch on the host
// row by row (src/data/data_loader.rs:192-207); that host loop stays the caller's.
#include <cstring>
#include <new>

#include "common.h"

using namespace rst;

namespace {

__global__ __launch_bounds__(256) void one_hot_from_labels_kernel(double* __restrict__ dst,
                                                                 const uint32_t* __restrict__ labels,
                                                                 size_t rows, size_t cols) {
  const size_t n = rows * cols;
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * 256;
  for (; i < n; i += stride) {
    const size_t r = i / cols, c = i - r * cols;
    dst[i] = (labels[r] == (uint32_t)c) ? 1.0 : 0.0;
  }
}

struct Slot {
  double* h_x = nullptr;        // pinned
  double* h_truth = nullptr;    // pinned, dense submissions only (allocated on first use)
  uint32_t* h_labels = nullptr; // pinned
  double* d_x = nullptr;
  double* d_truth = nullptr;
  uint32_t* d_labels = nullptr;
  hipEvent_t copied = nullptr;    // copy stream: this slot's batch is in HBM
  hipEvent_t released = nullptr;  // engine stream: consumers of the previous batch are done
  size_t rows = 0;
  bool in_flight = false;         // submitted, not yet handed out
  bool ever_used = false;
};

}  // namespace

struct rst_stager {
  rst_engine* engine = nullptr;
  hipStream_t copy_stream = nullptr;
  size_t max_rows = 0, x_cols = 0, classes = 0;
  std::vector<Slot> slots;
  size_t head = 0;  // next slot to fill
  size_t tail = 0;  // next slot to hand out
  size_t pending = 0;
};

namespace {

int begin_submit(rst_stager* s, size_t rows, Slot** out) {
  if (!s) return fail(RST_ERR_INVALID_ARGUMENT, "stager is null");
  RST_TRY(engine_activate(s->engine));
  if (rows == 0 || rows > s->max_rows)
    return fail(RST_ERR_SHAPE, "batch of %zu rows does not fit the stager (max %zu)", rows, s->max_rows);
  if (s->pending == s->slots.size())
    return fail(RST_ERR_STATE, "all %zu slots are submitted and none has been taken", s->slots.size());
  Slot& slot = s->slots[s->head];
  // the pinned buffers are free once the previous transfer out of them has finished
  if (slot.ever_used) RST_HIP(hipEventSynchronize(slot.copied));
  // the device buffers are free once everything enqueued on the engine's stream so far (which
  // includes every consumer of the batch this slot held) has run
  RST_HIP(hipEventRecord(slot.released, s->engine->stream));
  RST_HIP(hipStreamWaitEvent(s->copy_stream, slot.released, 0));
  slot.rows = rows;
  *out = &slot;
  return RST_OK;
}

int end_submit(rst_stager* s, Slot* slot) {
  RST_HIP(hipEventRecord(slot->copied, s->copy_stream));
  slot->in_flight = true;
  slot->ever_used = true;
  s->head = (s->head + 1) % s->slots.size();
  s->pending += 1;
  return RST_OK;
}

}  // namespace

extern "C" {

int rst_stager_create(rst_engine* e, size_t max_rows, size_t x_cols, size_t classes, int depth,
                      rst_stager** out) {
  RST_TRY(engine_activate(e));
  if (!out) return fail(RST_ERR_INVALID_ARGUMENT, "out is null");
  *out = nullptr;
  if (max_rows == 0 || x_cols == 0 || classes == 0 || depth < 1 || depth > 16)
    return fail(RST_ERR_INVALID_ARGUMENT, "stager needs rows, columns, classes > 0 and 1 <= depth <= 16");
  rst_stager* s = new (std::nothrow) rst_stager();
  if (!s) return fail(RST_ERR_OUT_OF_MEMORY, "host allocation failed");
  s->engine = e;
  s->max_rows = max_rows; s->x_cols = x_cols; s->classes = classes;
  s->slots.resize((size_t)depth);
  hipError_t err = hipStreamCreateWithFlags(&s->copy_stream, hipStreamNonBlocking);
  for (auto& slot : s->slots) {
    if (err == hipSuccess) err = hipHostMalloc(&slot.h_x, max_rows * x_cols * sizeof(double), hipHostMallocDefault);
    if (err == hipSuccess) err = hipHostMalloc(&slot.h_labels, max_rows * sizeof(uint32_t), hipHostMallocDefault);
    if (err == hipSuccess) err = hipMalloc(&slot.d_x, max_rows * x_cols * sizeof(double));
    if (err == hipSuccess) err = hipMalloc(&slot.d_truth, max_rows * classes * sizeof(double));
    if (err == hipSuccess) err = hipMalloc(&slot.d_labels, max_rows * sizeof(uint32_t));
    if (err == hipSuccess) err = hipEventCreateWithFlags(&slot.copied, hipEventDisableTiming);
    if (err == hipSuccess) err = hipEventCreateWithFlags(&slot.released, hipEventDisableTiming);
  }
  if (err != hipSuccess) {
    int status = fail_hip(err, "stager set-up", __FILE__, __LINE__);
    rst_stager_destroy(s);
    return status;
  }
  *out = s;
  return RST_OK;
}

int rst_stager_destroy(rst_stager* s) {
  if (!s) return RST_OK;
  (void)hipSetDevice(s->engine->device);
  if (s->copy_stream) (void)hipStreamSynchronize(s->copy_stream);
  (void)hipStreamSynchronize(s->engine->stream);
  for (auto& slot : s->slots) {
    if (slot.h_x) (void)hipHostFree(slot.h_x);
    if (slot.h_truth) (void)hipHostFree(slot.h_truth);
    if (slot.h_labels) (void)hipHostFree(slot.h_labels);
    if (slot.d_x) (void)hipFree(slot.d_x);
    if (slot.d_truth) (void)hipFree(slot.d_truth);
    if (slot.d_labels) (void)hipFree(slot.d_labels);
    if (slot.copied) (void)hipEventDestroy(slot.copied);
    if (slot.released) (void)hipEventDestroy(slot.released);
  }
  if (s->copy_stream) (void)hipStreamDestroy(s->copy_stream);
  delete s;
  return RST_OK;
}

int rst_stager_acquire_host(rst_stager* s, double** host_x, uint32_t** host_labels);
int rst_stager_commit_labels(rst_stager* s, size_t rows);

int rst_stager_submit_labels(rst_stager* s, const double* host_x, const uint32_t* host_labels,
                             size_t rows) {
  if (!host_x || !host_labels) return fail(RST_ERR_INVALID_ARGUMENT, "null host batch");
  if (!s) return fail(RST_ERR_INVALID_ARGUMENT, "stager is null");
  if (rows == 0 || rows > s->max_rows)
    return fail(RST_ERR_SHAPE, "batch of %zu rows does not fit the stager (max %zu)", rows, s->max_rows);
  double* px = nullptr;
  uint32_t* pl = nullptr;
  RST_TRY(rst_stager_acquire_host(s, &px, &pl));
  std::memcpy(px, host_x, rows * s->x_cols * sizeof(double));
  std::memcpy(pl, host_labels, rows * sizeof(uint32_t));
  return rst_stager_commit_labels(s, rows);
}

int rst_stager_acquire_host(rst_stager* s, double** host_x, uint32_t** host_labels) {
  if (!s) return fail(RST_ERR_INVALID_ARGUMENT, "stager is null");
  RST_TRY(engine_activate(s->engine));
  if (s->pending == s->slots.size())
    return fail(RST_ERR_STATE, "all %zu slots are submitted and none has been taken", s->slots.size());
  Slot& slot = s->slots[s->head];
  if (slot.ever_used) RST_HIP(hipEventSynchronize(slot.copied));  // its last transfer has left
  if (host_x) *host_x = slot.h_x;
  if (host_labels) *host_labels = slot.h_labels;
  return RST_OK;
}

int rst_stager_commit_labels(rst_stager* s, size_t rows) {
  Slot* slot = nullptr;
  RST_TRY(begin_submit(s, rows, &slot));
  for (size_t r = 0; r < rows; ++r)
    if (slot->h_labels[r] >= s->classes)
      return fail(RST_ERR_INVALID_ARGUMENT, "label %u of row %zu is not below %zu classes",
                  slot->h_labels[r], r, s->classes);
  RST_HIP(hipMemcpyAsync(slot->d_x, slot->h_x, rows * s->x_cols * sizeof(double), hipMemcpyHostToDevice,
                         s->copy_stream));
  RST_HIP(hipMemcpyAsync(slot->d_labels, slot->h_labels, rows * sizeof(uint32_t), hipMemcpyHostToDevice,
                         s->copy_stream));
  size_t n = rows * s->classes;
  size_t blocks = (n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(one_hot_from_labels_kernel, dim3((unsigned)blocks), dim3(256), 0, s->copy_stream,
                     slot->d_truth, slot->d_labels, rows, s->classes);
  RST_HIP(hipGetLastError());
  return end_submit(s, slot);
}

int rst_stager_submit_dense(rst_stager* s, const double* host_x, const double* host_truth,
                            size_t rows) {
  if (!host_x || !host_truth) return fail(RST_ERR_INVALID_ARGUMENT, "null host batch");
  Slot* slot = nullptr;
  RST_TRY(begin_submit(s, rows, &slot));
  if (!slot->h_truth)
    RST_HIP(hipHostMalloc(&slot->h_truth, s->max_rows * s->classes * sizeof(double), hipHostMallocDefault));
  std::memcpy(slot->h_x, host_x, rows * s->x_cols * sizeof(double));
  std::memcpy(slot->h_truth, host_truth, rows * s->classes * sizeof(double));
  RST_HIP(hipMemcpyAsync(slot->d_x, slot->h_x, rows * s->x_cols * sizeof(double), hipMemcpyHostToDevice,
                         s->copy_stream));
  RST_HIP(hipMemcpyAsync(slot->d_truth, slot->h_truth, rows * s->classes * sizeof(double),
                         hipMemcpyHostToDevice, s->copy_stream));
  return end_submit(s, slot);
}

int rst_stager_next(rst_stager* s, const double** x_dev, const double** truth_dev, size_t* rows) {
  if (!s) return fail(RST_ERR_INVALID_ARGUMENT, "stager is null");
  RST_TRY(engine_activate(s->engine));
  if (s->pending == 0) return fail(RST_ERR_STATE, "no batch has been submitted");
  Slot& slot = s->slots[s->tail];
  RST_HIP(hipStreamWaitEvent(s->engine->stream, slot.copied, 0));
  slot.in_flight = false;
  s->tail = (s->tail + 1) % s->slots.size();
  s->pending -= 1;
  if (x_dev) *x_dev = slot.d_x;
  if (truth_dev) *truth_dev = slot.d_truth;
  if (rows) *rows = slot.rows;
  return RST_OK;
}

}  // extern "C"
