// Cross entropy for callers that cannot allocate device memory (code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc): the per-row loss terms, the loss word and
// the NaN flags, which rst_cross_entropy keeps in buffers the engine allocates and grows, live
// here in one fixed array that is part of the library's device image.  Each GPU holds its own
// copy of that array at its own address for as long as the process lives.
#include <atomic>
#include <mutex>

#include "common.h"

namespace rst {
namespace {

constexpr size_t kStaticRows = RST_STATIC_CROSS_ENTROPY_MAX_ROWS;
constexpr size_t kLossSlot = kStaticRows;       // one double
constexpr size_t kFlagSlot = kStaticRows + 2;   // four ints, 16-byte aligned
constexpr size_t kScratchDoubles = kStaticRows + 32;

// In host code this name is only a handle for hipGetSymbolAddress: the device address is asked
// for once per device (static_scratch_setup) and everything below uses that pointer.
static __device__ __align__(256) double scratch[kScratchDoubles];

constexpr int kMaxDevices = 64;
// filled in once per device, under the lock, by the first engine that opens the device; read
// without the lock afterwards (an entry never changes once it is set)
std::mutex g_scratch_lock;
std::atomic<double*> g_scratch_ptr[kMaxDevices] = {};
// a call that stopped between its two launches may have left the working NaN word set
std::atomic<bool> g_scratch_dirty[kMaxDevices] = {};

__global__ void clear_flags_kernel(int* flags) {
  if (threadIdx.x < 4) flags[threadIdx.x] = 0;
}

}  // namespace

// Called by rst_engine_create with `device` current.  Only the first call for a device does
// anything: it looks the array's address up.  The array is zero when the device image is loaded,
// which is the state the flag words must start in, so nothing is launched here - a later engine
// on the same GPU must not touch words that another engine's call may be using.
int static_scratch_setup(int device, hipStream_t /*stream*/) {
  if (device < 0 || device >= kMaxDevices)
    return fail(RST_ERR_UNSUPPORTED, "device %d: the static scratch table holds %d devices", device, kMaxDevices);
  if (g_scratch_ptr[device].load(std::memory_order_acquire)) return RST_OK;
  std::lock_guard<std::mutex> guard(g_scratch_lock);
  if (g_scratch_ptr[device].load(std::memory_order_relaxed)) return RST_OK;
  void* ptr = nullptr;
  RST_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
  if (!ptr) return fail(RST_ERR_HIP, "hipGetSymbolAddress returned a null address");
  g_scratch_ptr[device].store(static_cast<double*>(ptr), std::memory_order_release);
  return RST_OK;
}

}  // namespace rst

using namespace rst;

extern "C" int rst_cross_entropy_static(rst_engine* e, const double* pred, const double* truth,
                                        double* grad_out, size_t rows, size_t cols,
                                        double* host_loss) {
  RST_TRY(engine_activate(e));
  if (!pred || !truth || !grad_out)
    return fail(RST_ERR_INVALID_ARGUMENT, "cross_entropy_static: null operand");
  if (rows == 0 || cols == 0) return fail(RST_ERR_SHAPE, "cross entropy of an empty batch");
  if (rows > kStaticRows)
    return fail(RST_ERR_UNSUPPORTED,
                "cross_entropy_static: %zu rows exceed the fixed scratch of %zu rows; use rst_cross_entropy",
                rows, kStaticRows);
  double* base = (e->device >= 0 && e->device < kMaxDevices)
                     ? g_scratch_ptr[e->device].load(std::memory_order_acquire) : nullptr;
  if (!base) return fail(RST_ERR_STATE, "the static scratch of device %d was never set up", e->device);
  int* flags = reinterpret_cast<int*>(base + kFlagSlot);
  if (g_scratch_dirty[e->device].exchange(true)) {
    hipLaunchKernelGGL(clear_flags_kernel, dim3(1), dim3(64), 0, e->stream, flags);
    RST_HIP(hipGetLastError());
  }
  LossMirror mirror;
  mirror.loss = e->hd_loss;
  mirror.flags = e->hd_flags;
  e->loss_ticket = 0;  // no ticket: the caller may be recording this call into a graph
  RST_TRY(launch_softmax_ce(e->stream, pred, truth, grad_out, nullptr, base, base + kLossSlot, flags,
                            rows, cols, mirror));
  g_scratch_dirty[e->device] = false;  // the reduction launch re-arms the working word
  e->loss_valid = true;
  if (host_loss) return rst_loss_value(e, host_loss);
  return RST_OK;
}
