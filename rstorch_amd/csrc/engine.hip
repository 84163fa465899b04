// Engine: device, stream, error reporting, device memory and stream timing.
#include "common.h"

#include <immintrin.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <new>

namespace rst {

namespace {
thread_local std::string g_error;
thread_local int g_hip_error = 0;
}  // namespace

int fail(int status, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_error = buf;
  g_hip_error = 0;
  return status;
}

int fail_hip(hipError_t err, const char* what, const char* file, int line) {
  char buf[512];
  snprintf(buf, sizeof(buf), "HIP error %d (%s) from %s at %s:%d", (int)err, hipGetErrorString(err),
           what, file, line);
  g_error = buf;
  g_hip_error = (int)err;
  return err == hipErrorOutOfMemory ? RST_ERR_OUT_OF_MEMORY : RST_ERR_HIP;
}

void clear_error() {
  g_error.clear();
  g_hip_error = 0;
}

int engine_activate(rst_engine* e) {
  if (!e) return fail(RST_ERR_INVALID_ARGUMENT, "engine is null");
  RST_HIP(hipSetDevice(e->device));
  return RST_OK;
}

unsigned engine_next_ticket(rst_engine* e) {
  if (++e->tickets_issued == 0) ++e->tickets_issued;
  return e->tickets_issued;
}

int engine_wait_ticket(rst_engine* e, unsigned ticket, int slots) {
  if (ticket != 0) {
    // about 100 us of polling; a result that takes longer is waited for the ordinary way
    for (int i = 0; i < 4000; ++i) {
      const bool loss_there = !(slots & 1) || __atomic_load_n(&e->h_slots[0].ticket, __ATOMIC_ACQUIRE) == ticket;
      const bool hits_there = !(slots & 2) || __atomic_load_n(&e->h_slots[1].ticket, __ATOMIC_ACQUIRE) == ticket;
      if (loss_there && hits_there) return RST_OK;
      _mm_pause();
    }
  }
  RST_HIP(hipStreamSynchronize(e->stream));
  return RST_OK;
}

int engine_reserve_row_loss(rst_engine* e, size_t rows) {
  if (rows <= e->row_loss_capacity) return RST_OK;
  if (e->d_row_loss) {
    RST_HIP(hipStreamSynchronize(e->stream));
    RST_HIP(hipFree(e->d_row_loss));
    e->d_row_loss = nullptr;
    e->row_loss_capacity = 0;
  }
  size_t cap = rows < 1024 ? 1024 : rows;
  RST_HIP(hipMalloc(&e->d_row_loss, cap * sizeof(double)));
  e->row_loss_capacity = cap;
  return RST_OK;
}

}  // namespace rst

using namespace rst;

extern "C" {

const char* rst_last_error(void) { return g_error.c_str(); }
int rst_last_hip_error(void) { return g_hip_error; }

const char* rst_status_string(int status) {
  switch (status) {
    case RST_OK: return "ok";
    case RST_ERR_INVALID_ARGUMENT: return "invalid argument";
    case RST_ERR_SHAPE: return "shape mismatch";
    case RST_ERR_STATE: return "invalid state";
    case RST_ERR_HIP: return "HIP error";
    case RST_ERR_NAN: return "NaN logits";
    case RST_ERR_OUT_OF_MEMORY: return "out of device memory";
    case RST_ERR_UNSUPPORTED: return "unsupported";
    default: return "unknown status";
  }
}

int rst_engine_create(int device, rst_engine** out) {
  if (!out) return fail(RST_ERR_INVALID_ARGUMENT, "out is null");
  *out = nullptr;
  int n = 0;
  RST_HIP(hipGetDeviceCount(&n));
  if (device < 0 || device >= n)
    return fail(RST_ERR_INVALID_ARGUMENT, "device %d not present (%d visible)", device, n);
  RST_HIP(hipSetDevice(device));
  rst_engine* e = new (std::nothrow) rst_engine();
  if (!e) return fail(RST_ERR_OUT_OF_MEMORY, "host allocation failed");
  e->device = device;
  hipError_t err = hipGetDeviceProperties(&e->props, device);
  if (err == hipSuccess) err = hipStreamCreateWithFlags(&e->stream, hipStreamNonBlocking);
  if (err == hipSuccess) err = hipMalloc(&e->d_loss, sizeof(double));
  if (err == hipSuccess) err = hipMalloc(&e->d_flags, 8 * sizeof(int));
  if (err == hipSuccess) err = hipMalloc(&e->d_hits, sizeof(unsigned long long));
  e->gemm_ws_count = (size_t)16 << 20;  // 16 Mi doubles = 128 MiB
  if (err == hipSuccess) err = hipMalloc(&e->d_gemm_ws, e->gemm_ws_count * sizeof(double));
  if (err == hipSuccess) err = hipHostMalloc(&e->h_loss, sizeof(double), hipHostMallocDefault);
  if (err == hipSuccess) err = hipHostMalloc(&e->h_flags, 4 * sizeof(int), hipHostMallocDefault);
  if (err == hipSuccess)
    err = hipHostMalloc(&e->h_hits, sizeof(unsigned long long), hipHostMallocDefault);
  if (err == hipSuccess) err = hipHostMalloc(&e->h_slots, 2 * sizeof(ResultSlot), hipHostMallocDefault);
  if (err == hipSuccess) err = hipHostGetDevicePointer((void**)&e->hd_slots, e->h_slots, 0);
  if (err == hipSuccess) std::memset(e->h_slots, 0, 2 * sizeof(ResultSlot));
  if (err == hipSuccess) err = hipHostGetDevicePointer((void**)&e->hd_loss, e->h_loss, 0);
  if (err == hipSuccess) err = hipHostGetDevicePointer((void**)&e->hd_flags, e->h_flags, 0);
  if (err == hipSuccess) err = hipHostGetDevicePointer((void**)&e->hd_hits, e->h_hits, 0);
  if (err == hipSuccess) {
    *e->h_loss = 0.0;
    e->h_flags[0] = e->h_flags[1] = e->h_flags[2] = e->h_flags[3] = 0;
    *e->h_hits = 0;
  }
  if (err == hipSuccess) err = hipMemsetAsync(e->d_flags, 0, 8 * sizeof(int), e->stream);
  if (err != hipSuccess) {
    int status = fail_hip(err, "engine set-up", __FILE__, __LINE__);
    rst_engine_destroy(e);
    return status;
  }
  int status = static_scratch_setup(device, e->stream);
  if (status == RST_OK && (err = hipStreamSynchronize(e->stream)) != hipSuccess)
    status = fail_hip(err, "engine set-up", __FILE__, __LINE__);
  if (status != RST_OK) {
    rst_engine_destroy(e);
    return status;
  }
  *out = e;
  return RST_OK;
}

int rst_engine_destroy(rst_engine* e) {
  if (!e) return RST_OK;
  (void)hipSetDevice(e->device);
  if (e->stream) (void)hipStreamSynchronize(e->stream);
  for (auto& kv : e->free_blocks)
    for (void* p : kv.second) (void)hipFree(p);
  for (auto& kv : e->live_blocks) (void)hipFree(kv.first);
  if (e->d_loss) (void)hipFree(e->d_loss);
  if (e->d_flags) (void)hipFree(e->d_flags);
  if (e->d_hits) (void)hipFree(e->d_hits);
  if (e->d_gemm_ws) (void)hipFree(e->d_gemm_ws);
  if (e->d_row_loss) (void)hipFree(e->d_row_loss);
  if (e->d_sgd_table) (void)hipFree(e->d_sgd_table);
  if (e->h_loss) (void)hipHostFree(e->h_loss);
  if (e->h_flags) (void)hipHostFree(e->h_flags);
  if (e->h_hits) (void)hipHostFree(e->h_hits);
  if (e->h_slots) (void)hipHostFree(e->h_slots);
  if (e->stream) (void)hipStreamDestroy(e->stream);
  delete e;
  return RST_OK;
}

int rst_engine_synchronize(rst_engine* e) {
  RST_TRY(engine_activate(e));
  RST_HIP(hipStreamSynchronize(e->stream));
  return RST_OK;
}

void* rst_engine_stream(rst_engine* e) { return e ? (void*)e->stream : nullptr; }

int rst_engine_device_info(rst_engine* e, char* name, size_t name_capacity, int* compute_units,
                           size_t* total_memory_bytes) {
  if (!e) return fail(RST_ERR_INVALID_ARGUMENT, "engine is null");
  if (name && name_capacity) {
    const char* src = e->props.name[0] ? e->props.name : e->props.gcnArchName;
    snprintf(name, name_capacity, "%s (%s)", src, e->props.gcnArchName);
  }
  if (compute_units) *compute_units = e->props.multiProcessorCount;
  if (total_memory_bytes) *total_memory_bytes = e->props.totalGlobalMem;
  return RST_OK;
}

// Allocation goes through a per-engine cache of freed blocks keyed by size: the layer-by-layer
// API allocates an output array per call (the reference allocates a fresh Array2 per expression
// too), and hipMalloc / hipFree would synchronise the device every time.  A cached block is
// only ever reused by work enqueued later on the engine's single stream, so reuse needs no wait.
int rst_malloc(rst_engine* e, size_t count, double** out) {
  RST_TRY(engine_activate(e));
  if (!out) return fail(RST_ERR_INVALID_ARGUMENT, "out is null");
  *out = nullptr;
  size_t bytes = ((count ? count : 1) * sizeof(double) + 255) / 256 * 256;
  auto it = e->free_blocks.find(bytes);
  if (it != e->free_blocks.end() && !it->second.empty()) {
    *out = static_cast<double*>(it->second.back());
    it->second.pop_back();
    e->cached_bytes -= bytes;
  } else {
    void* p = nullptr;
    hipError_t err = hipMalloc(&p, bytes);
    if (err == hipErrorOutOfMemory && e->cached_bytes) {  // give the cache back and retry
      (void)hipGetLastError();
      RST_TRY(rst_engine_trim(e));
      err = hipMalloc(&p, bytes);
    }
    if (err != hipSuccess) return fail_hip(err, "hipMalloc", __FILE__, __LINE__);
    *out = static_cast<double*>(p);
  }
  e->live_blocks[*out] = bytes;
  return RST_OK;
}

int rst_free(rst_engine* e, double* ptr) {
  if (!e) return fail(RST_ERR_INVALID_ARGUMENT, "engine is null");
  if (!ptr) return RST_OK;
  auto it = e->live_blocks.find(ptr);
  if (it == e->live_blocks.end())
    return fail(RST_ERR_INVALID_ARGUMENT, "rst_free: pointer was not allocated by rst_malloc on this engine");
  const size_t bytes = it->second;
  e->live_blocks.erase(it);
  e->free_blocks[bytes].push_back(ptr);
  e->cached_bytes += bytes;
  return RST_OK;
}

int rst_engine_trim(rst_engine* e) {
  RST_TRY(engine_activate(e));
  RST_HIP(hipStreamSynchronize(e->stream));
  for (auto& kv : e->free_blocks)
    for (void* p : kv.second) RST_HIP(hipFree(p));
  e->free_blocks.clear();
  e->cached_bytes = 0;
  return RST_OK;
}

int rst_upload(rst_engine* e, double* dst, const double* host_src, size_t count) {
  RST_TRY(engine_activate(e));
  if (count == 0) return RST_OK;
  if (!dst || !host_src) return fail(RST_ERR_INVALID_ARGUMENT, "null pointer in upload");
  RST_HIP(hipMemcpyAsync(dst, host_src, count * sizeof(double), hipMemcpyHostToDevice, e->stream));
  RST_HIP(hipStreamSynchronize(e->stream));  // the host buffer may be pageable and reused
  return RST_OK;
}

int rst_download(rst_engine* e, double* host_dst, const double* src, size_t count) {
  RST_TRY(engine_activate(e));
  if (count == 0) return RST_OK;
  if (!host_dst || !src) return fail(RST_ERR_INVALID_ARGUMENT, "null pointer in download");
  RST_HIP(hipMemcpyAsync(host_dst, src, count * sizeof(double), hipMemcpyDeviceToHost, e->stream));
  RST_HIP(hipStreamSynchronize(e->stream));
  return RST_OK;
}

int rst_copy(rst_engine* e, double* dst, const double* src, size_t count) {
  RST_TRY(engine_activate(e));
  if (count == 0) return RST_OK;
  if (!dst || !src) return fail(RST_ERR_INVALID_ARGUMENT, "null pointer in copy");
  RST_HIP(hipMemcpyAsync(dst, src, count * sizeof(double), hipMemcpyDeviceToDevice, e->stream));
  return RST_OK;
}

int rst_fill(rst_engine* e, double* dst, size_t count, double value) {
  RST_TRY(engine_activate(e));
  if (count == 0) return RST_OK;
  if (!dst) return fail(RST_ERR_INVALID_ARGUMENT, "null pointer in fill");
  return launch_fill(e->stream, dst, count, value);
}

}  // extern "C"

// ---- events -------------------------------------------------------------------------------------
struct rst_event {
  rst_engine* engine;
  int device;  // kept here so that destroying the event never reads an engine that is already gone
  hipEvent_t ev;
};

extern "C" {

int rst_event_create(rst_engine* e, rst_event** out) {
  RST_TRY(engine_activate(e));
  if (!out) return fail(RST_ERR_INVALID_ARGUMENT, "out is null");
  *out = nullptr;
  rst_event* ev = new (std::nothrow) rst_event();
  if (!ev) return fail(RST_ERR_OUT_OF_MEMORY, "host allocation failed");
  ev->engine = e;
  ev->device = e->device;
  hipError_t err = hipEventCreate(&ev->ev);
  if (err != hipSuccess) {
    delete ev;
    return fail_hip(err, "hipEventCreate", __FILE__, __LINE__);
  }
  *out = ev;
  return RST_OK;
}

int rst_event_destroy(rst_event* ev) {
  if (!ev) return RST_OK;
  (void)hipSetDevice(ev->device);
  (void)hipEventDestroy(ev->ev);
  delete ev;
  return RST_OK;
}

int rst_event_record(rst_event* ev) {
  if (!ev) return fail(RST_ERR_INVALID_ARGUMENT, "event is null");
  RST_TRY(engine_activate(ev->engine));
  RST_HIP(hipEventRecord(ev->ev, ev->engine->stream));
  return RST_OK;
}

int rst_event_wait(rst_engine* e, rst_event* ev) {
  if (!ev) return fail(RST_ERR_INVALID_ARGUMENT, "event is null");
  RST_TRY(engine_activate(e));
  if (ev->device != e->device) return fail(RST_ERR_INVALID_ARGUMENT, "the event belongs to another GPU");
  RST_HIP(hipStreamWaitEvent(e->stream, ev->ev, 0));
  return RST_OK;
}

int rst_event_elapsed_ms(rst_event* start, rst_event* stop, double* host_ms) {
  if (!start || !stop || !host_ms) return fail(RST_ERR_INVALID_ARGUMENT, "null argument");
  RST_TRY(engine_activate(stop->engine));
  RST_HIP(hipEventSynchronize(stop->ev));
  float ms = 0.f;
  RST_HIP(hipEventElapsedTime(&ms, start->ev, stop->ev));
  *host_ms = (double)ms;
  return RST_OK;
}

}  // extern "C"
