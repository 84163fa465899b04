// A stand-in for the HIP runtime, for ONE purpose: running the HOST side of librstorch_hip (argument
// checking, the arena layout, the state machine of the device model, the step-graph cache, the
// allocation cache, the stager's slot logic) under AddressSanitizer / UBSan on a machine without a
// GPU.  Device memory is host memory, kernels are never executed (a launch is a no-op), graphs only
// count their nodes.  Nothing here computes anything: no numerical result of the library can be
// produced or checked through it, and the product never links it.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <set>

namespace {
std::mutex g_mu;
std::set<void*> g_device, g_host;        // live allocations: a double free or a foreign pointer aborts
std::set<void*> g_events, g_streams, g_graphs, g_execs;
bool g_capturing = false;
int g_captured_nodes = 0;
long g_launches = 0;
long g_malloc_calls = 0, g_free_calls = 0;  // every allocating / releasing call, device and pinned
char g_symbol_storage[1 << 20];

[[noreturn]] void die(const char* what, const void* p) {
  std::fprintf(stderr, "hip_stub: %s (%p)\n", what, p);
  std::abort();
}
void* track(std::set<void*>& s, void* p) { std::lock_guard<std::mutex> l(g_mu); s.insert(p); return p; }
void untrack(std::set<void*>& s, void* p, const char* what) {
  std::lock_guard<std::mutex> l(g_mu);
  if (!s.erase(p)) die(what, p);
}
bool known(std::set<void*>& s, void* p) { std::lock_guard<std::mutex> l(g_mu); return s.count(p) != 0; }
}  // namespace

extern "C" long hip_stub_launch_count() { return g_launches; }
extern "C" long hip_stub_live_device_allocations() { return (long)g_device.size(); }
extern "C" long hip_stub_allocation_calls() { return g_malloc_calls + g_free_calls; }
// lets the driver put the engine's stream into capture mode the way a caller's own code would
extern "C" void hip_stub_begin_capture(void* stream) { (void)hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal); }
extern "C" int hip_stub_end_capture(void* stream) {
  hipGraph_t g = nullptr;
  (void)hipStreamEndCapture((hipStream_t)stream, &g);
  const int nodes = *(int*)g;
  (void)hipGraphDestroy(g);
  return nodes;
}

hipError_t hipGetDeviceCount(int* n) { *n = 1; return hipSuccess; }
hipError_t hipSetDevice(int d) { return d == 0 ? hipSuccess : hipErrorInvalidDevice; }
hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
hipError_t hipGetDevicePropertiesR0600(hipDeviceProp_t* p, int) {
  std::memset(p, 0, sizeof(*p));
  std::strcpy(p->name, "host stub");
  std::strcpy(p->gcnArchName, "none");
  p->multiProcessorCount = 256;
  p->totalGlobalMem = (size_t)1 << 34;
  return hipSuccess;
}
hipError_t hipDeviceGetAttribute(int* v, hipDeviceAttribute_t, int) { *v = 256; return hipSuccess; }
const char* hipGetErrorString(hipError_t) { return "stub error"; }
hipError_t hipGetLastError() { return hipSuccess; }

hipError_t hipMalloc(void** p, size_t bytes) {
  if (g_capturing) die("hipMalloc while the stream is capturing", nullptr);
  ++g_malloc_calls;
  *p = track(g_device, std::malloc(bytes ? bytes : 1));
  return hipSuccess;
}
hipError_t hipFree(void* p) {
  if (!p) return hipSuccess;
  if (g_capturing) die("hipFree while the stream is capturing", p);
  ++g_free_calls;
  untrack(g_device, p, "hipFree of a pointer that is not a live device allocation");
  std::free(p);
  return hipSuccess;
}
hipError_t hipHostMalloc(void** p, size_t bytes, unsigned) { ++g_malloc_calls; *p = track(g_host, std::calloc(1, bytes ? bytes : 1)); return hipSuccess; }
hipError_t hipHostFree(void* p) {
  if (!p) return hipSuccess;
  ++g_free_calls;
  untrack(g_host, p, "hipHostFree of a pointer that is not a live pinned allocation");
  std::free(p);
  return hipSuccess;
}
hipError_t hipHostGetDevicePointer(void** d, void* h, unsigned) { *d = h; return hipSuccess; }
hipError_t hipMemsetAsync(void* p, int v, size_t n, hipStream_t) {
  if (g_capturing) die("hipMemsetAsync recorded into a graph", p);
  std::memset(p, v, n);
  return hipSuccess;
}
hipError_t hipMemcpyAsync(void* d, const void* s, size_t n, hipMemcpyKind, hipStream_t) {
  if (g_capturing) { ++g_captured_nodes; return hipSuccess; }
  std::memmove(d, s, n);  // under ASan this checks both ranges
  return hipSuccess;
}
hipError_t hipMemcpy(void* d, const void* s, size_t n, hipMemcpyKind) { std::memmove(d, s, n); return hipSuccess; }
hipError_t hipGetSymbolAddress(void** p, const void*) { *p = g_symbol_storage; return hipSuccess; }

hipError_t hipStreamCreateWithFlags(hipStream_t* s, unsigned) { *s = (hipStream_t)track(g_streams, std::malloc(8)); return hipSuccess; }
hipError_t hipStreamDestroy(hipStream_t s) { untrack(g_streams, s, "hipStreamDestroy of an unknown stream"); std::free(s); return hipSuccess; }
hipError_t hipStreamSynchronize(hipStream_t s) {
  if (s && !known(g_streams, s)) die("hipStreamSynchronize on a destroyed stream", s);
  if (g_capturing) die("hipStreamSynchronize while the stream is capturing", s);
  return hipSuccess;
}
hipError_t hipStreamWaitEvent(hipStream_t, hipEvent_t e, unsigned) {
  if (!known(g_events, e)) die("hipStreamWaitEvent on a destroyed event", e);
  return hipSuccess;
}
hipError_t hipEventCreate(hipEvent_t* e) { *e = (hipEvent_t)track(g_events, std::malloc(8)); return hipSuccess; }
hipError_t hipEventCreateWithFlags(hipEvent_t* e, unsigned) { return hipEventCreate(e); }
hipError_t hipEventDestroy(hipEvent_t e) { untrack(g_events, e, "hipEventDestroy of an unknown event"); std::free(e); return hipSuccess; }
hipError_t hipEventRecord(hipEvent_t e, hipStream_t) {
  if (!known(g_events, e)) die("hipEventRecord on a destroyed event", e);
  return hipSuccess;
}
hipError_t hipEventSynchronize(hipEvent_t e) {
  if (!known(g_events, e)) die("hipEventSynchronize on a destroyed event", e);
  return hipSuccess;
}
hipError_t hipEventElapsedTime(float* ms, hipEvent_t a, hipEvent_t b) {
  if (!known(g_events, a) || !known(g_events, b)) die("hipEventElapsedTime on a destroyed event", a);
  *ms = 0.001f;
  return hipSuccess;
}

hipError_t hipStreamBeginCapture(hipStream_t, hipStreamCaptureMode) {
  if (g_capturing) die("nested capture", nullptr);
  g_capturing = true;
  g_captured_nodes = 0;
  return hipSuccess;
}
hipError_t hipStreamIsCapturing(hipStream_t, hipStreamCaptureStatus* status) {
  *status = g_capturing ? hipStreamCaptureStatusActive : hipStreamCaptureStatusNone;
  return hipSuccess;
}
hipError_t hipStreamEndCapture(hipStream_t, hipGraph_t* g) {
  if (!g_capturing) die("hipStreamEndCapture without a capture", nullptr);
  g_capturing = false;
  int* node_count = (int*)std::malloc(sizeof(int));
  *node_count = g_captured_nodes;
  *g = (hipGraph_t)track(g_graphs, node_count);
  return hipSuccess;
}
hipError_t hipGraphInstantiate(hipGraphExec_t* x, hipGraph_t g, hipGraphNode_t*, char*, size_t) {
  if (!known(g_graphs, g)) die("hipGraphInstantiate of a destroyed graph", g);
  int* node_count = (int*)std::malloc(sizeof(int));
  *node_count = *(int*)g;
  *x = (hipGraphExec_t)track(g_execs, node_count);
  return hipSuccess;
}
hipError_t hipGraphDestroy(hipGraph_t g) { untrack(g_graphs, g, "hipGraphDestroy of an unknown graph"); std::free(g); return hipSuccess; }
hipError_t hipGraphExecDestroy(hipGraphExec_t x) { untrack(g_execs, x, "hipGraphExecDestroy of an unknown executable"); std::free(x); return hipSuccess; }
hipError_t hipGraphLaunch(hipGraphExec_t x, hipStream_t) {
  if (!known(g_execs, x)) die("hipGraphLaunch of a destroyed executable", x);
  g_launches += *(int*)x;
  return hipSuccess;
}

// kernel launches: hipLaunchKernelGGL expands to the <<<>>> form, i.e. a push/pop of the launch
// configuration around the host-side kernel stub, which calls hipLaunchKernel
namespace { thread_local struct { dim3 g, b; size_t shmem; hipStream_t s; } g_cfg; }
extern "C" hipError_t __hipPushCallConfiguration(dim3 g, dim3 b, size_t shmem, hipStream_t s) {
  g_cfg = {g, b, shmem, s};
  return hipSuccess;
}
extern "C" hipError_t __hipPopCallConfiguration(dim3* g, dim3* b, size_t* shmem, hipStream_t* s) {
  *g = g_cfg.g; *b = g_cfg.b; *shmem = g_cfg.shmem; *s = g_cfg.s;
  return hipSuccess;
}
hipError_t hipLaunchKernel(const void*, dim3 g, dim3 b, void**, size_t, hipStream_t) {
  if (g.x == 0 || g.y == 0 || g.z == 0 || b.x == 0 || b.x * b.y * b.z > 1024) die("launch with an empty or oversized grid/block", nullptr);
  if (g_capturing) ++g_captured_nodes; else ++g_launches;
  return hipSuccess;
}
extern "C" void** __hipRegisterFatBinary(const void*) { static void* h; return &h; }
extern "C" void __hipUnregisterFatBinary(void**) {}
extern "C" void __hipRegisterFunction(void**, const void*, char*, const char*, unsigned, void*, void*, void*, void*, int*) {}
extern "C" void __hipRegisterVar(void**, void*, char*, const char*, int, size_t, int, int) {}
