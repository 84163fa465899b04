// Drives the C ABI of librstorch_hip, built for the host only against hip_stub.cpp, through the
// call sequences of the benchmark and of the tests - under AddressSanitizer and UBSan.  Kernels do
// not run, so only host-side behaviour is checked: status codes, state machine, shapes that the
// planners must accept, allocation and graph lifetimes (the stand-in aborts on a double free, on a
// launch of a destroyed graph, on an allocation or a synchronisation during stream capture).
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/rstorch_hip.h"

extern "C" long hip_stub_launch_count();
extern "C" long hip_stub_live_device_allocations();
extern "C" long hip_stub_allocation_calls();
extern "C" void hip_stub_begin_capture(void* stream);
extern "C" int hip_stub_end_capture(void* stream);

#define OK(expr)                                                                              \
  do {                                                                                        \
    int st_ = (expr);                                                                         \
    if (st_ != RST_OK) {                                                                      \
      std::fprintf(stderr, "%s:%d: %s -> %d (%s)\n", __FILE__, __LINE__, #expr, st_, rst_last_error()); \
      std::exit(1);                                                                           \
    }                                                                                         \
  } while (0)
#define EXPECT(expr, want)                                                                    \
  do {                                                                                        \
    int st_ = (expr);                                                                         \
    if (st_ != (want)) {                                                                      \
      std::fprintf(stderr, "%s:%d: %s -> %d, expected %d\n", __FILE__, __LINE__, #expr, st_, (int)(want)); \
      std::exit(1);                                                                           \
    }                                                                                         \
  } while (0)

struct Spec {
  std::vector<int> kinds;
  std::vector<size_t> in, out;
  void linear(size_t i, size_t o) { kinds.push_back(RST_LAYER_LINEAR); in.push_back(i); out.push_back(o); }
  void relu() { kinds.push_back(RST_LAYER_RELU); in.push_back(0); out.push_back(0); }
  void identity() { kinds.push_back(RST_LAYER_IDENTITY); in.push_back(0); out.push_back(0); }
};

static rst_model* build(rst_engine* e, const Spec& s) {
  rst_model* m = nullptr;
  OK(rst_model_create(e, s.kinds.data(), s.in.data(), s.out.data(), s.kinds.size(), &m));
  OK(rst_model_graph_enable(m, 1));  // whatever its depth: the graph lifetimes are what is checked here
  return m;
}

static double* dev(rst_engine* e, size_t n) {
  double* p = nullptr;
  OK(rst_malloc(e, n, &p));
  return p;
}

// warm-up steps (recorded and replayed as a graph), steps with per-launch events, the records read
static void timed_steps(rst_engine* e, rst_model* m, const double* x, const double* t, size_t batch, int steps) {
  for (int i = 0; i < 3; ++i) OK(rst_model_train_step(m, x, t, batch, 0.01, nullptr));
  OK(rst_engine_synchronize(e));
  OK(rst_model_profile_enable(m, 1));
  for (int i = 0; i < steps; ++i) OK(rst_model_train_step(m, x, t, batch, 0.01, nullptr));
  size_t n = 0;
  OK(rst_model_profile_read(m, nullptr, 0, &n));
  OK(rst_model_profile_enable(m, 0));
  double loss = 0.0;
  OK(rst_loss_value(e, &loss));
}

int main() {
  rst_engine* e = nullptr;
  OK(rst_engine_create(0, &e));
  EXPECT(rst_engine_create(0, nullptr), RST_ERR_INVALID_ARGUMENT);
  {
    rst_engine* none = nullptr;
    EXPECT(rst_engine_create(3, &none), RST_ERR_INVALID_ARGUMENT);  // one device in the stand-in
  }

  // ---- the benchmark's sequence, at its real shapes (memory is reserved, never touched) -----------
  Spec c4;
  for (int i = 0; i < 8; ++i) { c4.linear(4096, 4096); c4.relu(); }
  c4.linear(4096, 32768);
  {
    rst_model* m = build(e, c4);
    OK(rst_model_init_kaiming(m, 0x5EED, 0));
    double* x = dev(e, (size_t)1024 * 4096);
    double* t = dev(e, (size_t)1024 * 32768);
    timed_steps(e, m, x, t, 1024, 4);
    // a smaller and a larger batch on the same model: activations are reserved again, graphs dropped
    OK(rst_model_train_step(m, x, t, 512, 0.01, nullptr));
    OK(rst_model_train_step(m, x, t, 1024, 0.01, nullptr));
    OK(rst_model_destroy(m));
    OK(rst_free(e, x));
    OK(rst_free(e, t));
  }
  {  // SGD alone over 128 tensors, list and arena forms
    const size_t total = 64 * ((size_t)2048 * 2048 + 2048);
    double* p = dev(e, total);
    double* g = dev(e, total);
    std::vector<double*> pp;
    std::vector<const double*> gp;
    std::vector<size_t> cnt;
    size_t off = 0;
    for (int i = 0; i < 64; ++i) {
      pp.push_back(p + off); gp.push_back(g + off); cnt.push_back((size_t)2048 * 2048); off += cnt.back();
      pp.push_back(p + off); gp.push_back(g + off); cnt.push_back(2048); off += cnt.back();
    }
    for (int i = 0; i < 3; ++i) OK(rst_sgd_step(e, pp.data(), gp.data(), cnt.data(), cnt.size(), 0.01));
    OK(rst_sgd_step_flat(e, p, g, total, 0.01));
    OK(rst_free(e, p));
    OK(rst_free(e, g));
  }
  Spec readme;
  readme.identity(); readme.linear(784, 100); readme.relu(); readme.linear(100, 100); readme.relu(); readme.linear(100, 10);
  Spec c2;
  c2.linear(1024, 4096); c2.relu(); c2.linear(4096, 4096); c2.relu(); c2.linear(4096, 1000);
  struct { const Spec* s; size_t batch, in, out; } small[] = {{&readme, 32, 784, 10}, {&readme, 8192, 784, 10}, {&c2, 2048, 1024, 1000}};
  for (auto& c : small) {  // a freshly built model right after the big one went away
    rst_model* m = build(e, *c.s);
    double* x = dev(e, c.batch * c.in);
    double* t = dev(e, c.batch * c.out);
    timed_steps(e, m, x, t, c.batch, 5);
    OK(rst_model_destroy(m));
    OK(rst_free(e, x));
    OK(rst_free(e, t));
  }

  // ---- the README loop's calls: forward, loss + accuracy with the upper layers' input gradients launched
  //      ahead of the wait, backward with the update; and every way of not following that up -----------------
  for (size_t batch : {(size_t)32, (size_t)8192}) {
    rst_model* m = build(e, readme);
    double* x = dev(e, batch * 784);
    double* t = dev(e, batch * 10);
    double* logits = dev(e, batch * 10);
    double* g = dev(e, batch * 10);
    double* g2 = dev(e, batch * 10);
    double* gin = dev(e, batch * 784);
    double loss = 0.0, acc = 0.0;
    EXPECT(rst_model_loss_accuracy_to(m, logits, t, g, 1, &loss, &acc), RST_ERR_STATE);  // no forward pass yet
    for (int step = 0; step < 6; ++step) {
      OK(rst_model_forward_to(m, x, batch, logits));
      if (step == 0) EXPECT(rst_model_loss_accuracy_to(m, g2, t, g, 1, &loss, &acc), RST_ERR_STATE);  // not its logits
      if (step == 0) EXPECT(rst_model_loss_accuracy_to(m, logits, t, g, 1, nullptr, &acc), RST_ERR_INVALID_ARGUMENT);
      OK(rst_model_loss_accuracy_to(m, logits, t, g, step != 1, &loss, step == 2 ? nullptr : &acc));
      if (step == 3) OK(rst_model_discard_inputs(m));
      if (step == 4) OK(rst_model_loss_accuracy_to(m, logits, t, g2, 1, &loss, &acc));  // the loss taken twice
      OK(rst_model_backward_to(m, step == 4 ? g2 : step == 5 ? g2 : g, step % 2 ? gin : nullptr, 1, 0.01));
      EXPECT(rst_model_backward_to(m, g, nullptr, 1, 0.01), RST_ERR_STATE);  // the caches are consumed
    }
    OK(rst_model_forward_to(m, x, batch, logits));  // a forward pass that nothing follows
    OK(rst_model_loss_accuracy_to(m, logits, t, g, 1, &loss, &acc));
    OK(rst_model_forward_to(m, x, batch, logits));
    OK(rst_model_backward_to(m, g, nullptr, 0, 0.0));  // (the same address, after another forward: all of it runs)
    OK(rst_model_destroy(m));
    for (double* p : {x, t, logits, g, g2, gin}) OK(rst_free(e, p));
  }

  // ---- two models and an operator-level cross entropy sharing one engine -------------------------
  {
    rst_model* a = build(e, readme);
    rst_model* b = build(e, readme);
    double* x = dev(e, (size_t)8192 * 784);
    double* t = dev(e, (size_t)8192 * 10);
    double* g = dev(e, (size_t)8192 * 10);
    for (int round = 0; round < 3; ++round) {
      OK(rst_model_train_step(a, x, t, 256, 0.01, nullptr));
      OK(rst_cross_entropy(e, x, t, g, nullptr, 4096 + 1024 * round, 10, nullptr));
      OK(rst_model_train_step(b, x, t, 8192, 0.01, nullptr));
      OK(rst_model_train_step(a, x, t, 256, 0.01, nullptr));
      OK(rst_cross_entropy_static(e, x, t, g, 4096, 10, nullptr));
    }
    EXPECT(rst_cross_entropy_static(e, x, t, g, RST_STATIC_CROSS_ENTROPY_MAX_ROWS + 1, 2, nullptr), RST_ERR_UNSUPPORTED);
    {  // loss and accuracy after one wait: a batch for one workgroup, a long one, a wide one
      double loss = 0.0, acc = 0.0;
      OK(rst_cross_entropy_accuracy(e, x, t, g, 32, 10, &loss, &acc));
      OK(rst_cross_entropy_accuracy(e, x, t, g, 8192, 10, &loss, &acc));
      OK(rst_cross_entropy_accuracy(e, x, t, g, 2, 40000, &loss, &acc));
      EXPECT(rst_cross_entropy_accuracy(e, x, t, g, 2, 4, &loss, nullptr), RST_ERR_INVALID_ARGUMENT);
    }
    {
      // the entry point that allocates nothing: no allocating or releasing runtime call, device or
      // pinned, on a first use at a new size, on the largest batch it takes, or under stream capture
      // (where the stand-in aborts on an allocation or a synchronisation anyway)
      const long before = hip_stub_allocation_calls();
      double loss = 0.0;
      OK(rst_cross_entropy_static(e, x, t, g, 8192, 10, &loss));
      OK(rst_cross_entropy_static(e, x, t, g, 37, 1000, nullptr));
      OK(rst_cross_entropy_static(e, x, t, g, 1, 40000, nullptr));
      double* big = reinterpret_cast<double*>(x);  // 65536 x 2 doubles fit in the 8192 x 784 buffer
      OK(rst_cross_entropy_static(e, big, big, big, RST_STATIC_CROSS_ENTROPY_MAX_ROWS, 2, nullptr));
      hip_stub_begin_capture(rst_engine_stream(e));
      OK(rst_cross_entropy_static(e, x, t, g, 4096, 10, nullptr));
      const int nodes = hip_stub_end_capture(rst_engine_stream(e));
      if (nodes < 1) { std::fprintf(stderr, "the captured call recorded no kernel\n"); return 1; }
      if (hip_stub_allocation_calls() != before) {
        std::fprintf(stderr, "rst_cross_entropy_static allocated or freed: %ld runtime calls\n",
                     hip_stub_allocation_calls() - before);
        return 1;
      }
      // a second engine on the same GPU does not disturb the scratch (set-up runs once per device)
      const long launches_before = hip_stub_launch_count();
      rst_engine* second = nullptr;
      OK(rst_engine_create(0, &second));
      if (hip_stub_launch_count() != launches_before) { std::fprintf(stderr, "engine creation launched a kernel\n"); return 1; }
      OK(rst_engine_destroy(second));
    }
    // more distinct (x, truth, batch, lr) than the graph cache holds: the oldest executables go
    for (int k = 0; k < 20; ++k) OK(rst_model_train_step(a, x + 784 * (k % 11), t, 64, 0.01 + 0.001 * (k % 3), nullptr));
    OK(rst_model_fuse_sgd(a, 0));
    OK(rst_model_pair_gradients(a, 1));
    OK(rst_model_graph_enable(a, 0));
    OK(rst_model_train_step(a, x, t, 64, 0.01, nullptr));
    OK(rst_model_graph_enable(a, 1));
    OK(rst_model_train_step(a, x, t, 64, 0.01, nullptr));
    OK(rst_model_destroy(a));
    OK(rst_model_destroy(b));
    OK(rst_free(e, x)); OK(rst_free(e, t)); OK(rst_free(e, g));
  }

  // ---- the state machine of the layer-by-layer calls (Option::take() in the reference) -----------
  {
    rst_model* m = build(e, readme);
    double* x = dev(e, 32 * 784);
    double* t = dev(e, 32 * 10);
    const double* logits = nullptr;
    const double* gin = nullptr;
    double loss = 0.0;
    EXPECT(rst_model_backward(m, nullptr, 1, &gin), RST_ERR_STATE);   // backward before forward
    EXPECT(rst_model_loss(m, t, &loss), RST_ERR_STATE);
    EXPECT(rst_model_sgd_step(m, 0.1), RST_ERR_STATE);                // step before any backward
    OK(rst_model_forward(m, x, 32, &logits));
    EXPECT(rst_model_backward(m, nullptr, 1, &gin), RST_ERR_STATE);   // loss.backward() before loss.forward()
    OK(rst_model_loss(m, t, nullptr));
    OK(rst_model_backward(m, nullptr, 1, &gin));
    EXPECT(rst_model_backward(m, nullptr, 1, &gin), RST_ERR_STATE);   // the caches are consumed
    OK(rst_model_sgd_step(m, 0.1));
    EXPECT(rst_model_train_step(m, x, t, 0, 0.1, nullptr), RST_ERR_SHAPE);
    EXPECT(rst_model_train_step(m, nullptr, t, 4, 0.1, nullptr), RST_ERR_INVALID_ARGUMENT);
    size_t tensors = 0, elements = 0;
    OK(rst_model_parameter_count(m, &tensors, &elements));
    if (tensors != 6 || elements != 89610) { std::fprintf(stderr, "parameter count %zu / %zu\n", tensors, elements); return 1; }
    std::vector<double> flat(elements, 0.5);
    OK(rst_model_import_parameters(m, flat.data(), flat.size()));
    OK(rst_model_export_parameters(m, flat.data(), flat.size()));
    EXPECT(rst_model_export_parameters(m, flat.data(), flat.size() - 1), RST_ERR_SHAPE);
    double *p = nullptr, *g = nullptr;
    size_t r = 0, c = 0;
    OK(rst_model_parameter(m, 5, &p, &g, &r, &c));
    if (r != 1 || c != 10) return 1;
    EXPECT(rst_model_parameter(m, 6, &p, &g, &r, &c), RST_ERR_INVALID_ARGUMENT);
    OK(rst_model_destroy(m));
    OK(rst_free(e, x)); OK(rst_free(e, t));
    Spec bad;
    bad.linear(4, 5); bad.linear(6, 2);
    rst_model* none = nullptr;
    EXPECT(rst_model_create(e, bad.kinds.data(), bad.in.data(), bad.out.data(), 2, &none), RST_ERR_SHAPE);
    Spec empty;
    empty.relu();
    EXPECT(rst_model_create(e, empty.kinds.data(), empty.in.data(), empty.out.data(), 1, &none), RST_ERR_UNSUPPORTED);
  }

  // ---- operator level: every tile route of the contraction planner, odd and aligned shapes -------
  {
    const size_t shapes[][3] = {{1, 1, 1}, {32, 784, 100}, {8192, 784, 100}, {8192, 100, 10}, {2050, 2046, 2048},
                                {512, 2048, 4096}, {2048, 24576, 2046}, {24576, 2048, 2046}, {37, 101, 13},
                                {16384, 33, 65}, {4100, 7, 9}, {1024, 4096, 32768}};
    for (auto& s : shapes) {
      const size_t b = s[0], k = s[1], n = s[2];
      double *x = dev(e, b * k), *w = dev(e, n * k), *bias = dev(e, n), *out = dev(e, b * n);
      double *gw = dev(e, n * k), *gb = dev(e, n), *gx = dev(e, b * k);
      OK(rst_linear_forward(e, x, w, bias, out, b, k, n, 1));
      OK(rst_linear_forward(e, x, w, nullptr, out, b, k, n, 0));
      OK(rst_linear_backward(e, out, x, w, gw, gb, gx, x, b, k, n));
      OK(rst_linear_backward(e, out, x, w, gw, nullptr, nullptr, nullptr, b, k, n));
      OK(rst_softmax_backward(e, out, out, out, b < 64 ? b : 64, n < 512 ? n : 512));
      double* ptrs[] = {x, w, bias, out, gw, gb, gx};
      for (double* q : ptrs) OK(rst_free(e, q));
    }
    EXPECT(rst_linear_forward(e, nullptr, nullptr, nullptr, nullptr, 4, 4, 4, 0), RST_ERR_INVALID_ARGUMENT);
    OK(rst_engine_trim(e));
    double* foreign = reinterpret_cast<double*>(0x1000);
    EXPECT(rst_free(e, foreign), RST_ERR_INVALID_ARGUMENT);
  }

  // ---- stager: slot accounting -------------------------------------------------------------------
  {
    rst_stager* st = nullptr;
    OK(rst_stager_create(e, 16, 5, 4, 2, &st));
    std::vector<double> hx(16 * 5, 1.0), ht(16 * 4, 0.0);
    std::vector<uint32_t> hl(16, 1);
    const double *x = nullptr, *t = nullptr;
    size_t rows = 0;
    EXPECT(rst_stager_next(st, &x, &t, &rows), RST_ERR_STATE);           // nothing submitted
    OK(rst_stager_submit_labels(st, hx.data(), hl.data(), 16));
    OK(rst_stager_submit_dense(st, hx.data(), ht.data(), 7));
    EXPECT(rst_stager_submit_labels(st, hx.data(), hl.data(), 16), RST_ERR_STATE);  // both slots taken
    EXPECT(rst_stager_submit_labels(st, hx.data(), hl.data(), 17), RST_ERR_SHAPE);
    OK(rst_stager_next(st, &x, &t, &rows));
    if (rows != 16) return 1;
    double* px = nullptr;
    uint32_t* pl = nullptr;
    OK(rst_stager_acquire_host(st, &px, &pl));
    std::memset(px, 0, 16 * 5 * sizeof(double));                         // the whole slot is writable
    std::memset(pl, 0, 16 * sizeof(uint32_t));
    OK(rst_stager_commit_labels(st, 3));
    OK(rst_stager_next(st, &x, &t, &rows));
    OK(rst_stager_next(st, &x, &t, &rows));
    if (rows != 3) return 1;
    OK(rst_stager_destroy(st));
  }

  // ---- events and teardown -------------------------------------------------------------------------
  rst_event *a = nullptr, *b = nullptr;
  OK(rst_event_create(e, &a));
  OK(rst_event_create(e, &b));
  OK(rst_event_record(a));
  OK(rst_event_record(b));
  double ms = 0.0;
  OK(rst_event_elapsed_ms(a, b, &ms));
  OK(rst_event_wait(e, a));
  EXPECT(rst_event_wait(e, nullptr), RST_ERR_INVALID_ARGUMENT);
  OK(rst_event_destroy(a));
  OK(rst_event_destroy(b));
  const long launches = hip_stub_launch_count();
  OK(rst_engine_destroy(e));
  if (hip_stub_live_device_allocations() != 0) {
    std::fprintf(stderr, "%ld device allocations leaked\n", hip_stub_live_device_allocations());
    return 1;
  }
  std::printf("host logic ok: %ld kernel launches planned\n", launches);
  return 0;
}
