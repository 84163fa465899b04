// The single-call training step (rst_model_train_step) on FRESH inputs every step, driven from C++
// so that the host side costs what a compiled caller's would: two resident batches; while the
// training engine works on one, a second engine (a second stream of the same GPU) refills the other
// from the counter generator, generator stream number = step; events hand the buffers back and forth.
//
//   train_loop CONFIG STEPS WARMUP [loss] [one-stream]
// CONFIG: C0 (README network, batch 32, U[0,1) inputs) or C1 (the same at batch 8192).  "loss": the
// scalar loss of every step is read back (the one round trip the reference's loop makes).
// "one-stream": no second engine; the generator runs on the training stream ahead of every step, so
// its time is inside the step instead of hidden behind the previous one.
// Prints one line: steps/s, ms per step and the last loss.
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../include/rstorch_hip.h"

#define CHECK(expr)                                                                      \
  do {                                                                                   \
    int st_ = (expr);                                                                    \
    if (st_ != RST_OK) {                                                                 \
      std::fprintf(stderr, "%s -> %s: %s\n", #expr, rst_status_string(st_), rst_last_error()); \
      std::exit(1);                                                                      \
    }                                                                                    \
  } while (0)

int main(int argc, char** argv) {
  const char* config = argc > 1 ? argv[1] : "C0";
  const long steps = argc > 2 ? std::atol(argv[2]) : 2000;
  const long warmup = argc > 3 ? std::atol(argv[3]) : 100;
  bool read_loss = false, one_stream = false;
  for (int a = 4; a < argc; ++a) {
    if (!std::strcmp(argv[a], "loss")) read_loss = true;
    if (!std::strcmp(argv[a], "one-stream")) one_stream = true;
  }
  const size_t batch = !std::strcmp(config, "C1") ? 8192 : 32;
  const size_t n_in = 784, n_out = 10;
  const double lr = 0.01;
  const uint64_t seed = 0x5EED;

  rst_engine *eng = nullptr, *loader = nullptr;
  CHECK(rst_engine_create(0, &eng));
  CHECK(rst_engine_create(0, &loader));
  const int kinds[] = {RST_LAYER_IDENTITY, RST_LAYER_LINEAR, RST_LAYER_RELU, RST_LAYER_LINEAR, RST_LAYER_RELU, RST_LAYER_LINEAR};
  const size_t ins[] = {0, 784, 0, 100, 0, 100}, outs[] = {0, 100, 0, 100, 0, 10};
  rst_model* model = nullptr;
  CHECK(rst_model_create(eng, kinds, ins, outs, 6, &model));
  CHECK(rst_model_init_kaiming(model, seed, 0));
  double *x[2], *y[2];
  rst_event *filled[2], *used[2];
  for (int s = 0; s < 2; ++s) {
    CHECK(rst_malloc(eng, batch * n_in, &x[s]));
    CHECK(rst_malloc(eng, batch * n_out, &y[s]));
    CHECK(rst_event_create(loader, &filled[s]));
    CHECK(rst_event_create(eng, &used[s]));
  }
  auto refill = [&](int slot, long step) {
    CHECK(rst_fill_uniform(loader, x[slot], batch * n_in, seed, 1000 + 2 * step, 0.0, 1.0));
    CHECK(rst_fill_one_hot(loader, y[slot], batch, n_out, seed, 1001 + 2 * step));
    CHECK(rst_event_record(filled[slot]));
  };
  double loss = 0.0;
  auto run = [&](long first, long count) {
    if (one_stream) {
      for (long k = first; k < first + count; ++k) {
        CHECK(rst_fill_uniform(eng, x[0], batch * n_in, seed, 1000 + 2 * k, 0.0, 1.0));
        CHECK(rst_fill_one_hot(eng, y[0], batch, n_out, seed, 1001 + 2 * k));
        CHECK(rst_model_train_step(model, x[0], y[0], batch, lr, read_loss ? &loss : nullptr));
      }
      CHECK(rst_engine_synchronize(eng));
      return;
    }
    refill((int)(first % 2), first);
    for (long k = first; k < first + count; ++k) {
      const int slot = (int)(k % 2);
      if (k + 1 < first + count) {
        if (k >= first + 1) CHECK(rst_event_wait(loader, used[1 - slot]));  // the step that last read the other buffer
        refill(1 - slot, k + 1);
      }
      CHECK(rst_event_wait(eng, filled[slot]));
      CHECK(rst_model_train_step(model, x[slot], y[slot], batch, lr, read_loss ? &loss : nullptr));
      CHECK(rst_event_record(used[slot]));
    }
    CHECK(rst_engine_synchronize(eng));
    CHECK(rst_engine_synchronize(loader));
  };
  run(0, warmup);
  const auto t0 = std::chrono::steady_clock::now();
  run(warmup, steps);
  const double secs = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
  CHECK(rst_loss_value(eng, &loss));
  std::printf("%s batch %zu: %.1f steps/s, %.5f ms/step, last loss %.12f%s\n", config, batch, steps / secs,
              secs * 1e3 / steps, loss, read_loss ? " (loss read every step)" : "");
  if (one_stream) std::printf("  (generator on the training stream)\n");
  for (int s = 0; s < 2; ++s) {
    rst_event_destroy(filled[s]);
    rst_event_destroy(used[s]);
  }
  rst_model_destroy(model);
  rst_engine_destroy(loader);
  rst_engine_destroy(eng);
  return 0;
}
