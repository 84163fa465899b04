// The reference's README training loop (README.md:48-81) on the HIP backend, unchanged in shape:
//   model.forward(x) -> loss.forward(pred.clone(), y.clone()) -> accuracy(pred, y)
//   -> model.backward(loss.backward()) -> optim.step(model)
// MNIST needs the network, so batches are synthetic: a small fixed pool, so the loss can go down.
//
//   readme_loop [EPOCHS [STEPS [CONFIG [layers]]]]
// CONFIG: C0 (default; the README network at batch 32, U[0,1) inputs), C1 (the same at batch 8192),
// C2 (1024-4096-4096-1000 at batch 2048, N(0,1) inputs), C4 (8 x 4096 + a 32768-wide head at batch
// 1024).  A fifth argument "layers" runs the Sequential layer by layer (one call per layer) instead
// of in its compiled form.
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "rstorch.hpp"

using namespace rstorch;
using rstorch::utils::accuracy;

int main(int argc, char** argv) {
  const size_t EPOCHS = argc > 1 ? std::strtoul(argv[1], nullptr, 10) : 2;
  const size_t STEPS = argc > 2 ? std::strtoul(argv[2], nullptr, 10) : 1875;
  const char* config = argc > 3 ? argv[3] : "C0";
  const bool layer_by_layer = argc > 4 && std::strcmp(argv[4], "layers") == 0;
  try {
    Sequential model;
    size_t BATCH_SIZE = 32, in = 784, out = 10, POOL = 16;
    bool normal_inputs = false;
    if (!std::strcmp(config, "C0") || !std::strcmp(config, "C1")) {
      model = sequential(Identity(), Linear(784, 100), ReLU(), Linear(100, 100), ReLU(), Linear(100, 10));
      if (config[1] == '1') { BATCH_SIZE = 8192; POOL = 4; }
    } else if (!std::strcmp(config, "C2")) {
      model = sequential(Linear(1024, 4096), ReLU(), Linear(4096, 4096), ReLU(), Linear(4096, 1000));
      BATCH_SIZE = 2048; in = 1024; out = 1000; POOL = 4; normal_inputs = true;
    } else if (!std::strcmp(config, "C4")) {
      for (int i = 0; i < 8; ++i) { model.push(Linear(4096, 4096)); model.push(ReLU()); }
      model.push(Linear(4096, 32768));
      BATCH_SIZE = 1024; in = 4096; out = 32768; POOL = 2; normal_inputs = true;
    } else {
      std::fprintf(stderr, "unknown configuration %s\n", config);
      return 2;
    }
    if (layer_by_layer) model.set_compile(false);
    CrossEntropyLoss loss;
    SGD optim(0.01);
    std::vector<Array2> xs, ys;
    for (size_t i = 0; i < POOL; ++i) {
      xs.push_back(normal_inputs ? Array2::normal(BATCH_SIZE, in, 42, 2 * i, 0.0, 1.0) : Array2::uniform(BATCH_SIZE, in, 42, 2 * i));
      ys.push_back(Array2::one_hot(BATCH_SIZE, out, 42, 2 * i + 1));
    }
    for (size_t i = 0; i < EPOCHS; ++i) {
      const double n = double(STEPS);
      double total_loss = 0.0, total_acc = 0.0;
      auto t0 = std::chrono::steady_clock::now();
      for (size_t s = 0; s < STEPS; ++s) {
        Array2 x = xs[s % POOL], y = ys[s % POOL];
        Array2 pred = model.forward(x);
        double l = loss.forward(pred.clone(), y.clone());
        double acc = accuracy(pred, y);
        total_loss += l;
        total_acc += acc;
        model.backward(loss.backward());
        optim.step(model);
      }
      Engine::global()->synchronize();
      double secs = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
      std::printf("EPOCH %zu: Avarage loss %.6f - Avarage accuracy %.4f  (%.1f steps/s)\n", i,
                  total_loss / n, total_acc / n, n / secs);
    }
    if (out <= 1000) std::printf("%s\n", model.debug().c_str());
  } catch (const Panic& p) {
    std::fprintf(stderr, "panic: %s\n", p.what());
    return 1;
  }
  return 0;
}
