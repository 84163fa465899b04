// The reference's README training loop (README.md:48-81) on the HIP backend, unchanged in shape:
//   model.forward(x) -> loss.forward(pred.clone(), y.clone()) -> accuracy(pred, y)
//   -> model.backward(loss.backward()) -> optim.step(model)
// MNIST needs the network, so batches are synthetic: U[0,1) inputs, uniform one-hot labels.
#include <chrono>
#include <cstdio>
#include <cstdlib>

#include "rstorch.hpp"

using namespace rstorch;
using rstorch::utils::accuracy;

int main(int argc, char** argv) {
  const size_t BATCH_SIZE = 32;
  const size_t EPOCHS = argc > 1 ? std::strtoul(argv[1], nullptr, 10) : 2;
  const size_t STEPS = argc > 2 ? std::strtoul(argv[2], nullptr, 10) : 1875;
  try {
    Sequential model = sequential(Identity(), Linear(784, 100), ReLU(), Linear(100, 100), ReLU(),
                                  Linear(100, 10));
    CrossEntropyLoss loss;
    SGD optim(0.01);
    // a small fixed pool of batches, so the loss can actually go down
    const size_t POOL = 16;
    std::vector<Array2> xs, ys;
    for (size_t i = 0; i < POOL; ++i) {
      xs.push_back(Array2::uniform(BATCH_SIZE, 784, 42, 2 * i));
      ys.push_back(Array2::one_hot(BATCH_SIZE, 10, 42, 2 * i + 1));
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
      double secs = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
      std::printf("EPOCH %zu: Avarage loss %.6f - Avarage accuracy %.4f  (%.0f steps/s)\n", i,
                  total_loss / n, total_acc / n, n / secs);
    }
    std::printf("%s\n", model.debug().c_str());
  } catch (const Panic& p) {
    std::fprintf(stderr, "panic: %s\n", p.what());
    return 1;
  }
  return 0;
}
