// Sweeps the contraction planner over a few thousand (M, N, K, leading dimension, alignment, epilogue,
// workspace) cases on the host: every launch the library plans is walked lane by lane by the address
// model (address_model.cpp), which aborts on the first access outside an operand.  Operands are
// made-up addresses - nothing is dereferenced, kernels never run (hip_stub.cpp) - so leading
// dimensions of 2^22 or 2^26 doubles cost nothing.  Ends with the count of launches verified per
// kernel and fails if a kernel or a route of the planner was never reached.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../rstorch_amd/csrc/common.h"

extern "C" long address_model_checked(int kernel);
extern "C" long address_model_staged_checked(int tile);
extern "C" long address_model_sliced(int kernel);
extern "C" long address_model_unaligned(int kernel);
extern "C" long address_model_reserved(int kernel);
extern "C" long address_model_repeats();
extern "C" long long address_model_lane_checks();
extern "C" const char* address_model_kernel_name(int kernel);

using namespace rst;

namespace {

unsigned long long g_state = 0x9E3779B97F4A7C15ull;
unsigned rnd(unsigned n) {  // splitmix64, reproducible
  g_state += 0x9E3779B97F4A7C15ull;
  unsigned long long z = g_state;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z ^= z >> 31;
  return (unsigned)(z % n);
}

double* fake(unsigned long long region, bool misaligned) {
  return reinterpret_cast<double*>((region << 40) + (misaligned ? 8 : 0));
}

constexpr size_t kWorkspace = (size_t)16 << 20;  // the engine's: 16 Mi doubles

enum Layout { FORWARD, WEIGHT_GRAD, INPUT_GRAD };

struct Case {
  Layout layout;
  int M, N, K;       // of the contraction C[M,N] = sum_k
  long pad_a, pad_b, pad_c;  // added to the dense leading dimension
  bool misaligned_a, misaligned_b;
  int epilogue_variant;
  int workspace;     // 0 none, 1 the engine's, 2 tiny
};

GemmDesc make(const Case& c) {
  GemmDesc d{};
  d.M = c.M; d.N = c.N; d.K = c.K;
  d.a_kc = c.layout != WEIGHT_GRAD;
  d.b_kc = c.layout == FORWARD;
  d.lda = (d.a_kc ? c.K : c.M) + c.pad_a;
  d.ldb = (d.b_kc ? c.K : c.N) + c.pad_b;
  d.ldc = c.N + c.pad_c;
  d.A = fake(1, c.misaligned_a);
  d.B = fake(2, c.misaligned_b);
  d.C = fake(3, false);
  d.bias = fake(4, false);
  d.mask = nullptr;
  d.ldmask = c.N + (c.epilogue_variant & 4 ? 6 : 0);
  d.divisor = c.layout == WEIGHT_GRAD ? (c.epilogue_variant & 1 ? (double)c.K : 1024.0) : 1.0;
  switch (c.layout) {
    case FORWARD: {
      const int e[4] = {EPI_BIAS, EPI_BIAS_RELU, EPI_RELU, EPI_NONE};
      d.epilogue = e[c.epilogue_variant & 3];
      break;
    }
    case WEIGHT_GRAD:
      d.epilogue = EPI_DIVIDE;
      if (c.epilogue_variant & 2) { d.colsum = fake(5, false); d.colsum_div = d.divisor; }
      if (c.epilogue_variant & 4) {
        d.sgd_parm = fake(6, false);
        d.sgd_bias = d.colsum ? fake(7, false) : nullptr;
        d.sgd_lr = 0.01;
      }
      break;
    default:
      d.epilogue = c.epilogue_variant & 1 ? EPI_MASK : EPI_NONE;
      if (d.epilogue == EPI_MASK) d.mask = fake(8, false);
      break;
  }
  if (c.workspace == 1) { d.workspace = fake(9, false); d.workspace_count = kWorkspace; }
  if (c.workspace == 2) { d.workspace = fake(9, false); d.workspace_count = 4096; }
  return d;
}

long g_cases = 0;
void run(const Case& c) {
  const GemmDesc d = make(c);
  ++g_cases;
  if (launch_gemm(nullptr, d) != RST_OK) {
    std::fprintf(stderr, "launch_gemm refused layout %d M=%d N=%d K=%d: %s\n", (int)c.layout, c.M, c.N, c.K, rst_last_error());
    std::exit(1);
  }
}

}  // namespace

int main() {
  // ---- every layout over ragged extents, leading dimensions and alignments -----------------------------
  const int small[] = {1, 2, 3, 7, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 130, 255, 256, 257, 300};
  const int mid[] = {384, 500, 512, 784, 1000, 1023, 1024, 1025, 2046, 2048, 4096};
  const int ks[] = {1, 2, 3, 15, 16, 17, 31, 32, 33, 100, 127, 128, 130, 255, 256, 400, 784, 1000, 1024, 2048, 4096, 8192, 16400};
  const long pads[] = {0, 0, 0, 2, 1, 6, 64};
  for (int layout = 0; layout < 3; ++layout) {
    // exhaustive over the small extents with short contractions
    for (int m : small)
      for (int n : small) {
        Case c{(Layout)layout, m, n, ks[rnd(16)], pads[rnd(7)], pads[rnd(7)], pads[rnd(7)], rnd(8) == 0, rnd(8) == 0,
               (int)rnd(8), (int)rnd(3)};
        run(c);
      }
    // random mixes of small / mid extents and all contraction lengths, output capped at 4 Mi elements
    for (int it = 0; it < 900; ++it) {
      const int m = rnd(3) ? mid[rnd(11)] : small[rnd(22)];
      const int n = rnd(3) ? mid[rnd(11)] : small[rnd(22)];
      Case c{(Layout)layout, m, n, ks[rnd(23)], pads[rnd(7)], pads[rnd(7)], pads[rnd(7)], rnd(10) == 0, rnd(10) == 0,
             (int)rnd(8), rnd(6) ? 1 : (int)rnd(3)};
      run(c);
    }
    // long batches over narrow outputs (K slices, one round and several), with every workspace mode
    const int batches[] = {4096, 8192, 32768, 70000, 131072};
    for (int b : batches)
      for (int w : {10, 64, 100, 128, 256, 784})
        for (int ws = 0; ws < 3; ++ws) {
          if (b > 8192 && w > 100 && (layout != WEIGHT_GRAD || ws != 1)) continue;  // (keeps the sweep short)
          if (layout == WEIGHT_GRAD) run(Case{WEIGHT_GRAD, w, small[rnd(22)] + 1, b, 0, 0, 0, false, false, (int)rnd(8), ws});
          else run(Case{(Layout)layout, b, w, mid[rnd(11)], 0, 0, 0, false, false, (int)rnd(8), ws});
        }
    // rows of 70000 doubles, on either side
    run(Case{(Layout)layout, 130, 70000, 256, 0, 0, 0, false, false, 1, 1});
    run(Case{(Layout)layout, 70000, 34, 100, 0, 0, 0, false, false, 1, 1});
    run(Case{(Layout)layout, 64, 66, 70000, 0, 0, 0, false, false, 3, 1});
    run(Case{(Layout)layout, 258, 514, 70002, 2, 2, 0, false, false, 3, 1});
    // leading dimensions at the limits of the 32-bit lane offsets: 2^22 for the tile DMA (just under:
    // DMA path, at: register-staged path), 2^26 for the unpredicated epilogue
    const long at22 = 1L << 22, at26 = 1L << 26;
    for (long ld : {at22 - 2, at22, at22 + 2}) {
      const int dense_a = layout == WEIGHT_GRAD ? 2048 : 512, dense_b = layout == FORWARD ? 512 : 2048;
      run(Case{(Layout)layout, 2048, 2048, 512, ld - dense_a, ld - dense_b, 0, false, false, 2, 1});
      run(Case{(Layout)layout, 300, 200, 2048, ld - (layout == WEIGHT_GRAD ? 300 : 2048), ld - (layout == FORWARD ? 2048 : 200), 0, false, false, 2, 1});
    }
    for (long ld : {at26 - 2, at26})
      run(Case{(Layout)layout, 256, 384, 64, 0, 0, ld - 384, false, false, layout == INPUT_GRAD ? 5 : 6, 1});
  }
  // ---- the benchmark configurations' own products ------------------------------------------------------
  run(Case{FORWARD, 1024, 4096, 4096, 0, 0, 0, false, false, 1, 1});
  run(Case{FORWARD, 1024, 32768, 4096, 0, 0, 0, false, false, 0, 1});
  run(Case{INPUT_GRAD, 1024, 4096, 32768, 0, 0, 0, false, false, 1, 1});
  run(Case{WEIGHT_GRAD, 4096, 4096, 1024, 0, 0, 0, false, false, 6, 1});
  run(Case{WEIGHT_GRAD, 1000, 4096, 2048, 0, 0, 0, false, false, 6, 1});
  run(Case{FORWARD, 8192, 100, 784, 0, 0, 0, false, false, 1, 1});
  run(Case{INPUT_GRAD, 8192, 100, 100, 0, 0, 0, false, false, 1, 1});
  // ---- a network with every extent odd (1023-4095-4095-999 at batch 2047) and its neighbours: the tile DMA
  //      on 8-byte aligned pairs, the last K row kept back where a pair could reach behind the operand ------
  for (int batch : {2047, 2048, 2049})
    for (int pad : {0, 1}) {
      const int w[4] = {1023, 4095, 4095, 999};
      for (int l = 0; l < 3; ++l) {
        run(Case{FORWARD, batch, w[l + 1], w[l], pad, pad, 0, pad == 1, false, 1, 1});
        run(Case{WEIGHT_GRAD, w[l + 1], w[l], batch, pad, 0, pad, false, pad == 1, 6, 1});
        run(Case{INPUT_GRAD, batch, w[l], w[l + 1], 0, pad, 0, false, false, 1, 1});
      }
    }
  // K a multiple of 16 with an odd output-contiguous extent (the tail is then a whole step), mid sizes on slices
  run(Case{WEIGHT_GRAD, 4095, 1023, 2048, 0, 0, 0, false, false, 6, 1});
  run(Case{INPUT_GRAD, 2048, 1023, 4096, 0, 0, 0, false, false, 1, 1});
  run(Case{INPUT_GRAD, 8192, 101, 785, 0, 0, 0, false, false, 1, 1});
  run(Case{FORWARD, 8192, 101, 785, 0, 0, 0, false, false, 1, 1});
  run(Case{WEIGHT_GRAD, 1001, 1535, 4096, 0, 0, 0, false, false, 6, 1});
  run(Case{WEIGHT_GRAD, 999, 1023, 16, 0, 0, 0, false, false, 6, 1});
  run(Case{WEIGHT_GRAD, 4095, 4095, 16, 0, 0, 0, false, false, 6, 1});
  run(Case{WEIGHT_GRAD, 4095, 4095, 17, 0, 0, 0, false, false, 6, 1});
  // forward products of 257..511 tiles: K slices that even out the compute units (two, three slices; ragged, odd)
  run(Case{FORWARD, 1024, 4608, 4096, 0, 0, 0, false, false, 1, 1});
  run(Case{FORWARD, 1024, 4608, 2048, 0, 0, 0, false, false, 0, 1});
  run(Case{FORWARD, 1030, 4600, 2056, 0, 0, 0, false, false, 1, 1});
  run(Case{FORWARD, 1535, 4095, 4097, 0, 0, 0, false, false, 1, 1});
  run(Case{FORWARD, 1024, 4608, 4096, 0, 0, 0, false, false, 1, 0});  // (no workspace: unsliced)
  // 256..511 tiles over a very long contraction (two K halves), odd everywhere
  run(Case{WEIGHT_GRAD, 2047, 2045, 24577, 0, 0, 0, false, false, 6, 1});
  run(Case{WEIGHT_GRAD, 2047, 2045, 24576, 1, 0, 0, false, false, 6, 1});
  run(Case{INPUT_GRAD, 2049, 2047, 24593, 0, 0, 0, true, false, 1, 1});
  run(Case{FORWARD, 2047, 2049, 24577, 0, 0, 0, false, true, 1, 1});

  // ---- grouped launches: weight gradients of small layers, short and long batches ----------------------
  long groups = 0, pairs = 0;
  for (int it = 0; it < 300; ++it) {
    const int count = 2 + (int)rnd(7);
    const int batch = (const int[]){32, 100, 256, 1000, 4096, 8192, 32768}[rnd(7)];
    std::vector<GemmDesc> ds;
    bool ok = true;
    for (int i = 0; i < count; ++i) {
      // every third group has members of odd extents (single loads, 8-byte aligned tile DMA)
      const int odd = it % 3 == 2 ? 1 : 0;
      Case c{WEIGHT_GRAD, 2 * (1 + (int)rnd(150)) - odd * (int)rnd(2), 2 * (1 + (int)rnd(400)) - odd * (int)rnd(2), batch - odd * (int)rnd(2),
             0, 0, 0, false, false, 2 + 4 * (int)rnd(2), 1};
      GemmDesc d = make(c);
      if (it % 5 == 4 && i == count - 1) {  // a layer's input gradient riding along (mixed layouts)
        Case x{INPUT_GRAD, batch, 2 * (1 + (int)rnd(60)) - odd * (int)rnd(2), 2 * (1 + (int)rnd(60)) - odd * (int)rnd(2), 0, 0, 0, false, false,
               (int)rnd(2), 1};
        d = make(x);
      }
      ok = ok && can_group_gemm(d);
      ds.push_back(d);
    }
    if (!ok || gemm_group_workspace(ds.data(), count) > kWorkspace) continue;
    if (launch_gemm_group(nullptr, ds.data(), count) != RST_OK) {
      std::fprintf(stderr, "launch_gemm_group refused a group that can_group_gemm accepted: %s\n", rst_last_error());
      return 1;
    }
    ++groups;
  }
  // ---- paired launches: an input gradient with the weight gradient of the layer above ------------------
  const int widths[] = {2048, 4096, 4224, 8192, 32768, 4095, 2049};
  for (int batch : {1024, 2048, 4096, 1023, 2047})
    for (int w_in : widths)
      for (int w_out : widths) {
        // (one pair with the 32768-wide head, the others up to 32 Mi outputs)
        if ((long long)w_in * w_out > (1LL << 25) && !(batch == 1024 && w_in == 4096 && w_out == 32768)) continue;
        GemmDesc dx = make(Case{INPUT_GRAD, batch, w_in, w_out, 0, 0, 0, false, false, 1, 1});
        GemmDesc dw = make(Case{WEIGHT_GRAD, w_out, w_in, batch, 0, 0, 0, false, false, 6, 1});
        if (!can_pair_gemm(dx, dw)) continue;
        if (launch_gemm_pair(nullptr, dx, dw) != RST_OK) {
          std::fprintf(stderr, "launch_gemm_pair refused a pair that can_pair_gemm accepted: %s\n", rst_last_error());
          return 1;
        }
        ++pairs;
      }

  // ---- report, and insist that every kernel and every route was reached --------------------------------
  long total = 0;
  bool all = true;
  for (int k = 0; k <= 8; ++k) {
    std::printf("  %-20s %6ld launches verified (%ld on K slices)\n", address_model_kernel_name(k), address_model_checked(k),
                address_model_sliced(k));
    total += address_model_checked(k);
    all = all && address_model_checked(k) > 0;
  }
  for (int t : {32, 128}) {
    std::printf("  staged %3dx%-3d tiles  %6ld\n", t, t, address_model_staged_checked(t));
    all = all && address_model_staged_checked(t) > 0;
  }
  // sliced and unsliced direct-to-LDS launches, sliced register-staged ones
  all = all && address_model_sliced(0) > 0 && address_model_sliced(3) > 0 && address_model_sliced(6) > 0 &&
        address_model_checked(3) > address_model_sliced(3) && address_model_checked(6) > address_model_sliced(6);
  std::printf("  tile DMA on operands without aligned pairs: %ld + %ld launches (128x128 + 64x64), %ld + %ld with the last K row kept back\n",
              address_model_unaligned(3), address_model_unaligned(6), address_model_reserved(3), address_model_reserved(6));
  std::printf("  shared grids with such members: %ld + %ld + %ld + %ld launches (staged, mixed, 128x128 sliced, pairs)\n",
              address_model_unaligned(1), address_model_unaligned(2), address_model_unaligned(4), address_model_unaligned(5));
  all = all && address_model_unaligned(3) > 0 && address_model_unaligned(6) > 0 && address_model_reserved(3) > 0 &&
        address_model_reserved(6) > 0 && address_model_unaligned(1) > 0 && address_model_unaligned(2) > 0 &&
        address_model_unaligned(4) > 0 && address_model_unaligned(5) > 0 && address_model_reserved(4) > 0 &&
        address_model_reserved(5) > 0;
  std::printf("address sweep ok: %ld cases, %ld groups, %ld pairs, %ld launches verified (%ld repeats skipped), %lld address checks\n",
              g_cases, groups, pairs, total, address_model_repeats(), address_model_lane_checks());
  if (!all) {
    std::fprintf(stderr, "a kernel or a route of the planner was never reached by the sweep\n");
    return 1;
  }
  return 0;
}
