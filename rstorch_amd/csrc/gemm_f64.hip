// FP64 contraction kernels for gfx950 built on v_mfma_f64_16x16x4_f64.
//
// One kernel template covers the three products of a Linear layer
//   forward        Z[B,N]  = X[B,K] . W[N,K]^T        (A and B contraction-contiguous)
//   weight grad    dW[N,K] = G[B,N]^T . X[B,K]        (A and B output-contiguous)
//   input grad     dX[B,K] = G[B,N] . W[N,K]          (A contraction-contiguous, B output-contiguous)
// without materialising a transpose: the operand layout only changes how a tile is copied
// into LDS and which LDS stride the MFMA fragments are read with.
//
// Two kernels share the template parameters and the epilogues:
//   gemm_f64_mfma      register-staged tiles of 32x32, 64x64 or 128x128 (WGM x WGN wavefronts, each
//                      owning a (BM/WGM)x(BN/WGN) block of 16x16 MFMA tiles in registers), any
//                      shape and alignment, optional split-K for small outputs;
//   gemm_f64_mfma_dma  128x128 tiles, eight wavefronts of 64x32, operand tiles moved global -> LDS
//                      by global_load_lds_dwordx4 and a hand-scheduled inner loop: the path of
//                      the large products (at least 256 tiles, or fewer on K slices), whatever
//                      their alignment.
// K advances in steps of 16 through two LDS stages; the loads of step k+1 are in flight while
// step k is multiplied.
//
// MFMA register layout (64 lanes): A fragment lane l holds A[l%16][l/16], B fragment lane l
// holds B[l/16][l%16], and accumulator register r of lane l holds D[4*r + l/16][l%16].
#include <cmath>
#include <cstdlib>
#include <type_traits>

#include "common.h"
#include "gemm_addressing.h"

namespace rst {
namespace {

typedef double v4d __attribute__((ext_vector_type(4)));
typedef double v2d __attribute__((ext_vector_type(2)));

// LDS geometry of one operand tile of EXT rows/cols by BK contraction steps.
//   contraction-contiguous: [EXT][BK], element (e, k) at e*BK + (k ^ (e & 15)).  The XOR spreads
//       the 16 rows that one MFMA fragment read touches over all sixteen 8-byte bank pairs, for
//       any k, without padding; an aligned pair (k, k+1) stays inside one 16-byte slot.
//   output-contiguous:      [BK][EXT + 16], element (e, k) at k*(EXT+16) + e.  A fragment read
//       takes 16 consecutive doubles per k, and the stride is 16 mod 32 doubles so that two
//       neighbouring k rows fall into different halves of the banks.
template <int EXT, bool KC, int THREADS>
struct TileGeom {
  static constexpr int stride = KC ? BK : (EXT + 16);
  static constexpr int size = KC ? EXT * BK : BK * (EXT + 16);
  static constexpr int loads = EXT * BK / 2 / THREADS;  // 16-byte loads per thread per tile
  static_assert(EXT * BK / 2 % THREADS == 0, "tile must split evenly over the block");
};

// Copy one operand tile global -> registers without any divergent branch: which pair a thread slot
// takes, with its clamps and the zeroing of the masked K tail, is staged_pair_source's business.
template <int EXT, bool KC, bool VEC, bool TAIL, int THREADS>
__device__ __forceinline__ void load_tile(v2d* __restrict__ reg, const double* __restrict__ base,
                                          long ld, int ext0, int ext_n, int k0, int k_n, int tid) {
  constexpr int L = TileGeom<EXT, KC, THREADS>::loads;
#pragma unroll
  for (int u = 0; u < L; ++u) {
    const PairSource src = staged_pair_source<EXT, KC, VEC, TAIL>(tid + u * THREADS, ld, ext0, ext_n, k0, k_n);
    v2d v;
    if (src.vec) {
      v = *reinterpret_cast<const v2d*>(base + src.first);
    } else {
      v.x = base[src.first];
      v.y = base[src.second];
    }
    if (TAIL) {
      v.x = src.keep_first ? v.x : 0.0;
      v.y = src.keep_second ? v.y : 0.0;
    }
    reg[u] = v;
  }
}

// Registers -> LDS stage.
template <int EXT, bool KC, int THREADS>
__device__ __forceinline__ void store_tile(double* __restrict__ lds,
                                           const v2d* __restrict__ reg, int tid) {
  constexpr int L = TileGeom<EXT, KC, THREADS>::loads;
  constexpr int S = TileGeom<EXT, KC, THREADS>::stride;
#pragma unroll
  for (int u = 0; u < L; ++u) {
    const int q = tid + u * THREADS;
    if (KC) {
      const int e = q >> 3, k = 2 * (q & 7);
      // slot of the pair: (k ^ (e & 14)); inside the slot the two doubles swap when e is odd
      v2d v = reg[u];
      if (e & 1) v = (v2d){v.y, v.x};
      *reinterpret_cast<v2d*>(lds + e * S + (k ^ (e & 14))) = v;
    } else {
      const int off = (q / (EXT / 2)) * S + 2 * (q % (EXT / 2));
      *reinterpret_cast<v2d*>(lds + off) = reg[u];
    }
  }
}

// LDS -> MFMA fragment: element (e, k) of the tile, e = output index inside the tile.
template <int EXT, bool KC>
__device__ __forceinline__ double read_frag(const double* __restrict__ lds, int e, int k) {
  constexpr int S = TileGeom<EXT, KC, 64>::stride;
  return KC ? lds[e * S + (k ^ (e & 15))] : lds[k * S + e];
}

// parm - (lr * grad) with the product rounded before the subtraction (src/optim/sgd.rs:23)
__device__ __forceinline__ double sgd_apply(double w, double g, double lr) {
#pragma clang fp contract(off)
  const double step = lr * g;
  return w - step;
}

// Epilogue of one wavefront's block of 16x16 tiles: accumulator register r of fragment (i, j) is
// row row0 + 16*i + 4*r + lk, column col0 + 16*j + lr.  What an element needs from memory (the ReLU
// mask, or the parameter that the fused SGD update rewrites) is requested for one fragment row at
// a time from clamped, always valid addresses before any of it is used, so that the loads of a
// batch are in flight together; only the stores are predicated on the bounds.
template <int TM, int TN, int EPI, bool SGD>
__device__ __forceinline__ void store_block(const GemmParams& p, const v4d* acc, int row0, int col0,
                                            int lr, int lk) {
  constexpr int IB = 1;  // two rows at a time would spill in the 128x128 kernels
#pragma unroll
  for (int i0 = 0; i0 < TM; i0 += IB) {
    double extra[IB][TN][4];
    double bias[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = acc_col(col0, j, lr);
      const int cc = col < p.N ? col : p.N - 1;
      if (EPI == EPI_BIAS || EPI == EPI_BIAS_RELU) bias[j] = p.bias[cc];
      if (EPI == EPI_MASK || SGD) {
#pragma unroll
        for (int ii = 0; ii < IB; ++ii)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int row = acc_row(row0, i0 + ii, r, lk);
            const int rc = row < p.M ? row : p.M - 1;
            extra[ii][j][r] = (EPI == EPI_MASK) ? p.mask[(size_t)rc * p.ldmask + cc]
                                                : p.sgd_parm[(size_t)rc * p.ldc + cc];
          }
      }
    }
#pragma unroll
    for (int ii = 0; ii < IB; ++ii)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int col = acc_col(col0, j, lr);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = acc_row(row0, i0 + ii, r, lk);
          double v = acc[(i0 + ii) * TN + j][r];
          if (EPI == EPI_BIAS) v = v + bias[j];
          if (EPI == EPI_BIAS_RELU) v = fmax(v + bias[j], 0.0);
          if (EPI == EPI_RELU) v = fmax(v, 0.0);
          if (EPI == EPI_DIVIDE) v = v / p.divisor;
          if (EPI == EPI_MASK) v = v * (extra[ii][j][r] > 0.0 ? 1.0 : 0.0);
          if (row < p.M && col < p.N) {
            if (EPI == EPI_DIVIDE)  // a weight gradient: nothing reads it again soon
              __builtin_nontemporal_store(v, p.C + (size_t)row * p.ldc + col);
            else
              p.C[(size_t)row * p.ldc + col] = v;
            // the parameter is read and rewritten through the L2 (measured faster than streaming
            // either side of the read-modify-write past it)
            if (SGD) p.sgd_parm[(size_t)row * p.ldc + col] = sgd_apply(extra[ii][j][r], v, p.sgd_lr);
          }
        }
      }
  }
}

// The same epilogue for a block that lies wholly inside the matrix, which is nearly every block of
// a large product.  While a workgroup is in its epilogue the other workgroup of the CU keeps the
// matrix pipeline full, and FP64 MFMAs hold the vector ALU for all of their 64 cycles: a vector
// instruction of the epilogue gets in only between two of them.  Measured on the 4096 x 4096 weight
// gradient: the general epilogue above (a bounds test, a branch and 64-bit address arithmetic per
// element, and for the weight gradient a division: some 10 to 25 vector instructions per stored
// value) takes 27 us next to a running K loop, 47 us with the SGD update, against 2.8 us on a CU of
// its own; the last epilogue of every CU is exposed at the end of the launch.  Here an access is a
// wave-uniform row pointer kept in scalar registers (scalar adds from row to row), one 32-bit lane
// offset and an immediate column offset: no vector instruction per address, no predicates, and the
// division by a power of two (the usual batch size) is a multiplication by its exact reciprocal -
// the same bits for every operand, gradual underflow included.
template <int TM, int TN, int EPI, bool SGD, bool RECIP>
__device__ __forceinline__ void store_block_interior(const GemmParams& p, const v4d* acc, double* out,
                                                     long ld_out, int row0, int col0, int lr, int lk) {
  constexpr bool BIAS = EPI == EPI_BIAS || EPI == EPI_BIAS_RELU;
  uint32_t off_c = interior_lane_offset<uint32_t>(lk, lr, ld_out);
  uint32_t off_m = EPI == EPI_MASK ? interior_lane_offset<uint32_t>(lk, lr, p.ldmask) : 0u;
  char* c_row = reinterpret_cast<char*>(out + (size_t)row0 * ld_out + col0);
  char* w_row = SGD ? reinterpret_cast<char*>(p.sgd_parm + (size_t)row0 * ld_out + col0) : nullptr;
  const char* m_row = EPI == EPI_MASK ? reinterpret_cast<const char*>(p.mask + (size_t)row0 * p.ldmask + col0) : nullptr;
  const long c_step = 32 * ld_out;      // bytes from accumulator register r to r + 1: four rows
  const long m_step = 32 * p.ldmask;
  double bias[TN];
  if (BIAS) {
#pragma unroll
    for (int j = 0; j < TN; ++j) bias[j] = p.bias[col0 + j * 16 + lr];
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    double extra[TN][4];
    if (EPI == EPI_MASK || SGD) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const char* src = EPI == EPI_MASK ? m_row + r * m_step : w_row + r * c_step;  // scalar
        // hiding the offset from the optimiser before every use keeps "scalar base + 32-bit lane
        // offset + immediate" one addressing mode instead of a 64-bit vector addition per row
        asm volatile("" : "+v"(off_c), "+v"(off_m));
        const uint32_t off = EPI == EPI_MASK ? off_m : off_c;
#pragma unroll
        for (int j = 0; j < TN; ++j) extra[j][r] = *reinterpret_cast<const double*>(src + off + 128 * j);
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      char* dst_row = c_row + r * c_step;
      char* parm_row = SGD ? w_row + r * c_step : nullptr;
      asm volatile("" : "+v"(off_c));
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        double v = acc[i * TN + j][r];
        // (opaque, so that the arithmetic that two epilogue kinds have in common is not hoisted out
        // of the switch for all 32 values at once, which spills)
        if (EPI == EPI_DIVIDE || BIAS) asm volatile("" : "+v"(v));
        if (EPI == EPI_BIAS) v = v + bias[j];
        if (EPI == EPI_BIAS_RELU) v = fmax(v + bias[j], 0.0);
        if (EPI == EPI_RELU) v = fmax(v, 0.0);
        if (EPI == EPI_DIVIDE) v = RECIP ? v * p.divisor_reciprocal : v / p.divisor;
        if (EPI == EPI_MASK) v = v * (extra[j][r] > 0.0 ? 1.0 : 0.0);
        double* dst = reinterpret_cast<double*>(dst_row + off_c + 128 * j);
        if (EPI == EPI_DIVIDE) __builtin_nontemporal_store(v, dst);
        else *dst = v;
        if (SGD) *reinterpret_cast<double*>(parm_row + off_c + 128 * j) = sgd_apply(extra[j][r], v, p.sgd_lr);
      }
    }
    // One fragment row at a time: hoisting the arithmetic of later rows would double the live
    // registers.  Requesting the parameters of the next row before this one is stored was measured
    // too: the epilogue itself drops from 33 to 10 us, but the launch gets 4 % longer - every CU
    // reaches its epilogues at about the same time, and the shorter they are, the harder their
    // burst of loads and stores hits the tile loads of the workgroups that are still multiplying.
    // (Stretching the epilogue with sleeps between the rows, to 41 and 50 us, costs 2 % and 5 %.)
    __builtin_amdgcn_sched_barrier(0);
    c_row += 4 * c_step;
    if (SGD) w_row += 4 * c_step;
    if (EPI == EPI_MASK) m_row += 4 * m_step;
  }
}

// Writes the block either as raw partial products of K slice `split` (the reduction applies the
// epilogue later) or finished, with the epilogue the launch asks for.
template <int TM, int TN>
__device__ __forceinline__ void write_block(const GemmParams& p, const v4d* acc, int row0, int col0,
                                            int lr, int lk, int split) {
  // the block origin is the same for the whole wavefront: keep it in scalar registers
  row0 = __builtin_amdgcn_readfirstlane(row0);
  col0 = __builtin_amdgcn_readfirstlane(col0);
  // (leading dimensions below 2^26 doubles keep the 32-bit lane offsets in range)
  const bool interior = block_is_interior(p, row0, col0, TM, TN);
  if (p.split_k > 1) {
    double* __restrict__ out = p.ws + ws_slice_offset(p, split);
    if (interior) {
      store_block_interior<TM, TN, EPI_NONE, false, false>(p, acc, out, p.N, row0, col0, lr, lk);
      return;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int col = acc_col(col0, j, lr);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = acc_row(row0, i, r, lk);
          if (row < p.M && col < p.N) out[(size_t)row * p.N + col] = acc[i * TN + j][r];
        }
      }
    return;
  }
  // (a true division keeps to the general path: its temporaries on top of a batch of parameter
  // loads do not fit the registers that the accumulators leave)
  if (interior && (p.epilogue != EPI_DIVIDE || p.divisor_reciprocal != 0.0)) {
    switch (p.epilogue) {
      case EPI_BIAS: store_block_interior<TM, TN, EPI_BIAS, false, false>(p, acc, p.C, p.ldc, row0, col0, lr, lk); break;
      case EPI_BIAS_RELU: store_block_interior<TM, TN, EPI_BIAS_RELU, false, false>(p, acc, p.C, p.ldc, row0, col0, lr, lk); break;
      case EPI_RELU: store_block_interior<TM, TN, EPI_RELU, false, false>(p, acc, p.C, p.ldc, row0, col0, lr, lk); break;
      case EPI_MASK: store_block_interior<TM, TN, EPI_MASK, false, false>(p, acc, p.C, p.ldc, row0, col0, lr, lk); break;
      case EPI_DIVIDE:
        if (p.sgd_parm) store_block_interior<TM, TN, EPI_DIVIDE, true, true>(p, acc, p.C, p.ldc, row0, col0, lr, lk);
        else store_block_interior<TM, TN, EPI_DIVIDE, false, true>(p, acc, p.C, p.ldc, row0, col0, lr, lk);
        break;
      default: store_block_interior<TM, TN, EPI_NONE, false, false>(p, acc, p.C, p.ldc, row0, col0, lr, lk); break;
    }
    return;
  }
  switch (p.epilogue) {
    case EPI_BIAS: store_block<TM, TN, EPI_BIAS, false>(p, acc, row0, col0, lr, lk); break;
    case EPI_BIAS_RELU: store_block<TM, TN, EPI_BIAS_RELU, false>(p, acc, row0, col0, lr, lk); break;
    case EPI_RELU: store_block<TM, TN, EPI_RELU, false>(p, acc, row0, col0, lr, lk); break;
    case EPI_MASK: store_block<TM, TN, EPI_MASK, false>(p, acc, row0, col0, lr, lk); break;
    case EPI_DIVIDE:
      if (p.sgd_parm) store_block<TM, TN, EPI_DIVIDE, true>(p, acc, row0, col0, lr, lk);
      else store_block<TM, TN, EPI_DIVIDE, false>(p, acc, row0, col0, lr, lk);
      break;
    default: store_block<TM, TN, EPI_NONE, false>(p, acc, row0, col0, lr, lk); break;
  }
}

// Bias gradient inside the weight-gradient contraction (output-contiguous A = grad^T): the
// workgroups of tile column 0 also add up their A tile over the contraction index.  Thread t
// owns output row t % BM and every (THREADS/BM)-th contraction row; partial sums are combined
// through LDS in a fixed order at the end, so the result is reproducible.
template <int BM, int THREADS>
__device__ __forceinline__ void colsum_accumulate(double& partial, const double* __restrict__ lds_a_stage,
                                                  int tid) {
  constexpr int G = THREADS / BM;      // contraction-row groups
  constexpr int S = BM + 16;           // LDS stride of an output-contiguous tile
  const int e = tid % BM, kg = tid / BM;
#pragma unroll
  for (int k = kg; k < BK; k += G) partial += lds_a_stage[k * S + e];
}

template <int BM, int THREADS>
__device__ __forceinline__ void colsum_finish(double partial, double* __restrict__ scratch, int tid,
                                              int m0, int split, const GemmParams& p) {
  constexpr int G = THREADS / BM;
  const int e = tid % BM, kg = tid / BM;
  scratch[kg * BM + e] = partial;
  __syncthreads();
  if (kg == 0 && m0 + e < p.M) {
    double t = 0.0;
#pragma unroll
    for (int g = 0; g < G; ++g) t += scratch[g * BM + e];
    if (p.split_k > 1) {
      p.ws_colsum[ws_colsum_offset(p, split) + m0 + e] = t;  // slice sum, reduced later
    } else {
      const double g = t / p.colsum_div;
      p.colsum[m0 + e] = g;
      if (p.sgd_bias) p.sgd_bias[m0 + e] = sgd_apply(p.sgd_bias[m0 + e], g, p.sgd_lr);
    }
  }
}

// One output tile of the register-staged product: workgroup number `block` of problem p.
// BURST = 0: the operand tiles of K step kt+1 travel while step kt is multiplied (two LDS stages).
// BURST = D > 0, for grids of at most one workgroup per CU, where nothing else hides a load's
// latency: the tiles of D K steps are requested together, land in D LDS stages and are multiplied
// in K order, so a short contraction pays one trip to memory instead of one per step.  The
// accumulation order, and with it every bit of the result, is the same either way.
// lds_a / lds_b: room for kStages tiles of the respective operand (tile_lds_doubles).
template <int BM, int BN, int WGM, int WGN, bool A_KC, bool B_KC, bool VEC, int BURST = 0>
__device__ __forceinline__ void gemm_tile(const GemmParams& p, const int block, double* __restrict__ lds_a_base,
                                          double* __restrict__ lds_b_base) {
  constexpr int kThreads = WGM * WGN * 64;
  using GA = TileGeom<BM, A_KC, kThreads>;
  using GB = TileGeom<BN, B_KC, kThreads>;
  constexpr int WM = BM / WGM, WN = BN / WGN;  // per-wavefront block
  constexpr int TM = WM / 16, TN = WN / 16;  // MFMA tiles per wavefront
  static_assert(WM % 16 == 0 && WN % 16 == 0, "wave block must be whole MFMA tiles");

  constexpr int kStages = BURST > 0 ? BURST : 2;
  auto lds_a = [&](int stage) { return lds_a_base + stage * GA::size; };
  auto lds_b = [&](int stage) { return lds_b_base + stage * GB::size; };

  // (XCD-aware walk of the tile grid: tile_of_block)
  const TileCoord tc = tile_of_block(p.tiles_m, p.tiles_n, block);
  const int split = tc.split;  // K slice of this workgroup (0 without split-K)
  const int tile_m = tc.tile_m, tile_n = tc.tile_n;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WGN, wn = wave % WGN;
  const int lr = lane & 15, lk = lane >> 4;

  v4d acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = (v4d){0.0, 0.0, 0.0, 0.0};

  const StagedSteps ks = staged_k_steps(p.K, p.split_k, p.steps_per_split, split);
  const int nk_full = ks.nk_full;  // K steps that need no bounds handling
  const int kt0 = ks.kt0, nk = ks.nk;  // this workgroup's K steps: [kt0, nk)

  // Loads the operand tiles of K step `kt` into registers; only the last step can be partial.
  auto fetch = [&](int kt, v2d* ra, v2d* rb) {
    if (kt < nk_full) {
      load_tile<BM, A_KC, VEC, false, kThreads>(ra, p.A, p.lda, m0, p.M, kt * BK, p.K, tid);
      load_tile<BN, B_KC, VEC, false, kThreads>(rb, p.B, p.ldb, n0, p.N, kt * BK, p.K, tid);
    } else {
      load_tile<BM, A_KC, VEC, true, kThreads>(ra, p.A, p.lda, m0, p.M, kt * BK, p.K, tid);
      load_tile<BN, B_KC, VEC, true, kThreads>(rb, p.B, p.ldb, n0, p.N, kt * BK, p.K, tid);
    }
  };
  const bool do_colsum = !A_KC && p.colsum != nullptr && tile_n == 0;
  double colsum_partial = 0.0;
  // a wavefront whose whole block lies beyond the edge of the output (M = 100 in 32-row tiles:
  // rows 112..127) copies its share of the tiles but multiplies nothing
  const bool wave_live = m0 + wm * WM < p.M && n0 + wn * WN < p.N;
  // One K step out of LDS stage (sa, sb).
  auto multiply = [&](const double* __restrict__ sa, const double* __restrict__ sb) {
    if (!A_KC) {
      if (do_colsum) colsum_accumulate<BM, kThreads>(colsum_partial, sa, tid);
    }
    if (!wave_live) return;
#pragma unroll
    for (int ks = 0; ks < BK / 4; ++ks) {
      double fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) fa[i] = read_frag<BM, A_KC>(sa, wm * WM + i * 16 + lr, ks * 4 + lk);
#pragma unroll
      for (int j = 0; j < TN; ++j) fb[j] = read_frag<BN, B_KC>(sb, wn * WN + j * 16 + lr, ks * 4 + lk);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
  };

  if (BURST > 0) {
    v2d ra[kStages][GA::loads], rb[kStages][GB::loads];
    for (int k0 = kt0; k0 < nk; k0 += kStages) {
#pragma unroll
      for (int d = 0; d < kStages; ++d)
        if (k0 + d < nk) fetch(k0 + d, ra[d], rb[d]);
#pragma unroll
      for (int d = 0; d < kStages; ++d)
        if (k0 + d < nk) {
          store_tile<BM, A_KC, kThreads>(lds_a(d), ra[d], tid);
          store_tile<BN, B_KC, kThreads>(lds_b(d), rb[d], tid);
        }
      __syncthreads();
#pragma unroll
      for (int d = 0; d < kStages; ++d)
        if (k0 + d < nk) multiply(lds_a(d), lds_b(d));
      __syncthreads();
    }
  } else {
    v2d ra[GA::loads], rb[GB::loads];
    if (nk > kt0) {
      fetch(kt0, ra, rb);
      store_tile<BM, A_KC, kThreads>(lds_a(0), ra, tid);
      store_tile<BN, B_KC, kThreads>(lds_b(0), rb, tid);
    }
    __syncthreads();
    for (int kt = kt0; kt < nk; ++kt) {
      const int cur = (kt - kt0) & 1;
      const bool more = kt + 1 < nk;
      if (more) fetch(kt + 1, ra, rb);  // in flight while this step is multiplied
      multiply(lds_a(cur), lds_b(cur));
      if (more) {
        store_tile<BM, A_KC, kThreads>(lds_a(cur ^ 1), ra, tid);
        store_tile<BN, B_KC, kThreads>(lds_b(cur ^ 1), rb, tid);
      }
      __syncthreads();
    }
  }
  if (!A_KC) {
    if (do_colsum) colsum_finish<BM, kThreads>(colsum_partial, lds_b(0), tid, m0, split, p);
  }

  write_block<TM, TN>(p, &acc[0][0], m0 + wm * WM, n0 + wn * WN, lr, lk, split);
}

// LDS doubles that gemm_tile needs for one operand
template <int EXT, bool KC, int THREADS, int BURST>
constexpr int tile_lds_doubles() { return (BURST > 0 ? BURST : 2) * TileGeom<EXT, KC, THREADS>::size; }

template <int BM, int BN, int WGM, int WGN, bool A_KC, bool B_KC, bool VEC, int BURST = 0>
__global__ __launch_bounds__(WGM * WGN * 64, (BURST > 0 ? 1 : WGM * WGN >= 8 ? 4 : 2)) void gemm_f64_mfma(
    const GemmParams p) {
  __shared__ __attribute__((aligned(16))) double lds_a[tile_lds_doubles<BM, A_KC, WGM * WGN * 64, BURST>()];
  __shared__ __attribute__((aligned(16))) double lds_b[tile_lds_doubles<BN, B_KC, WGM * WGN * 64, BURST>()];
  gemm_tile<BM, BN, WGM, WGN, A_KC, B_KC, VEC, BURST>(p, (int)blockIdx.x, lds_a, lds_b);
}

// Up to kMaxGroup small products of the same operand layouts in one grid of 32x32 tiles (the
// weight gradients of a small network: each is a handful of tiles, and a launch of its own costs
// more than its arithmetic).  Workgroups [first_block[i], first_block[i+1]) belong to problem i;
// problems cut into K slices are finished by one shared reduction grid, whose workgroups
// [first_reduce_block[i], first_reduce_block[i+1]) belong to problem i.

template <bool A_KC, bool B_KC, int BURST>
__global__ __launch_bounds__(256, (BURST > 0 ? 1 : 2)) void gemm_f64_mfma_group(const GemmGroup g) {
  __shared__ __attribute__((aligned(16))) double lds_a[tile_lds_doubles<32, A_KC, 256, BURST>()];
  __shared__ __attribute__((aligned(16))) double lds_b[tile_lds_doubles<32, B_KC, 256, BURST>()];
  const int i = group_member_of_block(g.first_block, g.count, (int)blockIdx.x);
  // (uniform over the workgroup: a member whose operands do not promise aligned pairs loads singly)
  if (g.p[i].unaligned) gemm_tile<32, 32, 2, 2, A_KC, B_KC, false, BURST>(g.p[i], (int)blockIdx.x - g.first_block[i], lds_a, lds_b);
  else gemm_tile<32, 32, 2, 2, A_KC, B_KC, true, BURST>(g.p[i], (int)blockIdx.x - g.first_block[i], lds_a, lds_b);
}

// The same with a layout per problem (a layer's input gradient next to its weight gradient).
template <int BURST>
__global__ __launch_bounds__(256, (BURST > 0 ? 1 : 2)) void gemm_f64_mfma_mixed_group(const GemmGroup g) {
  // an output-contiguous tile is the larger of the two layouts
  __shared__ __attribute__((aligned(16))) double lds_a[tile_lds_doubles<32, false, 256, BURST>()];
  __shared__ __attribute__((aligned(16))) double lds_b[tile_lds_doubles<32, false, 256, BURST>()];
  const int i = group_member_of_block(g.first_block, g.count, (int)blockIdx.x);
  const int block = (int)blockIdx.x - g.first_block[i];
  switch (g.layout[i] | (g.p[i].unaligned ? 4 : 0)) {
    case 0: gemm_tile<32, 32, 2, 2, false, false, true, BURST>(g.p[i], block, lds_a, lds_b); break;
    case 1: gemm_tile<32, 32, 2, 2, true, false, true, BURST>(g.p[i], block, lds_a, lds_b); break;
    case 2: gemm_tile<32, 32, 2, 2, false, true, true, BURST>(g.p[i], block, lds_a, lds_b); break;
    case 3: gemm_tile<32, 32, 2, 2, true, true, true, BURST>(g.p[i], block, lds_a, lds_b); break;
    // members whose operands do not promise aligned pairs: single loads
    case 4: gemm_tile<32, 32, 2, 2, false, false, false, BURST>(g.p[i], block, lds_a, lds_b); break;
    case 5: gemm_tile<32, 32, 2, 2, true, false, false, BURST>(g.p[i], block, lds_a, lds_b); break;
    case 6: gemm_tile<32, 32, 2, 2, false, true, false, BURST>(g.p[i], block, lds_a, lds_b); break;
    default: gemm_tile<32, 32, 2, 2, true, true, false, BURST>(g.p[i], block, lds_a, lds_b); break;
  }
}

// ---- 128x128 tiles fed by direct global -> LDS loads ------------------------------------------
// The main path for large problems.  K need not be a multiple of 16: its remainder is a masked
// extra tile.  The operands need no more than their 8-byte alignment: global_load_lds_dwordx4 takes
// a global address that is only 8-byte aligned at its full rate (measured), so odd leading
// dimensions and extents travel the same way; for those the K tail is fetched by single loads and
// GemmParams::k_reserve keeps the operand's last K row for it when a pair could reach behind it.
// global_load_lds_dwordx4 moves 16 bytes per lane straight into LDS (lane l lands at
// base + 16*l), so no staging registers and no ds_write instructions are spent on the operand
// tiles; a wavefront moves one 1 KiB chunk of a tile per instruction:
//   contraction-contiguous operand: a chunk is 8 rows x 16 doubles; lane l fetches, for row
//       l/8, the pair k = 2*((l%8) ^ (row&7)), i.e. the XOR swizzle is applied by choosing the
//       global address; a fragment read takes the whole 16-byte slot (ds_read_b128), and with
//       this swizzle any eight consecutive lanes (eight rows, one pair) hit eight different
//       slots: SQ_LDS_BANK_CONFLICT reads 0;
//   output-contiguous operand: a chunk is one k row of 128 doubles; rows sit 144 doubles apart.
// STAGES LDS stages form a ring, tile kt+DIST is requested while tile kt is multiplied; the
// wait before the barrier only covers the tile needed next.
typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

__device__ __forceinline__ void dma16(const double* g, double* lds_wave_base) {
  // every lane moves 16 bytes; lane l lands at lds_wave_base + 16*l
  __builtin_amdgcn_global_load_lds((gbl_ptr_t)g, (lds_ptr_t)(uintptr_t)lds_wave_base, 16, 0, 0);
}

// Registers -> LDS in the layouts of the DMA tiles (for the masked K tail): pair q of the tile as
// load_tile numbers them.
template <int EXT, bool KC, int THREADS>
__device__ __forceinline__ void store_tile_dma(double* __restrict__ lds, const v2d* __restrict__ reg,
                                               int tid) {
  constexpr int L = EXT * BK / 2 / THREADS;
#pragma unroll
  for (int u = 0; u < L; ++u) {
    const int q = tid + u * THREADS;
    if (KC) {
      const int e = q >> 3, pr = q & 7;  // row, pair k/2
      *reinterpret_cast<v2d*>(lds + frag_lds_kc(e, pr)) = reg[u];
    } else {
      *reinterpret_cast<v2d*>(lds + (q / (EXT / 2)) * (EXT + 16) + 2 * (q % (EXT / 2))) = reg[u];
    }
  }
}

__device__ __forceinline__ void wait_vmcnt(int n) {
  // s_waitcnt with only the vector-memory counter constrained (gfx9 encoding)
  switch (n) {
    case 0: __builtin_amdgcn_s_waitcnt(0x0F70 | 0); break;
    case 1: __builtin_amdgcn_s_waitcnt(0x0F70 | 1); break;
    case 2: __builtin_amdgcn_s_waitcnt(0x0F70 | 2); break;
    case 3: __builtin_amdgcn_s_waitcnt(0x0F70 | 3); break;
    case 4: __builtin_amdgcn_s_waitcnt(0x0F70 | 4); break;
    case 6: __builtin_amdgcn_s_waitcnt(0x0F70 | 6); break;
    case 8: __builtin_amdgcn_s_waitcnt(0x0F70 | 8); break;
    case 12: __builtin_amdgcn_s_waitcnt(0x0F70 | 12); break;
    default: __builtin_amdgcn_s_waitcnt(0x0F70 | 0); break;
  }
}

// One fragment of one pair of K steps: 16 bytes per lane, .x feeds the first step, .y the second.
//   contraction-contiguous tile: the 16-byte slot (k, k+1) of row I*16 + lr -> one ds_read_b128;
//   output-contiguous tile: column I*16 + lr of k rows k and k+1 (144 doubles apart) -> ds_read2_b64.
template <bool KC, int I>
__device__ __forceinline__ void read_quad(v2d& q, uint32_t addr) {
  static_assert(I >= 0 && I < 4, "four fragments at most");
  if constexpr (KC) {
    if constexpr (I == 0) asm volatile("ds_read_b128 %0, %1" : "=v"(q) : "v"(addr) : "memory");
    if constexpr (I == 1) asm volatile("ds_read_b128 %0, %1 offset:2048" : "=v"(q) : "v"(addr) : "memory");
    if constexpr (I == 2) asm volatile("ds_read_b128 %0, %1 offset:4096" : "=v"(q) : "v"(addr) : "memory");
    if constexpr (I == 3) asm volatile("ds_read_b128 %0, %1 offset:6144" : "=v"(q) : "v"(addr) : "memory");
  } else {
    if constexpr (I == 0) asm volatile("ds_read2_b64 %0, %1 offset1:144" : "=v"(q) : "v"(addr) : "memory");
    if constexpr (I == 1) asm volatile("ds_read2_b64 %0, %1 offset0:16 offset1:160" : "=v"(q) : "v"(addr) : "memory");
    if constexpr (I == 2) asm volatile("ds_read2_b64 %0, %1 offset0:32 offset1:176" : "=v"(q) : "v"(addr) : "memory");
    if constexpr (I == 3) asm volatile("ds_read2_b64 %0, %1 offset0:48 offset1:192" : "=v"(q) : "v"(addr) : "memory");
  }
}

// Work of one workgroup: output tile number `block` (and its K slice) of problem p.  lds_a / lds_b
// are the workgroup's STAGES operand stages (A_SIZE / B_SIZE doubles each, at most kDmaStage).
constexpr int kDmaStage = BK * (128 + 16);  // the larger of the two tile layouts

// RAGGED: a wavefront multiplies only the 16x16 fragments of its 64x32 block that reach into the
// output (wave-uniform tests around the MFMAs).  For grids of few tiles around narrow outputs - a
// 100 x 784 weight gradient - where the fragments beyond the edge are a fifth of the work; the
// large products leave it off and keep their instruction stream free of branches.
template <bool A_KC, bool B_KC, int WGM, int WGN, int STAGES, int DIST, bool RAGGED = false>
__device__ __forceinline__ void dma_tile(const GemmParams& p, int block, double* __restrict__ lds_a,
                                         double* __restrict__ lds_b) {
  constexpr int BM = 128, BN = 128, NW = WGM * WGN;
  constexpr int WM = BM / WGM, WN = BN / WGN, TM = WM / 16, TN = WN / 16;
  constexpr int CH = 16 / NW;  // 1 KiB chunks of each operand tile moved by one wavefront
  static_assert(16 % NW == 0 && CH >= 1, "chunks must split over the wavefronts");
  constexpr int A_SIZE = A_KC ? BM * BK : BK * (BM + 16);
  constexpr int B_SIZE = B_KC ? BN * BK : BK * (BN + 16);
  static_assert(A_SIZE <= kDmaStage && B_SIZE <= kDmaStage, "stage size");

  const TileCoord tc = tile_of_block(p.tiles_m, p.tiles_n, block);
  const int split = tc.split;  // K slice of this workgroup (0 without split-K)
  const int tile_m = tc.tile_m, tile_n = tc.tile_n;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WGN, wn = wave % WGN;
  const int lr = lane & 15, lk = lane >> 4;

  // Tile DMA addressing: a uniform byte pointer per operand (tile origin, advanced along K by
  // scalar adds) plus one constant 32-bit lane offset per chunk, so that issuing a tile costs no
  // vector ALU work at all; the LDS destinations are uniform too (the wavefront number is read
  // into a scalar register).
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);
  const char* a_ptr = reinterpret_cast<const char*>(p.A + (A_KC ? (size_t)m0 * p.lda : (size_t)m0));
  const char* b_ptr = reinterpret_cast<const char*>(p.B + (B_KC ? (size_t)n0 * p.ldb : (size_t)n0));
  uint32_t ao[CH], bo[CH];
  int la[CH], lb[CH];
#pragma unroll
  for (int h = 0; h < CH; ++h) {
    const int c = wave + NW * h, cs = wave_s + NW * h;
    if (A_KC) {
      ao[h] = dma_offset_kc<uint32_t>(c, lane, m0, p.M, p.lda);
      la[h] = dma_lds_chunk_kc(cs);
    } else {
      ao[h] = dma_offset_oc128<uint32_t>(c, lane, m0, p.M, p.lda);
      la[h] = dma_lds_chunk_oc128(cs, BM);
    }
    if (B_KC) {
      bo[h] = dma_offset_kc<uint32_t>(c, lane, n0, p.N, p.ldb);
      lb[h] = dma_lds_chunk_kc(cs);
    } else {
      bo[h] = dma_offset_oc128<uint32_t>(c, lane, n0, p.N, p.ldb);
      lb[h] = dma_lds_chunk_oc128(cs, BN);
    }
  }
  const long a_step = dma_k_step_bytes(A_KC, p.lda);  // bytes per K step
  const long b_step = dma_k_step_bytes(B_KC, p.ldb);

  v4d acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = (v4d){0.0, 0.0, 0.0, 0.0};

  // K steps of this workgroup: all whole ones, or slice `split` of a split contraction.  What is
  // left of K beyond its last whole step (K % 16 indices) is an extra first tile of slice 0, copied
  // into stage 0 by ordinary masked loads; the whole steps follow through the DMA pipeline.
  const DmaSteps ks = dma_k_steps(p.K, p.split_k, p.steps_per_split, split, p.k_reserve);
  const int nk_all = dma_whole_steps(p.K, p.k_reserve);
  const int kt0 = ks.kt0, nk_dma = ks.nk_dma;
  const bool k_tail = ks.k_tail;
  const int nk = nk_dma + (k_tail ? 1 : 0);
  a_ptr += (long)kt0 * a_step;
  b_ptr += (long)kt0 * b_step;
  auto issue = [&](int stage) {
#pragma unroll
    for (int h = 0; h < CH; ++h) {
      // the empty asm keeps the zero-extension of the offset next to the load, where instruction
      // selection can fold "scalar base + 32-bit lane offset" into the load's addressing mode
      asm volatile("" : "+v"(ao[h]), "+v"(bo[h]));
      dma16(reinterpret_cast<const double*>(a_ptr + ao[h]), lds_a + stage * A_SIZE + la[h]);
      dma16(reinterpret_cast<const double*>(b_ptr + bo[h]), lds_b + stage * B_SIZE + lb[h]);
    }
    a_ptr += a_step;
    b_ptr += b_step;
  };
  // The two workgroups that share a CU start together and, with equal tiles, would also reach
  // their epilogues together, round after round, and with them every other CU's: a burst of stores
  // (and, with the SGD update, of parameter loads) during which the matrix cores idle.  For some
  // tile lengths this costs 15-20 % of the launch (the weight gradient with SGD at K = 1800..2600).
  // So, in the first round, the workgroup in the upper wave slots of its CU starts about a quarter
  // of a tile late - the other has the CU to itself meanwhile, nothing is lost - and from then on
  // the two alternate.  Only the timing depends on what the hardware ID register says.
  if (p.dephase_ticks > 0 && block < p.first_round) {
    const unsigned wave_slot = __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 4);  // HW_ID.WAVE_ID
    if (wave_slot & 2) {
      const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();  // 100 MHz
      while (__builtin_amdgcn_s_memrealtime() - t0 < (unsigned long long)p.dephase_ticks)
        __builtin_amdgcn_s_sleep(32);
    }
  }
  // prologue: tile 0 in stage 0 and, with DIST > 1, tiles 1 .. DIST-1 on their way
  static_assert(DIST >= 1 && DIST < STAGES && (DIST - 1) * 2 * CH <= 4, "ring of STAGES stages, DIST tiles ahead");
  if (k_tail) {
    v2d ra[(BM * BK / 2) / (NW * 64)], rb[(BN * BK / 2) / (NW * 64)];
    if (p.unaligned) {  // (uniform over the launch)
      load_tile<BM, A_KC, false, true, NW * 64>(ra, p.A, p.lda, m0, p.M, nk_all * BK, p.K, tid);
      load_tile<BN, B_KC, false, true, NW * 64>(rb, p.B, p.ldb, n0, p.N, nk_all * BK, p.K, tid);
    } else {
      load_tile<BM, A_KC, true, true, NW * 64>(ra, p.A, p.lda, m0, p.M, nk_all * BK, p.K, tid);
      load_tile<BN, B_KC, true, true, NW * 64>(rb, p.B, p.ldb, n0, p.N, nk_all * BK, p.K, tid);
    }
    store_tile_dma<BM, A_KC, NW * 64>(lds_a, ra, tid);
    store_tile_dma<BN, B_KC, NW * 64>(lds_b, rb, tid);
  } else if (nk > 0) {
    issue(0);
  }
#pragma unroll
  for (int t = 1; t < DIST; ++t)
    if (t < nk) issue(t % STAGES);
  {
    // tile 0 is there once only the younger tiles of the prologue are still outstanding
    const int younger = nk - 1 < DIST - 1 ? (nk > 0 ? nk - 1 : 0) : DIST - 1;
    wait_vmcnt(2 * CH * younger);
  }
  if (k_tail) __syncthreads();
  else __builtin_amdgcn_s_barrier();

  const bool do_colsum = !A_KC && p.colsum != nullptr && tile_n == 0;
  double colsum_partial = 0.0;

  // The 16 contraction indices of a tile are consumed as two pairs of MFMA steps; in pair s the
  // lane group lk multiplies k = 8s + 2lk in the first step and k = 8s + 2lk + 1 in the second (both
  // operands use the same assignment, so only the order of the summation changes).  That makes a
  // fragment of both steps one 16-byte LDS read per lane.  The reads are inline assembly so that
  // their place in the instruction stream is fixed: each A fragment of the next pair is requested
  // as soon as the MFMAs that consume the current one have been issued, the two B fragments are
  // double-buffered and requested a whole step ahead, and across a tile boundary the requests go
  // out right after the barrier, under the second step of the last pair.  Every wait carries the
  // registers it covers as operands, which keeps the MFMAs that read them behind it.
  static_assert(TM == 4 && TN == 2 && BK == 16, "the schedule below is written for 64x32 wave tiles");
  uint32_t a_off[2], b_off[2];  // byte offset of this lane's fragment 0 inside a stage, per pair
#pragma unroll
  for (int s2 = 0; s2 < 2; ++s2) {
    const int pr = 4 * s2 + lk;  // pair index = k / 2
    a_off[s2] = 8u * (uint32_t)(A_KC ? frag_lds_kc(wm * WM + lr, pr) : frag_lds_oc128(wm * WM + lr, pr, BM));
    b_off[s2] = 8u * (uint32_t)(B_KC ? frag_lds_kc(wn * WN + lr, pr) : frag_lds_oc128(wn * WN + lr, pr, BN));
  }
  const uint32_t a_base = (uint32_t)(uintptr_t)lds_a, b_base = (uint32_t)(uintptr_t)lds_b;
  v2d fa[4], fb[2][2];  // A fragments (single set), B fragments [buffer][j]
  auto a_addr = [&](int stage, int s2) { return a_base + (uint32_t)stage * (A_SIZE * 8) + a_off[s2]; };
  auto b_addr = [&](int stage, int s2) { return b_base + (uint32_t)stage * (B_SIZE * 8) + b_off[s2]; };
  // fragments of this wavefront's block that reach into the output: rows of 16 and columns of 16
  int tm_live = TM, tn_live = TN;
  if (RAGGED) {
    const LiveFragments live = live_fragments(p.M, p.N, m0 + wm * WM, n0 + wn * WN, TM, TN);
    tm_live = __builtin_amdgcn_readfirstlane(live.rows);
    tn_live = __builtin_amdgcn_readfirstlane(live.cols);
  }
  auto mfma_row = [&](int i, double a, double b0, double b1) {
    if (!RAGGED || i < tm_live) {
      acc[i][0] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b0, acc[i][0], 0, 0, 0);
      if (!RAGGED || tn_live > 1) acc[i][1] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b1, acc[i][1], 0, 0, 0);
    }
  };
  // first step of a pair: the six reads B0 B1 A0 A1 A2 A3 are outstanding in that order
  auto first_step = [&](int bb) {
    asm volatile("s_waitcnt lgkmcnt(3)" : "+v"(fa[0]), "+v"(fb[bb][0]), "+v"(fb[bb][1]));
    mfma_row(0, fa[0].x, fb[bb][0].x, fb[bb][1].x);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(fa[1]));
    mfma_row(1, fa[1].x, fb[bb][0].x, fb[bb][1].x);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt lgkmcnt(1)" : "+v"(fa[2]));
    mfma_row(2, fa[2].x, fb[bb][0].x, fb[bb][1].x);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa[3]));
    mfma_row(3, fa[3].x, fb[bb][0].x, fb[bb][1].x);
    __builtin_amdgcn_sched_barrier(0);
  };
  // second step of a pair, requesting the fragments of pair (stage, s2) meanwhile.  After the
  // last tile the requests fetch stale LDS contents that nobody uses; they are drained below.
  auto second_step = [&](int bb, int stage, int s2) {
    const uint32_t aa = a_addr(stage, s2), ba = b_addr(stage, s2);
    read_quad<B_KC, 0>(fb[bb ^ 1][0], ba);
    read_quad<B_KC, 1>(fb[bb ^ 1][1], ba);
    mfma_row(0, fa[0].y, fb[bb][0].y, fb[bb][1].y);
    __builtin_amdgcn_sched_barrier(0);
    read_quad<A_KC, 0>(fa[0], aa);
    mfma_row(1, fa[1].y, fb[bb][0].y, fb[bb][1].y);
    __builtin_amdgcn_sched_barrier(0);
    read_quad<A_KC, 1>(fa[1], aa);
    mfma_row(2, fa[2].y, fb[bb][0].y, fb[bb][1].y);
    __builtin_amdgcn_sched_barrier(0);
    read_quad<A_KC, 2>(fa[2], aa);
    mfma_row(3, fa[3].y, fb[bb][0].y, fb[bb][1].y);
    __builtin_amdgcn_sched_barrier(0);
    read_quad<A_KC, 3>(fa[3], aa);
  };
  {
    const uint32_t aa = a_addr(0, 0), ba = b_addr(0, 0);
    read_quad<B_KC, 0>(fb[0][0], ba);
    read_quad<B_KC, 1>(fb[0][1], ba);
    read_quad<A_KC, 0>(fa[0], aa);
    read_quad<A_KC, 1>(fa[1], aa);
    read_quad<A_KC, 2>(fa[2], aa);
    read_quad<A_KC, 3>(fa[3], aa);
  }
  int cur = 0, nxt = DIST % STAGES;
  for (int kt = 0; kt < nk; ++kt) {
    if (kt + DIST < nk) issue(nxt);
    if (!A_KC) {
      if (do_colsum) colsum_accumulate<BM, NW * 64>(colsum_partial, lds_a + cur * A_SIZE, tid);
    }
    first_step(0);
    second_step(0, cur, 1);
    first_step(1);  // ends with lgkmcnt(0): this wave's LDS reads of `cur` are done
    // tile kt+1 must have landed: at most DIST-1 younger tiles may still be in flight
    if (kt + DIST < nk) wait_vmcnt((DIST - 1) * 2 * CH); else wait_vmcnt(0);
    __builtin_amdgcn_s_barrier();
    cur = cur + 1 == STAGES ? 0 : cur + 1;
    nxt = nxt + 1 == STAGES ? 0 : nxt + 1;
    second_step(1, cur, 0);
  }
  // the fragment registers stay reserved until the last (unused) requests have returned
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]),
               "+v"(fb[0][0]), "+v"(fb[0][1]), "+v"(fb[1][0]), "+v"(fb[1][1]));
  if (!A_KC) {
    if (do_colsum) colsum_finish<BM, NW * 64>(colsum_partial, lds_b, tid, m0, split, p);
  }

  write_block<TM, TN>(p, &acc[0][0], m0 + wm * WM, n0 + wn * WN, lr, lk, split);
}

template <bool A_KC, bool B_KC, int WGM, int WGN, int STAGES, int DIST>
__global__ __launch_bounds__(WGM * WGN * 64, 4) void gemm_f64_mfma_dma(const GemmParams p) {
  constexpr int A_SIZE = A_KC ? 128 * BK : kDmaStage, B_SIZE = B_KC ? 128 * BK : kDmaStage;
  __shared__ __attribute__((aligned(1024))) double lds_a[STAGES * A_SIZE];
  __shared__ __attribute__((aligned(1024))) double lds_b[STAGES * B_SIZE];
  dma_tile<A_KC, B_KC, WGM, WGN, STAGES, DIST>(p, (int)blockIdx.x, lds_a, lds_b);
}

// Up to kMaxGroup weight gradients with few output tiles each but a long contraction (the batch)
// in one grid of 128x128 direct-to-LDS tiles: every problem is cut into K slices so that together
// they give about one workgroup per CU; workgroups [first_block[i], first_block[i+1]) belong to
// problem i and the shared reduction grid adds the slices up in order.
// (Three LDS stages with two tiles in flight were measured here, since the grid is one workgroup per
// CU: 46.0 us against 44.7 us with two stages on C1's weight gradients - the matrix cores, not the
// trip to memory, set the pace of a K step.)
__global__ __launch_bounds__(512, 4) void gemm_f64_mfma_dma_group(const GemmGroup g) {
  __shared__ __attribute__((aligned(1024))) double lds_a[2 * kDmaStage];
  __shared__ __attribute__((aligned(1024))) double lds_b[2 * kDmaStage];
  const int i = group_member_of_block(g.first_block, g.count, (int)blockIdx.x);
  dma_tile<false, false, 2, 4, 2, 1, true>(g.p[i], (int)blockIdx.x - g.first_block[i], lds_a, lds_b);
}

// ---- 64x64 tiles fed by direct global -> LDS loads ---------------------------------------------
// The mid-size path: products whose 128x128 tiling gives the chip too few workgroups (an 8192 x 100
// output is 64 tiles of 128x128 but 256 of 64x64; a 100 x 784 weight gradient is 7 against 26).
// Four wavefronts of 32x32 (2x2 MFMA tiles each), operand tiles of 64 x 16 doubles (8 KiB) moved by
// global_load_lds_dwordx4 as in the 128x128 kernel, FOUR LDS stages with three tiles in flight (a
// K step is only 16 MFMAs per wavefront, far shorter than a trip to memory, and with one or two
// workgroups per CU nothing else covers it), one barrier per K step.
//   contraction-contiguous operand: [64][16], 16-byte slots XOR-swizzled by row & 7 (as above);
//   output-contiguous operand: [16][64] dense (a 1 KiB wavefront load is two k rows of 64), the
//       16-byte slots of k rows 2g, 2g+1 XOR-ed with 8 * (g & 3): the four lane groups of a fragment
//       read (k rows 2lk, 2lk+1 of a pair) then fall into four different 128-byte windows.
// The contraction indices are assigned to MFMA steps as in the 128x128 kernel (pair s, lane group lk:
// k = 8s + 2lk, then 8s + 2lk + 1).
typedef const __attribute__((address_space(3))) v2d* lds_cv2d_t;
typedef const __attribute__((address_space(3))) double* lds_cf64_t;

constexpr int kT64 = 64;
constexpr int kT64Stage = kT64 * BK;  // doubles per operand and stage
constexpr int kT64Stages = 4;

template <bool KC>
__device__ __forceinline__ void store_tile_dma64(double* __restrict__ lds, const v2d* __restrict__ reg, int tid) {
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int q = tid + u * 256;
    if (KC) {
      const int e = q >> 3, pr = q & 7;
      *reinterpret_cast<v2d*>(lds + frag_lds_kc(e, pr)) = reg[u];
    } else {
      const int kr = q >> 5, cp = q & 31;
      *reinterpret_cast<v2d*>(lds + kr * kT64 + 2 * (cp ^ (8 * ((kr >> 1) & 3)))) = reg[u];
    }
  }
}

// one fragment of one pair of K steps (.x: first step, .y: second) for MFMA tile row/column `e0 + lr`
template <bool KC>
__device__ __forceinline__ v2d read_pair64(uint32_t stage_bytes, int e, int pr) {
  if constexpr (KC) {
    return *(lds_cv2d_t)(uintptr_t)(stage_bytes + 8u * (uint32_t)frag_lds_kc(e, pr));
  } else {
    const uint32_t at = stage_bytes + 8u * (uint32_t)frag_lds_oc64(e, pr);
    v2d r;
    r.x = *(lds_cf64_t)(uintptr_t)at;
    r.y = *(lds_cf64_t)(uintptr_t)(at + 8u * kT64);
    return r;
  }
}

template <bool B_KC>
__global__ __launch_bounds__(256, 2) void gemm_f64_mfma_dma64(const GemmParams p) {
  constexpr bool A_KC = true;  // the forward and input-gradient layouts (where this kernel pays)
  __shared__ __attribute__((aligned(1024))) double lds_a[kT64Stages * kT64Stage];
  __shared__ __attribute__((aligned(1024))) double lds_b[kT64Stages * kT64Stage];
  constexpr int BM = kT64, BN = kT64, NW = 4, TM = 2, TN = 2, CH = 2;
  const int block = (int)blockIdx.x;
  const TileCoord tc = tile_of_block(p.tiles_m, p.tiles_n, block);
  const int split = tc.split;  // K slice of this workgroup (0 without split-K)
  const int tile_m = tc.tile_m, tile_n = tc.tile_n;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int lr = lane & 15, lk = lane >> 4;

  // tile DMA: uniform byte pointer per operand + constant 32-bit lane offsets, uniform LDS targets
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);
  const char* a_ptr = reinterpret_cast<const char*>(p.A + (A_KC ? (size_t)m0 * p.lda : (size_t)m0));
  const char* b_ptr = reinterpret_cast<const char*>(p.B + (B_KC ? (size_t)n0 * p.ldb : (size_t)n0));
  uint32_t ao[CH], bo[CH];
  int lchunk[CH];
#pragma unroll
  for (int h = 0; h < CH; ++h) {
    const int c = wave + NW * h;  // chunk 0..7 of the tile
    lchunk[h] = dma_lds_chunk_kc(wave_s + NW * h);  // (the same for both layouts of this tile size)
    ao[h] = dma_offset_kc<uint32_t>(c, lane, m0, p.M, p.lda);
    if (B_KC) bo[h] = dma_offset_kc<uint32_t>(c, lane, n0, p.N, p.ldb);
    else bo[h] = dma_offset_oc64<uint32_t>(c, lane, n0, p.N, p.ldb);
  }
  const long a_step = dma_k_step_bytes(A_KC, p.lda);
  const long b_step = dma_k_step_bytes(B_KC, p.ldb);

  v4d acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = (v4d){0.0, 0.0, 0.0, 0.0};

  // tiles of this workgroup: [the masked remainder of K (slice 0 only)] + the whole steps of its slice
  const DmaSteps ks = dma_k_steps(p.K, p.split_k, p.steps_per_split, split, p.k_reserve);
  const int nk_all = dma_whole_steps(p.K, p.k_reserve);
  const int kt0 = ks.kt0, nk_dma = ks.nk_dma;
  const bool k_tail = ks.k_tail;
  const int first_dma = k_tail ? 1 : 0;
  const int nk = nk_dma + first_dma;
  a_ptr += (long)kt0 * a_step;
  b_ptr += (long)kt0 * b_step;
  // chunk h of this wavefront's share of a tile, both operands; after the last chunk the pointers move on
  auto issue_chunk = [&](int stage, int h) {
    asm volatile("" : "+v"(ao[h]), "+v"(bo[h]));
    dma16(reinterpret_cast<const double*>(a_ptr + ao[h]), lds_a + stage * kT64Stage + lchunk[h]);
    dma16(reinterpret_cast<const double*>(b_ptr + bo[h]), lds_b + stage * kT64Stage + lchunk[h]);
    if (h == CH - 1) {
      a_ptr += a_step;
      b_ptr += b_step;
    }
  };
  auto issue = [&](int stage) {
#pragma unroll
    for (int h = 0; h < CH; ++h) issue_chunk(stage, h);
  };
  // prologue: tiles 0 .. kT64Stages-1 on their way.  The remainder tile, if any, is tile 0 and goes
  // through registers into stage 0; its masked loads are issued behind the tile DMA of the others, so
  // that all of them are in flight together (one round trip to memory instead of two).
#pragma unroll
  for (int t = 0; t < kT64Stages; ++t)
    if (t >= first_dma && t < nk) issue(t);
  if (k_tail) {
    v2d ra[2], rb[2];
    if (p.unaligned) {  // (uniform over the launch)
      load_tile<BM, A_KC, false, true, 256>(ra, p.A, p.lda, m0, p.M, nk_all * BK, p.K, tid);
      load_tile<BN, B_KC, false, true, 256>(rb, p.B, p.ldb, n0, p.N, nk_all * BK, p.K, tid);
    } else {
      load_tile<BM, A_KC, true, true, 256>(ra, p.A, p.lda, m0, p.M, nk_all * BK, p.K, tid);
      load_tile<BN, B_KC, true, true, 256>(rb, p.B, p.ldb, n0, p.N, nk_all * BK, p.K, tid);
    }
    store_tile_dma64<A_KC>(lds_a, ra, tid);
    store_tile_dma64<B_KC>(lds_b, rb, tid);
  }

  const uint32_t a_base = (uint32_t)(uintptr_t)lds_a, b_base = (uint32_t)(uintptr_t)lds_b;
  const int a_e = wm * 32 + lr, b_e = wn * 32 + lr;  // fragment 0; fragment 1 is 16 further
  // A tile's 16 contraction indices are consumed as two pairs of MFMA steps (pair s2: k = 8 s2 + 2 lk in
  // the first step, 8 s2 + 2 lk + 1 in the second); a fragment of a pair is one 16-byte read per lane.
  auto read_a = [&](int stage, int s2, int i) {
    return read_pair64<A_KC>(a_base + (uint32_t)stage * (kT64Stage * 8), a_e + 16 * i, 4 * s2 + lk);
  };
  auto read_b = [&](int stage, int s2, int j) {
    return read_pair64<B_KC>(b_base + (uint32_t)stage * (kT64Stage * 8), b_e + 16 * j, 4 * s2 + lk);
  };
  v2d pa[TM], pb[TN];  // the fragments of a tile's first pair
  v2d qa[TM], qb[TN];  // of its second pair
  auto mx = [&](const v2d (&fa)[TM], const v2d (&fb)[TN], int i, int j) {
    acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa[i].x, fb[j].x, acc[i][j], 0, 0, 0);
  };
  auto my = [&](const v2d (&fa)[TM], const v2d (&fb)[TN], int i, int j) {
    acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa[i].y, fb[j].y, acc[i][j], 0, 0, 0);
  };
#define RST_FENCE() __builtin_amdgcn_sched_barrier(0)

  // One tile.  With one wavefront per SIMD nothing else fills the matrix cores while this one waits,
  // so everything that is not an MFMA is placed between two of them, one or two instructions at a
  // time (the fences keep the compiler from gathering them): the reads of the second pair under the
  // first pair's MFMAs; the wait for tile kt + 1 and the barrier after the fourth MFMA of the second
  // pair, when all fragments of tile kt are in registers; then, under the last four MFMAs, the reads
  // of tile kt + 1's first pair and the requests for tile kt + 4, which takes the stage of tile kt.
  // STEADY: tiles kt + 1 .. kt + 4 all exist (no tests in the instruction stream).
  auto tile = [&](int kt, auto steady_tag) {
    constexpr bool STEADY = decltype(steady_tag)::value;
    const int stage = kt % kT64Stages, next = (kt + 1) % kT64Stages;
    mx(pa, pb, 0, 0); RST_FENCE();
    qa[0] = read_a(stage, 1, 0); RST_FENCE();
    mx(pa, pb, 0, 1); RST_FENCE();
    qb[0] = read_b(stage, 1, 0); RST_FENCE();
    mx(pa, pb, 1, 0); RST_FENCE();
    qb[1] = read_b(stage, 1, 1); RST_FENCE();
    mx(pa, pb, 1, 1); RST_FENCE();
    qa[1] = read_a(stage, 1, 1); RST_FENCE();
    my(pa, pb, 0, 0); my(pa, pb, 0, 1); my(pa, pb, 1, 0); my(pa, pb, 1, 1); RST_FENCE();
    mx(qa, qb, 0, 0); mx(qa, qb, 0, 1); mx(qa, qb, 1, 0); mx(qa, qb, 1, 1); RST_FENCE();
    const bool more = STEADY || kt + 1 < nk;
    if (more) {
      // tile kt + 1 has landed once at most the younger tiles in flight remain outstanding (4 loads each)
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wavefront's reads of tile kt are over
      if (STEADY) {
        wait_vmcnt(4 * (kT64Stages - 2));
      } else {
        const int younger = nk - 2 - kt < kT64Stages - 2 ? nk - 2 - kt : kT64Stages - 2;
        wait_vmcnt(4 * younger);
      }
      __builtin_amdgcn_s_barrier();  // everybody's share of tile kt + 1 is in LDS; everybody has read tile kt
    }
    RST_FENCE();
    my(qa, qb, 0, 0); RST_FENCE();
    if (more) {
      pa[0] = read_a(next, 0, 0);
      pb[0] = read_b(next, 0, 0);
    }
    RST_FENCE();
    my(qa, qb, 0, 1); RST_FENCE();
    if (more) {
      pb[1] = read_b(next, 0, 1);
      pa[1] = read_a(next, 0, 1);
    }
    RST_FENCE();
    my(qa, qb, 1, 0); RST_FENCE();
    if (STEADY) issue_chunk(stage, 0);
    RST_FENCE();
    my(qa, qb, 1, 1); RST_FENCE();
    if (STEADY) issue_chunk(stage, 1);
    RST_FENCE();
  };
  {
    const int younger = nk - 1 < kT64Stages - 1 ? nk - 1 : kT64Stages - 1;
    wait_vmcnt(4 * younger);
    __syncthreads();
    pa[0] = read_a(0, 0, 0);
    pb[0] = read_b(0, 0, 0);
    pb[1] = read_b(0, 0, 1);
    pa[1] = read_a(0, 0, 1);
  }
  int kt = 0;
  for (; kt + kT64Stages < nk; ++kt) tile(kt, std::true_type{});
  for (; kt < nk; ++kt) tile(kt, std::false_type{});
#undef RST_FENCE
  write_block<TM, TN>(p, &acc[0][0], m0 + wm * 32, n0 + wn * 32, lr, lk, split);
}

// Two independent products in one grid: workgroups [0, first_blocks) work on `first`, the others on
// `second`.  Used for the input gradient of one layer (256 long tiles at C4's hidden width: on its
// own one workgroup per CU) together with the weight gradient of the layer above it (many short
// tiles): the long tiles are dispatched first, the short ones fill the second workgroup slot of
// every CU, so both run at the two-workgroups-per-CU rate.
template <bool A_KC1, bool B_KC1, bool A_KC2, bool B_KC2>
__global__ __launch_bounds__(512, 4) void gemm_f64_mfma_dma_pair(const GemmParams first, const GemmParams second,
                                                                  int first_blocks) {
  __shared__ __attribute__((aligned(1024))) double lds_a[2 * kDmaStage];
  __shared__ __attribute__((aligned(1024))) double lds_b[2 * kDmaStage];
  // Workgroup b goes to XCD b % 8.  The first 2*first_blocks workgroups alternate between the two
  // problems in groups of eight (one per XCD), with the phase flipped every 32 groups, so that the
  // long tiles of `first` spread over the CUs under the usual hand-out orders; tile numbers keep
  // their value mod 8, which the XCD-aware tile walk relies on.  The placement is still the
  // dispatcher's: a CU that ends up with two runs of short tiles (each ending in an SGD epilogue)
  // finishes about 10 % late.
  const PairSlot slot = pair_slot_of_block((int)blockIdx.x, first_blocks);
  if (slot.problem == 0)
    dma_tile<A_KC1, B_KC1, 2, 4, 2, 1>(first, slot.block, lds_a, lds_b);
  else
    dma_tile<A_KC2, B_KC2, 2, 4, 2, 1>(second, slot.block, lds_a, lds_b);
}

// Sum of `count` values `stride` doubles apart, added in order; up to 32 loads are in flight at a
// time (the slices were written by other XCDs, so every load is a trip to memory).
__device__ __forceinline__ double ordered_slice_sum(const double* __restrict__ first, size_t stride, int count) {
  double v = 0.0;
  int s = 0;
  for (; s + 32 <= count; s += 32) {
    double t[32];
#pragma unroll
    for (int j = 0; j < 32; ++j) t[j] = first[(size_t)(s + j) * stride];
#pragma unroll
    for (int j = 0; j < 32; ++j) v += t[j];
  }
  for (; s + 8 <= count; s += 8) {
    double t[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) t[j] = first[(size_t)(s + j) * stride];
#pragma unroll
    for (int j = 0; j < 8; ++j) v += t[j];
  }
  if (s < count) {
    double t[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) t[j] = s + j < count ? first[(size_t)(s + j) * stride] : 0.0;
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (s + j < count) v += t[j];
  }
  return v;
}

// Adds the K slices of a split contraction in slice order and applies the epilogue: workgroup
// `block` (256 threads) of problem p.
__device__ __forceinline__ void split_reduce_body(const GemmParams& p, const size_t block) {
  const size_t mn = (size_t)p.M * p.N;
  const size_t i = block * 256 + threadIdx.x;
  if (i < mn) {
    double v = ordered_slice_sum(p.ws + i, mn, p.split_k);
    const int row = (int)(i / p.N), col = (int)(i - (size_t)row * p.N);
    switch (p.epilogue) {
      case EPI_BIAS: v = v + p.bias[col]; break;
      case EPI_BIAS_RELU: v = fmax(v + p.bias[col], 0.0); break;
      case EPI_RELU: v = fmax(v, 0.0); break;
      case EPI_DIVIDE: v = v / p.divisor; break;
      case EPI_MASK: v = v * (p.mask[(size_t)row * p.ldmask + col] > 0.0 ? 1.0 : 0.0); break;
      default: break;
    }
    p.C[(size_t)row * p.ldc + col] = v;
    if (p.sgd_parm) {
      double* w = p.sgd_parm + (size_t)row * p.ldc + col;
      *w = sgd_apply(*w, v, p.sgd_lr);
    }
  }
  if (p.colsum != nullptr && i < (size_t)p.M) {
    const double t = ordered_slice_sum(p.ws_colsum + i, (size_t)p.M, p.split_k);
    const double g = t / p.colsum_div;
    p.colsum[i] = g;
    if (p.sgd_bias) p.sgd_bias[i] = sgd_apply(p.sgd_bias[i], g, p.sgd_lr);
  }
}

__global__ __launch_bounds__(256) void split_reduce_kernel(const GemmParams p) {
  split_reduce_body(p, blockIdx.x);
}

__global__ __launch_bounds__(256) void split_reduce_group_kernel(const GemmGroup g) {
  const int i = group_member_of_block(g.first_reduce_block, g.count, (int)blockIdx.x);
  split_reduce_body(g.p[i], (size_t)((int)blockIdx.x - g.first_reduce_block[i]));
}

int launch_split_reduce(hipStream_t stream, const GemmParams& p) {
  const size_t mn = (size_t)p.M * p.N;
  RST_OBSERVE_GEMM(GemmKernel::kSplitReduce, 0, 0, 0, 0, false, false, false, 0, (long long)((mn + 255) / 256), 256, &p, nullptr, 0, nullptr);
  hipLaunchKernelGGL(split_reduce_kernel, dim3((unsigned)((mn + 255) / 256)), dim3(256), 0, stream, p);
  RST_HIP(hipGetLastError());
  return RST_OK;
}

constexpr int kSplitMinSteps = 1536;  // K >= 24576

int compute_units() {
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    return n;
  }();
  return cus;
}

// want_split > 1: cut K into that many slices (the caller has checked the workspace)
template <bool A_KC, bool B_KC>
int launch_dma(hipStream_t stream, GemmParams p, int want_split = 0) {
  p.tiles_m = (p.M + 127) / 128;
  p.tiles_n = (p.N + 127) / 128;
  p.split_k = 1;
  p.steps_per_split = dma_whole_steps(p.K, p.k_reserve);
  long long blocks = (long long)p.tiles_m * p.tiles_n;
  // Two independent workgroups per compute unit interleave their barriers and LDS waits: measured
  // on 256 tiles, the K loop runs about 1.5 points of the MFMA peak faster with two than with one.
  // With fewer than 512 tiles K can be cut in two halves so that every CU gets two workgroups;
  // the two partial products are then added (in slice order) by split_reduce_kernel, a fixed cost
  // of about 30 us per launch at 1024 x 4096 outputs: level at K = 16384 (1838 us unsplit, 1847
  // split), 0.5 % ahead at K = 32768.
  const int nk = dma_whole_steps(p.K, p.k_reserve);
  const size_t need = 2 * ((size_t)p.M * p.N + (size_t)p.M);
  if (want_split > 1) {
    p.steps_per_split = (nk + want_split - 1) / want_split;
    p.split_k = (nk + p.steps_per_split - 1) / p.steps_per_split;
    p.ws_colsum = p.ws + (size_t)p.split_k * p.M * p.N;
    blocks *= p.split_k;
  } else if (blocks < 512 && nk >= kSplitMinSteps && p.ws != nullptr && p.ws_capacity >= need) {
    p.split_k = 2;
    p.steps_per_split = (nk + 1) / 2;
    p.ws_colsum = p.ws + (size_t)2 * p.M * p.N;
    blocks *= 2;
  }
  if (blocks > 0x7fffffffLL) return fail(RST_ERR_UNSUPPORTED, "contraction grid too large");
  // more than one round of workgroups (two per CU fit): stagger the first round by 0.4 us per K step
  p.first_round = 2 * compute_units();
  p.dephase_ticks = blocks > p.first_round ? (p.steps_per_split < 250 ? 40 * p.steps_per_split : 10000) : 0;
  RST_OBSERVE_GEMM(GemmKernel::kDma128, 128, 128, 2, 4, A_KC, B_KC, p.unaligned == 0, 0, blocks, 512, &p, nullptr, 0, nullptr);
  hipLaunchKernelGGL((gemm_f64_mfma_dma<A_KC, B_KC, 2, 4, 2, 1>), dim3((unsigned)blocks),
                     dim3(512), 0, stream, p);
  RST_HIP(hipGetLastError());
  if (p.split_k > 1) RST_TRY(launch_split_reduce(stream, p));
  return RST_OK;
}

// 64x64 direct-to-LDS tiles, optionally on `slices` K slices (the caller has checked the workspace)
template <bool B_KC>
int launch_dma64(hipStream_t stream, GemmParams p, int slices) {
  p.tiles_m = (p.M + kT64 - 1) / kT64;
  p.tiles_n = (p.N + kT64 - 1) / kT64;
  const int nk = dma_whole_steps(p.K, p.k_reserve);
  p.split_k = 1;
  p.steps_per_split = nk;
  long long blocks = (long long)p.tiles_m * p.tiles_n;
  if (slices > 1) {
    p.steps_per_split = (nk + slices - 1) / slices;
    p.split_k = (nk + p.steps_per_split - 1) / p.steps_per_split;
    if (p.split_k > 1) {
      p.ws_colsum = p.ws + (size_t)p.split_k * p.M * p.N;
      blocks *= p.split_k;
    }
  }
  if (blocks > 0x7fffffffLL) return fail(RST_ERR_UNSUPPORTED, "contraction grid too large");
  RST_OBSERVE_GEMM(GemmKernel::kDma64, 64, 64, 2, 2, true, B_KC, p.unaligned == 0, 0, blocks, 256, &p, nullptr, 0, nullptr);
  hipLaunchKernelGGL((gemm_f64_mfma_dma64<B_KC>), dim3((unsigned)blocks), dim3(256), 0, stream, p);
  RST_HIP(hipGetLastError());
  if (p.split_k > 1) RST_TRY(launch_split_reduce(stream, p));
  return RST_OK;
}

// Few output tiles (`blocks` < split_below) but a long contraction: the number of K slices that
// fills the chip (want_blocks workgroups, about eight per CU), 1 = none.
long long small_tile_slices(const GemmParams& p, long long blocks, long long split_below, long long want_blocks) {
  const int nk = (p.K + BK - 1) / BK;
  if (!(blocks < split_below && nk >= 8 && p.ws != nullptr)) return 1;
  long long want = (want_blocks + blocks - 1) / blocks;
  if (want > 64) want = 64;                                // keep the ordered reduction short
  const long long max_by_steps = nk / 4;                   // at least 4 K steps per slice
  const long long max_by_ws = (long long)(p.ws_capacity / ((size_t)p.M * p.N + (size_t)p.M));
  long long s = want < max_by_steps ? want : max_by_steps;
  if (s > max_by_ws) s = max_by_ws;
  return s > 1 ? s : 1;
}

// 32x32 tiles on at most one workgroup per CU: K steps are fetched eight at a time (gemm_tile)
constexpr int kBurst = 8;
// 32x32 tiles are cut into K slices while they give fewer than two workgroups per CU (a 1024 x 256
// output at K = 4096, 256 tiles: 110 us unsplit, one chain of 256 K steps per workgroup)
constexpr long long kSmallTileSplitBelow = 512;

// Fills in split_k, steps_per_split and ws_colsum of a small-tile launch of `blocks` output tiles.
void plan_slices(GemmParams& p, long long blocks, long long split_below, long long want_blocks) {
  const int nk = (p.K + BK - 1) / BK;
  p.split_k = 1;
  p.steps_per_split = nk;
  const long long s = small_tile_slices(p, blocks, split_below, want_blocks);
  if (s > 1) {
    p.steps_per_split = (int)((nk + s - 1) / s);
    p.split_k = (nk + p.steps_per_split - 1) / p.steps_per_split;
    p.ws_colsum = p.ws + (size_t)p.split_k * p.M * p.N;
  }
}

template <int BM, int BN, int WGM, int WGN, bool A_KC, bool B_KC, bool VEC>
int launch_one(hipStream_t stream, GemmParams p, long long split_below = 256, long long want_blocks = 2048) {
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  long long blocks = (long long)p.tiles_m * p.tiles_n;
  plan_slices(p, blocks, split_below, want_blocks);
  blocks *= p.split_k;
  if (blocks > 0x7fffffffLL) return fail(RST_ERR_UNSUPPORTED, "contraction grid too large");
  const bool burst = BM == 32 && BN == 32 && blocks <= compute_units();
  RST_OBSERVE_GEMM(GemmKernel::kStaged, BM, BN, WGM, WGN, A_KC, B_KC, VEC, burst ? kBurst : 0, blocks, WGM * WGN * 64, &p, nullptr, 0, nullptr);
  if (burst)
    hipLaunchKernelGGL((gemm_f64_mfma<BM, BN, WGM, WGN, A_KC, B_KC, VEC, (BM == 32 ? kBurst : 0)>),
                       dim3((unsigned)blocks), dim3(WGM * WGN * 64), 0, stream, p);
  else
    hipLaunchKernelGGL((gemm_f64_mfma<BM, BN, WGM, WGN, A_KC, B_KC, VEC>), dim3((unsigned)blocks),
                       dim3(WGM * WGN * 64), 0, stream, p);
  RST_HIP(hipGetLastError());
  if (p.split_k > 1) RST_TRY(launch_split_reduce(stream, p));
  return RST_OK;
}

// Which kernel a product goes to.  128x128 tiles once they fill the 256 compute units; below that
// the direct-to-LDS kernels on K slices or 64x64 tiles where the measured rules below say so, else
// register-staged 32x32 tiles (which cut the contraction into slices when that gives too few
// workgroups).
enum class Route { kDma, kDmaSliced, kDma64, kTile128, kTile32 };

// RSTORCH_DMA64: "0" never routes to the 64x64 direct-to-LDS kernel, "1" routes every eligible
// product there (for measurements); unset: the measured rule in choose_route.
int dma64_mode() {
  static const int mode = [] {
    const char* v = std::getenv("RSTORCH_DMA64");
    if (v && v[0] == '0') return 0;
    if (v && v[0] == '1') return 1;
    return -1;
  }();
  return mode;
}

// K slices (1 = none) for a product of 257..511 tiles of 128x128, by a cost model in microseconds fitted
// to this part: 512 workgroups in flight (two per CU) advance one K step in 3.65 us, up to 256 (one per
// CU) in 1.95 us, later workgroups start as earlier ones leave; the reduction of s slices moves
// (2 s + 1) M N doubles at 4.5 TB/s behind a launch of 8 us.  Constants, not the device's own counts:
// the number of slices fixes the order of the summation, which must not change from device to device.
int band_slices(const GemmParams& p, long long t128) {
  const int nk = dma_whole_steps(p.K, p.k_reserve);
  auto cost = [&](int s) {
    const int steps = (nk + s - 1) / s;
    const long long wgs = t128 * s, full = wgs / 512, rem = wgs % 512;
    double c = (double)full * 3.65 * steps;
    if (rem > 256) c += 3.65 * steps;
    else if (rem > 0) c += 1.95 * steps;
    if (s > 1) c += 8.0 + (2.0 * s + 1.0) * (double)p.M * (double)p.N * 8.0 / 4.5e6;
    return c;
  };
  int best = 1;
  double best_cost = cost(1);
  for (int s = 2; s <= 4; ++s) {
    if (nk / s < 32 || p.ws_capacity < (size_t)s * ((size_t)p.M * p.N + (size_t)p.M)) break;
    const double c = cost(s);
    if (c < 0.95 * best_cost) {  // (a slice more has to pay for itself by a margin)
      best = s;
      best_cost = c;
    }
  }
  return best;
}

Route choose_route(const GemmParams& p, int* dma_slices, bool is_a_kc = false, bool is_b_kc = false) {
  auto tiles = [&](int bm, int bn) {
    return (long long)((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn);
  };
  // (leading dimensions below 2^22 doubles keep the 32-bit lane offsets of the tile DMA in range;
  // the tile DMA needs no more than the 8-byte alignment every operand has)
  const bool dma_ok = p.K > 0 && p.M >= 2 && p.N >= 2 && p.lda < (1L << 22) && p.ldb < (1L << 22);
  const long long t128 = tiles(128, 128);
  *dma_slices = 0;
  if (t128 >= 256) {
    if (!dma_ok) return Route::kTile128;
    // Forward products of 257..511 tiles: two workgroups fit on a CU, so all tiles start at once, the CUs
    // that got two finish in twice the time of those that got one, and the launch takes as long as 512
    // tiles would (1024 x 4608 at K = 4096, 288 tiles: 907 us, 54 % of the MFMA peak).  K slices make the
    // pieces small enough to even that out, at the price of the partial results and their reduction.
    if (is_a_kc && is_b_kc && t128 > 256 && t128 < 512 && p.ws != nullptr) {
      const int s = band_slices(p, t128);
      if (s > 1) {
        *dma_slices = s;
        return Route::kDmaSliced;
      }
    }
    return Route::kDma;
  }
  // 32..255 tiles of 128x128 with a long contraction: the direct-to-LDS kernel on up to eight K
  // slices (about two workgroups per CU, at least 32 K steps each) plus the ordered reduction
  // beats the smaller register-staged tiles by far (128 tiles, K = 4096: 87 % of the MFMA peak
  // against 62 %), as long as the slices still fill the chip.
  int s128 = 0;       // its slices, 0 = not taken
  bool multi_round = false;
  if (dma_ok && p.ws != nullptr) {
    const int nk = dma_whole_steps(p.K, p.k_reserve);
    auto fits = [&](int s) { return p.ws_capacity >= (size_t)s * ((size_t)p.M * p.N + (size_t)p.M); };
    int s = (int)((512 + t128 - 1) / t128);
    if (s > 8) s = 8;
    while (s > 1 && (nk / s < 32 || !fits(s))) --s;
    multi_round = s > 1 && t128 * s >= 256;
    if (!multi_round) {
      // a shorter contraction: one round of workgroups (at most one per CU, at least three CUs in
      // four busy) on slices of 12 K steps or more still beats the register-staged small tiles
      // (8192 x 100 x 784 on 64 tiles: 39 us on four slices against 47 us); a round and a bit
      // does not (64 tiles on five slices: 70 us against 60 us)
      s = (int)(256 / t128);
      if (s > 8) s = 8;
      if (!(s > 1 && t128 * s >= 192 && nk / s >= 12 && fits(s))) s = 1;
    }
    s128 = s > 1 ? s : 0;
  }
  // 64x64 direct-to-LDS tiles (forward and input-gradient layouts): one workgroup per CU or more on
  // slices of at least eight K steps.  The rule below is fitted to a sweep of 386 mid-size shapes
  // (batch 128..16384, widths 64..4096), each timed with this route forced and with it off:
  //   * never below 192 workgroups, and never against several rounds of long 128x128 slices
  //     (contractions above 2048) - there the 128x128 kernel is ahead;
  //   * always where a dimension of 64 or less leaves the 128-wide tiles half empty (up to 40 %);
  //   * forward products otherwise whenever the slices are either not needed (four K steps are
  //     enough), or at least four, or at least 24 steps long: 5-28 % ahead of the 32x32 tiles and
  //     of one round of 128x128 slices (two slices of 8-16 steps lose 15-50 %); the rule picks
  //     within 0.6 % (geometric mean) of the better of the two routes, 10 % at worst;
  //   * input gradients of at least 2.5e8 flops with a contraction of up to 4096 on slices of 24 steps
  //     or more (12 unsliced): 5-24 % ahead on rst_linear_backward as a whole; smaller ones stay on the
  //     32x32 tiles, where they share a grid with their layer's weight gradient, which is worth more
  //     than the faster kernel.
  if (dma_ok && dma64_mode() != 0 && is_a_kc) {
    const long long t64 = tiles(64, 64);
    const int nk = dma_whole_steps(p.K, p.k_reserve);
    long long s = t64 >= 256 ? 1 : (256 + t64 - 1) / t64;
    if (s > 32) s = 32;
    while (s > 1 && nk / s < 8) --s;
    const bool fits = s == 1 || (p.ws != nullptr && p.ws_capacity >= (size_t)s * ((size_t)p.M * p.N + (size_t)p.M));
    const long long steps = nk / s;
    const double flops = 2.0 * p.M * p.N * (double)p.K;
    const double area128 = (double)t128 * 128.0 * 128.0, area64 = (double)t64 * 64.0 * 64.0;
    bool take = dma64_mode() == 1 && t64 * s >= 128 && nk >= 1;
    if (dma64_mode() != 1 && t64 * s >= 192) {
      const bool half_empty = area128 >= 1.4 * area64 && steps >= 12;
      if (is_b_kc) {
        const bool slices_ok = s == 1 ? steps >= 4 : (steps >= 8 && nk >= 32 && (s >= 4 || steps >= 24));
        take = half_empty || (multi_round ? nk <= 128 : (slices_ok && (s128 <= 1 || nk <= 128)));
      } else {
        const bool long_enough = nk <= 256 && (s == 1 ? steps >= 12 : steps >= 24);
        take = flops >= 2.5e8 && (half_empty || long_enough);
      }
    }
    if (take && fits) {
      *dma_slices = (int)s;
      return Route::kDma64;
    }
  }
  if (s128 > 1) {
    *dma_slices = s128;
    return Route::kDmaSliced;
  }
  // (register-staged 64x64 tiles have no place here: 1024 of them would mean 256 tiles of 128x128)
  return Route::kTile32;
}

template <bool A_KC, bool B_KC, bool VEC>
int launch_layout(hipStream_t stream, const GemmParams& p) {
  int slices = 0;
  switch (choose_route(p, &slices, A_KC, B_KC)) {
    case Route::kDma: return launch_dma<A_KC, B_KC>(stream, p);
    case Route::kDmaSliced: return launch_dma<A_KC, B_KC>(stream, p, slices);
    case Route::kDma64:
      if constexpr (A_KC) return launch_dma64<B_KC>(stream, p, slices);
      else return fail(RST_ERR_UNSUPPORTED, "no 64x64 direct-to-LDS kernel for this layout");
    case Route::kTile128: return launch_one<128, 128, 2, 4, A_KC, B_KC, VEC>(stream, p);
    default: return launch_one<32, 32, 2, 2, A_KC, B_KC, VEC>(stream, p, kSmallTileSplitBelow);
  }
}

}  // namespace

namespace {

// 16-byte register loads need both operands aligned with even leading dimensions and extents;
// launches on other operands load singly (GemmParams::unaligned)
bool desc_vec_ok(const GemmDesc& d) {
  auto ok = [](const double* ptr, long ld, int contiguous_extent) {
    return (reinterpret_cast<uintptr_t>(ptr) % 16 == 0) && (ld % 2 == 0) &&
           (contiguous_extent % 2 == 0);
  };
  return ok(d.A, d.lda, d.a_kc ? d.K : d.M) && ok(d.B, d.ldb, d.b_kc ? d.K : d.N);
}

GemmParams make_params(const GemmDesc& d) {
  GemmParams p;
  p.A = d.A; p.B = d.B; p.C = d.C;
  p.M = d.M; p.N = d.N; p.K = d.K;
  p.lda = d.lda; p.ldb = d.ldb; p.ldc = d.ldc;
  p.epilogue = d.epilogue;
  p.bias = d.bias; p.divisor = d.divisor; p.mask = d.mask; p.ldmask = d.ldmask;
  {
    // a power of two whose reciprocal is a normal number: x * (1 / d) and x / d are then the same
    // correctly rounded value for every x
    int exponent = 0;
    const double mantissa = std::frexp(d.divisor, &exponent);
    p.divisor_reciprocal = (std::fabs(mantissa) == 0.5 && exponent > -1000 && exponent < 1000) ? 1.0 / d.divisor : 0.0;
  }
  p.colsum = (!d.a_kc) ? d.colsum : nullptr;
  p.colsum_div = d.colsum_div;
  p.sgd_parm = (d.epilogue == EPI_DIVIDE) ? d.sgd_parm : nullptr;
  p.sgd_bias = p.colsum ? d.sgd_bias : nullptr;
  p.sgd_lr = d.sgd_lr;
  p.split_k = 1; p.steps_per_split = 0;
  p.ws = d.workspace; p.ws_colsum = nullptr; p.ws_capacity = d.workspace ? d.workspace_count : 0;
  p.tiles_m = p.tiles_n = 0;
  p.dephase_ticks = 0; p.first_round = 0;
  p.unaligned = desc_vec_ok(d) ? 0 : 1;
  p.k_reserve = ((!d.a_kc && d.M % 2 != 0) || (!d.b_kc && d.N % 2 != 0)) ? 1 : 0;
  return p;
}

// true when launch_gemm would run d as unsplit 128x128 direct-to-LDS tiles
bool takes_plain_dma(const GemmDesc& d, long long* blocks) {
  if (d.M < 2 || d.N < 2 || d.K <= 0) return false;
  if (d.lda >= (1L << 22) || d.ldb >= (1L << 22)) return false;
  *blocks = (long long)((d.M + 127) / 128) * ((d.N + 127) / 128);
  if (*blocks < 256) return false;
  const GemmParams p = make_params(d);
  return !(*blocks < 512 && dma_whole_steps(p.K, p.k_reserve) >= kSplitMinSteps && d.workspace != nullptr);
}

}  // namespace

int launch_gemm(hipStream_t stream, const GemmDesc& d) {
  if (d.M <= 0 || d.N <= 0) return RST_OK;
  const GemmParams p = make_params(d);
  const bool vec = desc_vec_ok(d);
  if (d.a_kc && d.b_kc)
    return vec ? launch_layout<true, true, true>(stream, p) : launch_layout<true, true, false>(stream, p);
  if (!d.a_kc && !d.b_kc)
    return vec ? launch_layout<false, false, true>(stream, p) : launch_layout<false, false, false>(stream, p);
  if (d.a_kc && !d.b_kc)
    return vec ? launch_layout<true, false, true>(stream, p) : launch_layout<true, false, false>(stream, p);
  return vec ? launch_layout<false, true, true>(stream, p) : launch_layout<false, true, false>(stream, p);
}

int max_gemm_group() { return kMaxGroup; }

namespace {
// the slices of a group member: what launch_gemm would choose for it alone
void plan_group_member(GemmParams& p) {
  p.tiles_m = (p.M + 31) / 32;
  p.tiles_n = (p.N + 31) / 32;
  plan_slices(p, (long long)p.tiles_m * p.tiles_n, kSmallTileSplitBelow, 2048);
}
}  // namespace

bool can_group_gemm(const GemmDesc& d) {
  if (d.M <= 0 || d.N <= 0) return false;
  const GemmParams p = make_params(d);
  int slices = 0;
  return choose_route(p, &slices, d.a_kc, d.b_kc) == Route::kTile32;
}

namespace {
// RSTORCH_DMA_GROUP: "0" keeps every group on the 32x32 kernels, "1" sends every eligible group
// to the sliced 128x128 kernel (for measurements); unset: the rule in plan_dma_group.
int dma_group_mode() {
  static const int mode = [] {
    const char* v = std::getenv("RSTORCH_DMA_GROUP");
    if (v && v[0] == '0') return 0;
    if (v && v[0] == '1') return 1;
    return -1;
  }();
  return mode;
}

constexpr int kDmaGroupMaxSlices = 32;
constexpr int kDmaGroupMinSteps = 8;
// The grid the planner aims at: one workgroup for each of the 256 compute units of the part.  A
// constant, not the device's own count: the number of slices fixes the order in which a weight
// gradient is summed, and results must not change with the number of CUs a device exposes.
constexpr int kDmaGroupGrid = 256;

// a weight gradient that the sliced 128x128 group kernel can take at all: at most eight output
// tiles (more have enough workgroups of their own, and the slices of a larger output would crowd
// the shared workspace)
bool dma_group_member(const GemmDesc& d) {
  return !d.a_kc && !d.b_kc && d.K / BK >= 2 * kDmaGroupMinSteps && d.M >= 2 && d.N >= 2 &&
         (long long)((d.M + 127) / 128) * ((d.N + 127) / 128) <= 8 && d.lda < (1L << 22) && d.ldb < (1L << 22) &&
         d.workspace != nullptr;
}

// MFMAs per K step of 4 that the busiest SIMD of a 128x128 workgroup issues when only me x ne of its
// outputs exist (the kernel skips fragments beyond the edge): wavefronts w and w + 4 share a SIMD.
// 16 for a full tile.
int ragged_tile_cost(int me, int ne) {
  int worst = 0;
  for (int simd = 0; simd < 4; ++simd) {
    int c = 0;
    for (int w = simd; w < 8; w += 4) {
      const LiveFragments live = live_fragments(me, ne, (w / 4) * 64, (w % 4) * 32, 4, 2);
      c += live.rows * live.cols;
    }
    if (c > worst) worst = c;
  }
  return worst;
}

// Plans d[0..count) as one grid of K-sliced 128x128 tiles of about one workgroup per CU (two per CU
// measured 4 % slower on the step).  The kernel skips the MFMA fragments beyond a tile's edge, so a
// tile costs what its busiest SIMD issues (ragged_tile_cost); a member is cut into as many slices as
// its cost says, so that all workgroups of the grid take about equally long, and the narrow last tile
// column of a member (784 = 6 x 128 + 16) becomes a piece of its own with fewer, longer slices.
// False when the members do not qualify, the tiles would be mostly padding, the grid would leave more
// than a quarter of the chip idle (batches below about 4096 for a handful of tiles), or the
// workspace is too small.  *ws_need: doubles of the shared workspace that the plan takes.
bool plan_dma_group(const GemmDesc* d, int count, GemmGroup* g, long long* blocks_out, long long* reduce_out,
                    size_t* ws_need = nullptr) {
  if (dma_group_mode() == 0) return false;
  long long tiles = 0;
  double outputs = 0.0;
  for (int i = 0; i < count; ++i) {
    if (!dma_group_member(d[i])) return false;
    tiles += (long long)((d[i].M + 127) / 128) * ((d[i].N + 127) / 128);
    outputs += (double)d[i].M * d[i].N;
  }
  if (tiles > kDmaGroupGrid / 8) return false;
  // Measured on whole training steps of small networks at batch 8192: with 61 % of the 128x128
  // tiles' area in use (784-100-100-10) the step is 6 % shorter than on the 32x32 group (13 % at
  // batch 32768), with 90 % (256-256-256-10) 7 %; with 41 % (1024-64-64-64-16) it is 9 % longer.
  if (dma_group_mode() != 1 && outputs < 0.55 * 16384.0 * (double)tiles) return false;
  // the pieces: every member, minus a cheap last tile column that goes on its own
  GemmDesc piece[kMaxGroup];
  int cost[kMaxGroup];
  int pieces = 0;
  for (int i = 0; i < count; ++i) {
    const GemmDesc& m = d[i];
    const int me = m.M < 128 ? m.M : 128;
    const int rem = m.N % 128;
    const int spare = kMaxGroup - pieces - (count - i);  // slots left once every later member has one
    if (m.N > 128 && rem != 0 && spare >= 1 && 2 * ragged_tile_cost(me, rem) <= ragged_tile_cost(me, 128)) {
      GemmDesc head = m, tail = m;
      head.N = m.N - rem;
      tail.N = rem;
      tail.B = m.B + head.N;  // both operands of a weight gradient are output-contiguous: a column offset
      tail.C = m.C + head.N;
      if (m.sgd_parm) tail.sgd_parm = m.sgd_parm + head.N;
      tail.colsum = nullptr;  // the column sums of A belong to the piece that holds tile column 0
      tail.sgd_bias = nullptr;
      cost[pieces] = ragged_tile_cost(me, 128);
      piece[pieces++] = head;
      cost[pieces] = ragged_tile_cost(me, rem);
      piece[pieces++] = tail;
    } else {
      cost[pieces] = ragged_tile_cost(me, m.N < 128 ? m.N : 128);
      piece[pieces++] = m;
    }
  }
  int cost_max = 1;
  double weight = 0.0;
  for (int i = 0; i < pieces; ++i) {
    // a K step costs a workgroup at least its barrier and the wait for the next tile, about what
    // six MFMAs per SIMD take (measured: 0.8 us against 2.2 us for a full tile's sixteen)
    if (cost[i] < 6) cost[i] = 6;
    if (cost[i] > cost_max) cost_max = cost[i];
    weight += (double)cost[i] * (double)(((piece[i].M + 127) / 128) * ((piece[i].N + 127) / 128));
  }
  const double full_slices = (double)kDmaGroupGrid * (double)cost_max / weight;  // of a piece of the highest cost
  long long blocks = 0, reduce_blocks = 0;
  size_t ws_used = 0;
  g->count = pieces;
  for (int i = 0; i < pieces; ++i) {
    GemmParams p = make_params(piece[i]);
    p.tiles_m = (p.M + 127) / 128;
    p.tiles_n = (p.N + 127) / 128;
    const int nk = dma_whole_steps(p.K, p.k_reserve);
    long long s = (long long)(full_slices * (double)cost[i] / (double)cost_max + 0.5);
    if (s > kDmaGroupMaxSlices) s = kDmaGroupMaxSlices;
    if (s > nk / kDmaGroupMinSteps) s = nk / kDmaGroupMinSteps;
    if (s < 2) s = 2;
    if (nk / s < 1) return false;
    p.steps_per_split = (int)((nk + s - 1) / s);
    p.split_k = (nk + p.steps_per_split - 1) / p.steps_per_split;
    if (p.split_k < 2) return false;
    const size_t need = (size_t)p.split_k * ((size_t)p.M * p.N + (size_t)p.M);
    if (ws_used + need > p.ws_capacity) return false;
    p.ws += ws_used;
    p.ws_colsum = p.ws + (size_t)p.split_k * p.M * p.N;
    ws_used += need;
    g->first_block[i] = (int)blocks;
    g->first_reduce_block[i] = (int)reduce_blocks;
    g->layout[i] = 0;
    blocks += (long long)p.tiles_m * p.tiles_n * p.split_k;
    reduce_blocks += (long long)(((size_t)p.M * p.N + 255) / 256);
    g->p[i] = p;
  }
  g->first_block[pieces] = (int)blocks;
  g->first_reduce_block[pieces] = (int)reduce_blocks;
  if (dma_group_mode() != 1 && blocks < (3 * kDmaGroupGrid) / 4) return false;
  *blocks_out = blocks;
  *reduce_out = reduce_blocks;
  if (ws_need) *ws_need = ws_used;
  return true;
}
}  // namespace

// What launch_gemm_group(d, count) will take from the workspace the descriptors share: the need of
// the sliced 128x128 grid when the group as a whole qualifies for it, else the sum over the members'
// own 32x32 slice plans.
size_t gemm_group_workspace(const GemmDesc* d, int count) {
  if (count >= 1 && count <= kMaxGroup) {
    GemmGroup g{};
    long long blocks = 0, reduce_blocks = 0;
    size_t need = 0;
    if (plan_dma_group(d, count, &g, &blocks, &reduce_blocks, &need)) return need;
  }
  size_t need = 0;
  for (int i = 0; i < count; ++i) {
    GemmParams p = make_params(d[i]);
    plan_group_member(p);
    if (p.split_k > 1) need += (size_t)p.split_k * ((size_t)p.M * p.N + (size_t)p.M);
  }
  return need;
}

int launch_gemm_group(hipStream_t stream, const GemmDesc* d, int count) {
  if (count < 1 || count > kMaxGroup) return fail(RST_ERR_INVALID_ARGUMENT, "a group holds 1..%d contractions", kMaxGroup);
  GemmGroup g{};
  long long blocks = 0, reduce_blocks = 0;
  for (int i = 0; i < count; ++i)
    if (d[i].workspace != d[0].workspace || d[i].workspace_count != d[0].workspace_count)
      return fail(RST_ERR_INVALID_ARGUMENT, "the contractions of a group share one workspace");
  if (plan_dma_group(d, count, &g, &blocks, &reduce_blocks)) {
    RST_OBSERVE_GEMM(GemmKernel::kDma128Group, 128, 128, 2, 4, false, false, true, 0, blocks, 512, nullptr, nullptr, 0, &g);
    hipLaunchKernelGGL(gemm_f64_mfma_dma_group, dim3((unsigned)blocks), dim3(512), 0, stream, g);
    RST_HIP(hipGetLastError());
    RST_OBSERVE_GEMM(GemmKernel::kSplitReduceGroup, 0, 0, 0, 0, false, false, false, 0, reduce_blocks, 256, nullptr, nullptr, 0, &g);
    hipLaunchKernelGGL(split_reduce_group_kernel, dim3((unsigned)reduce_blocks), dim3(256), 0, stream, g);
    RST_HIP(hipGetLastError());
    return RST_OK;
  }
  g = GemmGroup{};
  g.count = count;
  blocks = reduce_blocks = 0;
  size_t ws_used = 0;
  bool mixed = false;  // anything but weight-gradient layouts
  for (int i = 0; i < count; ++i) {
    if (!can_group_gemm(d[i])) return fail(RST_ERR_INVALID_ARGUMENT, "contraction %d cannot join a group", i);
    GemmParams p = make_params(d[i]);
    plan_group_member(p);
    g.first_block[i] = (int)blocks;
    g.first_reduce_block[i] = (int)reduce_blocks;
    g.layout[i] = (unsigned char)((d[i].a_kc ? 1 : 0) | (d[i].b_kc ? 2 : 0));
    mixed = mixed || g.layout[i] != 0;
    blocks += (long long)p.tiles_m * p.tiles_n * p.split_k;
    if (p.split_k > 1) {
      // every problem gets a region of its own in the shared workspace
      const size_t need = (size_t)p.split_k * ((size_t)p.M * p.N + (size_t)p.M);
      if (ws_used + need > p.ws_capacity) return fail(RST_ERR_INVALID_ARGUMENT, "group workspace exhausted");
      p.ws += ws_used;
      p.ws_colsum = p.ws + (size_t)p.split_k * p.M * p.N;
      ws_used += need;
      reduce_blocks += (long long)(((size_t)p.M * p.N + 255) / 256);
    }
    g.p[i] = p;
  }
  if (blocks > 0x7fffffffLL || reduce_blocks > 0x7fffffffLL) return fail(RST_ERR_UNSUPPORTED, "contraction grid too large");
  g.first_block[count] = (int)blocks;
  g.first_reduce_block[count] = (int)reduce_blocks;
  const bool burst = blocks <= compute_units();
  RST_OBSERVE_GEMM(mixed ? GemmKernel::kStagedMixedGroup : GemmKernel::kStagedGroup, 32, 32, 2, 2, false, false, true,
                   burst ? kBurst : 0, blocks, 256, nullptr, nullptr, 0, &g);
  if (mixed && burst)
    hipLaunchKernelGGL((gemm_f64_mfma_mixed_group<kBurst>), dim3((unsigned)blocks), dim3(256), 0, stream, g);
  else if (mixed)
    hipLaunchKernelGGL((gemm_f64_mfma_mixed_group<0>), dim3((unsigned)blocks), dim3(256), 0, stream, g);
  else if (burst)
    hipLaunchKernelGGL((gemm_f64_mfma_group<false, false, kBurst>), dim3((unsigned)blocks), dim3(256), 0, stream, g);
  else
    hipLaunchKernelGGL((gemm_f64_mfma_group<false, false, 0>), dim3((unsigned)blocks), dim3(256), 0, stream, g);
  RST_HIP(hipGetLastError());
  if (reduce_blocks > 0) {
    RST_OBSERVE_GEMM(GemmKernel::kSplitReduceGroup, 0, 0, 0, 0, false, false, false, 0, reduce_blocks, 256, nullptr, nullptr, 0, &g);
    hipLaunchKernelGGL(split_reduce_group_kernel, dim3((unsigned)reduce_blocks), dim3(256), 0, stream, g);
    RST_HIP(hipGetLastError());
  }
  return RST_OK;
}

bool can_pair_gemm(const GemmDesc& input_grad, const GemmDesc& weight_grad) {
  long long b1 = 0, b2 = 0;
  const bool layouts = input_grad.a_kc && !input_grad.b_kc && !weight_grad.a_kc && !weight_grad.b_kc;
  // worth it when the input gradient alone would leave one workgroup per CU
  return layouts && takes_plain_dma(input_grad, &b1) && takes_plain_dma(weight_grad, &b2) && b1 < 512 &&
         b1 % 8 == 0 && b2 >= b1 && b1 + b2 <= 0x7fffffffLL;
}

int launch_gemm_pair(hipStream_t stream, const GemmDesc& input_grad, const GemmDesc& weight_grad) {
  if (!can_pair_gemm(input_grad, weight_grad))
    return fail(RST_ERR_INVALID_ARGUMENT, "these two contractions cannot share a grid");
  GemmParams p1 = make_params(input_grad), p2 = make_params(weight_grad);
  p1.tiles_m = (p1.M + 127) / 128; p1.tiles_n = (p1.N + 127) / 128; p1.steps_per_split = dma_whole_steps(p1.K, p1.k_reserve);
  p2.tiles_m = (p2.M + 127) / 128; p2.tiles_n = (p2.N + 127) / 128; p2.steps_per_split = dma_whole_steps(p2.K, p2.k_reserve);
  const long long b1 = (long long)p1.tiles_m * p1.tiles_n, b2 = (long long)p2.tiles_m * p2.tiles_n;
  RST_OBSERVE_GEMM(GemmKernel::kDma128Pair, 128, 128, 2, 4, true, false, true, 0, b1 + b2, 512, &p1, &p2, (int)b1, nullptr);
  hipLaunchKernelGGL((gemm_f64_mfma_dma_pair<true, false, false, false>), dim3((unsigned)(b1 + b2)), dim3(512),
                     0, stream, p1, p2, (int)b1);
  RST_HIP(hipGetLastError());
  return RST_OK;
}

}  // namespace rst
