// Index arithmetic of the FP64 contraction kernels, as host-and-device functions.
//
// Every address a lane of these kernels forms - where a tile-DMA lane reads its 16 bytes, which LDS
// bytes it lands on, which pair a register-staged load takes (clamps and the masked K tail
// included), where an accumulator register is stored, which K steps a slice covers, where a slice's
// partial products sit in the workspace - is computed by one of the functions below.  The kernels
// call them on the device; a host-side model (tests/host_stub) calls the very same functions for
// every workgroup, wavefront and lane of a planned launch and checks each byte range against the
// operand it belongs to, because a wrong offset on the GPU is a memory fault that takes the machine
// with it and leaves no trace to read.
#pragma once

#include <cstddef>
#include <cstdint>

#if defined(__HIPCC__) || defined(__CUDACC__)
#define RST_HD __host__ __device__ __forceinline__
#else
#define RST_HD inline
#endif

namespace rst {

constexpr int BK = 16;  // contraction indices per LDS tile

struct GemmParams {
  const double* A;
  const double* B;
  double* C;
  int M, N, K;
  long lda, ldb, ldc;
  int epilogue;
  const double* bias;
  double divisor;
  double divisor_reciprocal;  // exact 1 / divisor when divisor is a power of two, else 0
  const double* mask;
  long ldmask;
  double* colsum;        // weight-gradient launches only: colsum[i] = (sum_k A(i,k)) / colsum_div
  double colsum_div;
  // weight-gradient launches of the fused training step: once C = acc / divisor (and colsum) are
  // stored, the SGD update parm -= lr * grad is applied to the parameter of the same index
  double* sgd_parm;      // same shape and leading dimension as C, or NULL
  double* sgd_bias;      // same shape as colsum, or NULL
  double sgd_lr;
  int tiles_m, tiles_n;
  // split-K (small outputs with a long contraction): slice s of the K steps is multiplied by
  // workgroups [s*tiles, (s+1)*tiles) and lands, without epilogue, in ws[s][M][N] (and its
  // column sums in ws_colsum[s][M]); split_reduce_kernel adds the slices in order afterwards.
  int split_k;           // number of slices, 1 = off
  int steps_per_split;   // K steps (of BK) per slice
  double* ws;
  double* ws_colsum;
  size_t ws_capacity;    // doubles available at ws
  // 128x128 direct-to-LDS kernel, launches of more than one round of workgroups: the workgroups of
  // the first round that sit in the upper wave slots of their CU start this many 10 ns ticks late
  int dephase_ticks;
  int first_round;       // workgroups that fit on the chip at once
  // Direct-to-LDS kernels on operands that do not promise 16-byte aligned pairs (an odd leading
  // dimension or extent, a base address that is only 8-byte aligned).  The tile DMA itself takes
  // 8-byte aligned addresses; what changes is the masked K tail (single loads) and, when an
  // output-contiguous operand has an odd extent, which K rows travel by DMA: the pair that holds
  // the operand's last column also fetches the double behind it, which for the operand's very last
  // K row would lie behind the operand, so that row is kept back for the tail (k_reserve = 1).
  int unaligned;         // 1 = the K tail is fetched by single loads
  int k_reserve;         // K rows (0 or 1) kept out of the whole steps that travel by DMA
};

// Up to kMaxGroup products in one grid: workgroups [first_block[i], first_block[i+1]) belong to
// problem i; problems cut into K slices are finished by one shared reduction grid, whose workgroups
// [first_reduce_block[i], first_reduce_block[i+1]) belong to problem i.
constexpr int kMaxGroup = 8;
struct GemmGroup {
  int count;
  int first_block[kMaxGroup + 1];
  int first_reduce_block[kMaxGroup + 1];
  unsigned char layout[kMaxGroup];  // bit 0: A contraction-contiguous, bit 1: B (the mixed kernel reads it)
  GemmParams p[kMaxGroup];
};
static_assert(sizeof(GemmGroup) <= 4096, "a group travels as one kernel argument");

// ---- which output tile and K slice a workgroup works on -----------------------------------------
// Workgroups are handed to the 8 XCDs round-robin; they are renumbered so that each XCD (and its
// private L2) works on one compact patch of the tile grid, and the patch is walked in groups of 8
// tile rows so that concurrently resident workgroups share operand panels.  A bijection between
// [0, tiles_m * tiles_n * split_k) and (split, tile_m, tile_n).
struct TileCoord {
  int split, tile_m, tile_n;
};
RST_HD TileCoord tile_of_block(int tiles_m, int tiles_n, int block) {
  const int n_blocks = tiles_m * tiles_n;
  TileCoord t;
  t.split = block / n_blocks;
  int logical;
  {
    const int pid = block - t.split * n_blocks;
    const int xcd = pid & 7, local = pid >> 3;
    const int base = n_blocks >> 3, rem = n_blocks & 7;
    logical = xcd * base + (xcd < rem ? xcd : rem) + local;
  }
  constexpr int GROUP = 8;
  const int group_size = GROUP * tiles_n;
  const int group = logical / group_size;
  const int first_m = group * GROUP;
  const int gm = (tiles_m - first_m) < GROUP ? (tiles_m - first_m) : GROUP;
  const int in_group = logical - group * group_size;
  t.tile_m = first_m + in_group % gm;
  t.tile_n = in_group / gm;
  return t;
}

// ---- which K steps a workgroup multiplies --------------------------------------------------------
// Register-staged kernels: K steps [kt0, nk) of BK indices each; steps below nk_full are whole, the
// one at nk_full (if K % BK != 0) is partial and belongs to the last slice.
struct StagedSteps {
  int kt0, nk, nk_full;
};
RST_HD StagedSteps staged_k_steps(int K, int split_k, int steps_per_split, int split) {
  StagedSteps s;
  s.nk_full = K / BK;
  const int nk_all = s.nk_full + (K % BK != 0 ? 1 : 0);
  s.kt0 = split * steps_per_split;
  s.nk = (split_k > 1 && s.kt0 + steps_per_split < nk_all) ? s.kt0 + steps_per_split : nk_all;
  return s;
}
// Direct-to-LDS kernels: whole steps [kt0, kt0 + nk_dma) travel by tile DMA; what is left of K
// beyond the last of them (1 to BK indices starting at dma_whole_steps * BK) is an extra first tile
// of slice 0, copied by masked register loads.  k_reserve (0 or 1) rows at the end of K never
// travel by DMA (GemmParams::k_reserve).
RST_HD int dma_whole_steps(int K, int k_reserve) { return (K - k_reserve) / BK; }
struct DmaSteps {
  int kt0, nk_dma;
  bool k_tail;
};
RST_HD DmaSteps dma_k_steps(int K, int split_k, int steps_per_split, int split, int k_reserve) {
  DmaSteps s;
  const int nk_all = dma_whole_steps(K, k_reserve);
  s.kt0 = split * steps_per_split;
  s.nk_dma = (split_k > 1) ? ((nk_all - s.kt0 < steps_per_split) ? nk_all - s.kt0 : steps_per_split) : nk_all;
  s.k_tail = K > nk_all * BK && split == 0;
  return s;
}

// ---- tile DMA: global byte offset of a lane's 16 bytes -------------------------------------------
// The offset is relative to the tile origin at K step 0 of the workgroup (operand + o0 * ld for a
// contraction-contiguous operand, operand + o0 for an output-contiguous one, o0 = first output row
// or column of the tile) and is the same for every K step; the kernels keep it in 32 bits (T =
// uint32_t), the host model also evaluates it in 64 bits to see that nothing wrapped.
//
// Contraction-contiguous operand, 1 KiB chunk `chunk` = 8 tile rows x 16 doubles: lane l fetches,
// for tile row 8*chunk + l/8, the pair k = 2*((l%8) ^ (row&7)) - the XOR swizzle of the LDS layout
// is applied by choosing the global address.  Rows beyond the operand's extent are clamped onto its
// last row (they only feed outputs that are never stored).
template <typename T>
RST_HD T dma_offset_kc(int chunk, int lane, int o0, int ext, long ld) {
  const int row = 8 * chunk + (lane >> 3);
  const int rr = o0 + row < ext ? row : ext - 1 - o0;
  return (T)8 * (T)((size_t)rr * (size_t)ld + (size_t)(2 * ((lane & 7) ^ (row & 7))));
}
// Output-contiguous operand of the 128-wide tiles, chunk = one k row of 128 doubles: lane l fetches
// columns 2l, 2l+1; a pair that begins beyond the extent is moved back onto the last two columns.
// With an odd extent the pair that begins on the last column stays where it is and also fetches the
// double behind the row's end (the next row's first one, or padding): it feeds an output that is
// never stored, and GemmParams::k_reserve keeps the one row where it would leave the operand away
// from the DMA.
template <typename T>
RST_HD T dma_offset_oc128(int chunk, int lane, int o0, int ext, long ld) {
  const int back = ext - 2 - o0 > 0 ? ext - 2 - o0 : 0;  // (0: a tile that holds the one last column of an odd extent)
  const int ge = o0 + 2 * lane < ext ? 2 * lane : back;
  return (T)8 * (T)((size_t)chunk * (size_t)ld + (size_t)(long)ge);
}
// Output-contiguous operand of the 64-wide tiles, chunk = two k rows of 64 doubles (k rows 2*chunk
// and 2*chunk + 1): lanes 0-31 the first, 32-63 the second; the 16-byte slots of k rows 2g, 2g+1 are
// XOR-ed with 8 * (g & 3), again by choosing the global address.
template <typename T>
RST_HD T dma_offset_oc64(int chunk, int lane, int o0, int ext, long ld) {
  const int kr = 2 * chunk + (lane >> 5);
  const int e = 2 * ((lane & 31) ^ (8 * (chunk & 3)));
  const int back = ext - 2 - o0 > 0 ? ext - 2 - o0 : 0;
  const int ge = o0 + e < ext ? e : back;  // as for the 128-wide tiles
  return (T)8 * (T)((size_t)kr * (size_t)ld + (size_t)(long)ge);
}
// bytes from one K step of a tile to the next
RST_HD long dma_k_step_bytes(bool kc, long ld) { return 8 * (kc ? (long)BK : (long)BK * ld); }
// LDS destination (in doubles, inside a stage) of chunk `chunk`; lane l lands 2*l doubles further
RST_HD int dma_lds_chunk_kc(int chunk) { return chunk * 128; }
RST_HD int dma_lds_chunk_oc128(int chunk, int ext) { return chunk * (ext + 16); }
RST_HD int dma_lds_chunk_oc64(int chunk) { return chunk * 128; }
// doubles of one LDS stage of an operand tile of `ext` rows or columns
RST_HD constexpr int dma_stage_doubles(bool kc, int ext) { return kc ? ext * BK : BK * (ext + 16); }

// ---- LDS side of the tile DMA: where a fragment read finds element (e, pair) ------------------------
// e = row (or column) inside the tile, pair = k / 2 inside the tile's BK contraction steps; the
// result is in doubles from the start of the stage and names the first double of the pair (k even);
// k odd is the next double (contraction-contiguous) or one k row further (output-contiguous).
RST_HD int frag_lds_kc(int e, int pair) { return e * BK + 2 * (pair ^ (e & 7)); }
RST_HD int frag_lds_oc128(int e, int pair, int ext) { return 2 * pair * (ext + 16) + e; }
RST_HD int frag_lds_oc64(int e, int pair) { return 2 * pair * 64 + 2 * ((e >> 1) ^ (8 * (pair & 3))) + (e & 1); }

// ---- register-staged loads: which pair of doubles thread-slot q takes -----------------------------
// A tile of EXT rows/cols by BK contraction steps is EXT*BK/2 pairs.  first/second: element
// offsets (in doubles, from the operand's base pointer) of the two doubles; vec: they are adjacent
// and 16-byte aligned and travel as one load; keep_*: false where the value lies beyond K and is
// replaced by zero (both operands do so, so no stray NaN or infinity meets a zero).
//   ext0 / ext_n: first row (or column) of the tile along the output dimension and its limit; rows
//   beyond the limit are clamped onto the last valid ones - they only feed outputs never stored.
//   k0 / k_n: first contraction index and its limit.  TAIL = false promises k0 + BK <= k_n.
//   VEC = true promises 16-byte alignment of every pair (even leading dimension, even extent).
struct PairSource {
  size_t first, second;
  bool vec, keep_first, keep_second;
};
template <int EXT, bool KC, bool VEC, bool TAIL>
RST_HD PairSource staged_pair_source(int q, long ld, int ext0, int ext_n, int k0, int k_n) {
  PairSource s;
  int e, k;  // coordinates of the first of the two doubles
  if (KC) {
    e = ext0 + (q >> 3);  // BK/2 = 8 pairs per row
    k = k0 + 2 * (q & 7);
    const int ec = e < ext_n ? e : ext_n - 1;
    int ka = k, kb = k + 1;
    if (TAIL) {
      ka = ka < k_n ? ka : k_n - 1;
      kb = kb < k_n ? kb : k_n - 1;
    }
    s.first = (size_t)ec * (size_t)ld + (size_t)ka;
    s.second = (size_t)ec * (size_t)ld + (size_t)kb;
    s.vec = VEC && !TAIL;
    s.keep_first = !TAIL || k < k_n;
    s.keep_second = !TAIL || k + 1 < k_n;
  } else {
    k = k0 + q / (EXT / 2);
    e = ext0 + 2 * (q % (EXT / 2));
    int kc = k;
    if (TAIL) kc = kc < k_n ? kc : k_n - 1;
    if (VEC) {
      const int ec = e + 1 < ext_n ? e : ext_n - 2;
      s.first = (size_t)kc * (size_t)ld + (size_t)ec;
      s.second = s.first + 1;
    } else {
      const int ea = e < ext_n ? e : ext_n - 1;
      const int eb = e + 1 < ext_n ? e + 1 : ext_n - 1;
      s.first = (size_t)kc * (size_t)ld + (size_t)ea;
      s.second = (size_t)kc * (size_t)ld + (size_t)eb;
    }
    s.vec = VEC;
    s.keep_first = s.keep_second = !TAIL || k < k_n;
  }
  return s;
}

// ---- epilogue ----------------------------------------------------------------------------------------
// Accumulator register r of MFMA fragment (i, j) of a wavefront block at (row0, col0) holds output
// row row0 + 16*i + 4*r + lk, column col0 + 16*j + lr (lr = lane % 16, lk = lane / 16).
RST_HD int acc_row(int row0, int i, int r, int lk) { return row0 + i * 16 + 4 * r + lk; }
RST_HD int acc_col(int col0, int j, int lr) { return col0 + j * 16 + lr; }
// How many of the tm x tn fragments (16 x 16) of a wavefront block at (row0, col0) reach into an
// M x N output: rows of fragments and columns of fragments (0 x 0 when the block is wholly outside).
struct LiveFragments {
  int rows, cols;
};
RST_HD LiveFragments live_fragments(int M, int N, int row0, int col0, int tm, int tn) {
  LiveFragments l;
  l.rows = row0 < M ? (M - row0 + 15) / 16 : 0;
  l.cols = col0 < N ? (N - col0 + 15) / 16 : 0;
  if (l.rows > tm) l.rows = tm;
  if (l.cols > tn) l.cols = tn;
  if (l.rows == 0 || l.cols == 0) l.rows = l.cols = 0;
  return l;
}
// A block of TM x TN fragments that lies wholly inside the output takes the unpredicated epilogue,
// whose lane offsets are 32-bit: every leading dimension involved must stay below 2^26 doubles.
RST_HD bool block_is_interior(const GemmParams& p, int row0, int col0, int tm, int tn) {
  return row0 + 16 * tm <= p.M && col0 + 16 * tn <= p.N && p.ldc < (1L << 26) && (long)p.N < (1L << 26) &&
         p.ldmask < (1L << 26);
}
// byte offset of a lane from the wave-uniform row pointer (row row0 + 16*i + 4*r, column col0); the
// fragment column j adds 128*j bytes
template <typename T>
RST_HD T interior_lane_offset(int lk, int lr, long ld) {
  return (T)8 * (T)((size_t)lk * (size_t)ld + (size_t)lr);
}
// where K slice `split` of a split contraction keeps its partial products [M][N] and, behind all
// slices' products, its column sums [M]
RST_HD size_t ws_slice_offset(const GemmParams& p, int split) { return (size_t)split * (size_t)p.M * (size_t)p.N; }
RST_HD size_t ws_colsum_offset(const GemmParams& p, int split) { return (size_t)split * (size_t)p.M; }


// ---- grids that hold more than one problem -----------------------------------------------------------
// member of a group that workgroup `block` belongs to
RST_HD int group_member_of_block(const int* first_block, int count, int block) {
  int i = 0;
  while (i + 1 < count && block >= first_block[i + 1]) ++i;
  return i;
}
// The paired grid (two products, the first with first_blocks workgroups, the second with at least as
// many): the first 2*first_blocks workgroups alternate between the two problems in groups of eight
// (one per XCD), with the phase flipped every 32 groups, so that the long tiles of the first problem
// spread over the CUs under the usual hand-out orders; tile numbers keep their value mod 8, which
// the XCD-aware tile walk relies on.  The remaining workgroups all belong to the second problem.
struct PairSlot {
  int problem;  // 0 = first, 1 = second
  int block;    // workgroup number inside that problem
};
RST_HD PairSlot pair_slot_of_block(int b, int first_blocks) {
  PairSlot s;
  if (b < 2 * first_blocks) {
    const int g = b >> 3;
    s.block = (g >> 1) * 8 + (b & 7);
    s.problem = ((g + (g >> 5)) & 1) == 0 ? 0 : 1;
  } else {
    s.problem = 1;
    s.block = b - first_blocks;
  }
  return s;
}

// ---- a launch as an observer sees it ----------------------------------------------------------------
// The test build (tests/host_stub, -DRST_GEMM_LAUNCH_OBSERVER) defines observe_gemm_launch and walks
// every lane of the planned grid through the functions above; the product build compiles the hook
// away.
enum class GemmKernel {
  kStaged,            // gemm_f64_mfma<BM, BN, WGM, WGN, A_KC, B_KC, VEC, BURST>
  kStagedGroup,       // gemm_f64_mfma_group<A_KC, B_KC, BURST>: 32x32 tiles, 2x2 wavefronts, VEC
  kStagedMixedGroup,  // gemm_f64_mfma_mixed_group<BURST>: layout per member
  kDma128,            // gemm_f64_mfma_dma<A_KC, B_KC, 2, 4, 2, 1>
  kDma128Group,       // gemm_f64_mfma_dma_group (both operands output-contiguous)
  kDma128Pair,        // gemm_f64_mfma_dma_pair<true, false, false, false>
  kDma64,             // gemm_f64_mfma_dma64<B_KC> (A contraction-contiguous)
  kSplitReduce,       // split_reduce_kernel
  kSplitReduceGroup   // split_reduce_group_kernel
};
struct GemmLaunch {
  GemmKernel kernel;
  int bm, bn, wgm, wgn;
  bool a_kc, b_kc, vec;
  int burst;
  long long blocks;
  int threads;
  const GemmParams* p;      // the problem (the first one of a pair)
  const GemmParams* p2;     // the second problem of a pair
  int first_blocks;         // workgroups of the first problem of a pair
  const GemmGroup* group;   // the members of a grouped launch
};
#ifdef RST_GEMM_LAUNCH_OBSERVER
void observe_gemm_launch(const GemmLaunch& launch);
#define RST_OBSERVE_GEMM(...) ::rst::observe_gemm_launch(::rst::GemmLaunch{__VA_ARGS__})
#else
#define RST_OBSERVE_GEMM(...) do { } while (0)
#endif

}  // namespace rst
