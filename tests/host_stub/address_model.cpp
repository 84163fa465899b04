// Host-side model of the addressing of the FP64 contraction kernels.
//
// The library, built for the host with -DRST_GEMM_LAUNCH_OBSERVER, reports every contraction launch
// it plans to observe_gemm_launch below.  For that launch the model walks every workgroup, wavefront
// and lane of the grid through the SAME index functions the kernels run on the device
// (rstorch_amd/csrc/gemm_addressing.h) and checks, before anything could reach a GPU:
//   * every global read lies inside the logical footprint of its operand ((rows-1)*ld + cols doubles)
//     and every 16-byte register load is 16-byte aligned (the tile DMA needs 8 bytes only: launches
//     that promise aligned operands are held to 16, the others to 8 and to never displacing an
//     element that exists); the 32-bit lane offsets equal their 64-bit values;
//   * every tile-DMA lane lands inside its LDS stage, every fragment read stays inside the stage, and
//     the slot a fragment read takes for (row, pair) is the slot the DMA put that (row, pair) in;
//   * the workgroups of a grid map one-to-one onto (K slice, output tile), the K slices of a tile
//     cover the contraction exactly once, and every output element is stored exactly once per slice;
//   * partial products and column sums of a split contraction stay inside the workspace, and the
//     regions of the members of a grouped launch do not overlap;
//   * the reduction grid reads exactly what the slices wrote.
// A violation prints what it found and aborts, which fails the test that drives the library.
// Nothing is dereferenced: operands may be made-up addresses.  Test infrastructure, never shipped.
#include <cinttypes>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <set>
#include <string>
#include <vector>

#include "../../rstorch_amd/csrc/gemm_addressing.h"

namespace rst {
namespace {

long g_checked[16] = {};       // launches verified, per GemmKernel
long g_staged_by_tile[2] = {}; // register-staged launches verified: 32x32, 128x128 tiles
long g_sliced[16] = {};        // of g_checked: launches on K slices
long g_unaligned[16] = {};     // of g_checked: tile-DMA launches on operands without 16-byte aligned pairs
long g_reserved[16] = {};      // of g_unaligned: launches that keep the last K row back for the tail
long g_skipped_repeats = 0;    // launches seen before (same kernel, same parameters)
long long g_lane_checks = 0;   // individual address checks
std::set<std::string> g_seen;

const char* kernel_name(GemmKernel k) {
  switch (k) {
    case GemmKernel::kStaged: return "staged";
    case GemmKernel::kStagedGroup: return "staged_group";
    case GemmKernel::kStagedMixedGroup: return "staged_mixed_group";
    case GemmKernel::kDma128: return "dma128";
    case GemmKernel::kDma128Group: return "dma128_group";
    case GemmKernel::kDma128Pair: return "dma128_pair";
    case GemmKernel::kDma64: return "dma64";
    case GemmKernel::kSplitReduce: return "split_reduce";
    default: return "split_reduce_group";
  }
}

std::string g_context;  // what is being checked, for the failure message

[[noreturn]] void bad(const char* fmt, ...) {
  std::fprintf(stderr, "address model: %s: ", g_context.c_str());
  va_list ap;
  va_start(ap, fmt);
  std::vfprintf(stderr, fmt, ap);
  va_end(ap);
  std::fprintf(stderr, "\n");
  std::abort();
}

std::string describe(const GemmParams& p, bool a_kc, bool b_kc) {
  char buf[256];
  std::snprintf(buf, sizeof(buf), "M=%d N=%d K=%d lda=%ld ldb=%ld ldc=%ld a_kc=%d b_kc=%d epi=%d split=%d x %d steps",
                p.M, p.N, p.K, p.lda, p.ldb, p.ldc, (int)a_kc, (int)b_kc, p.epilogue, p.split_k, p.steps_per_split);
  return buf;
}

// logical footprint, in doubles, of an operand of `ext` output rows/columns and K contraction indices
size_t footprint(bool kc, int ext, int K, long ld) {
  if (ext <= 0 || K <= 0) return 0;
  return kc ? (size_t)(ext - 1) * (size_t)ld + (size_t)K : (size_t)(K - 1) * (size_t)ld + (size_t)ext;
}

// [first, first + count) doubles must lie inside [0, limit)
void in_range(const char* what, size_t first, size_t count, size_t limit) {
  ++g_lane_checks;
  if (first + count > limit || first + count < first)
    bad("%s: doubles [%zu, %zu) outside the operand's %zu", what, first, first + count, limit);
}

void aligned16(const char* what, const void* base, size_t byte_offset) {
  if ((reinterpret_cast<uintptr_t>(base) + byte_offset) % 16 != 0)
    bad("%s: 16-byte access at a misaligned address (base %p + %zu)", what, base, byte_offset);
}

// each (slice, output element) exactly once
struct Coverage {
  int M, N, splits;
  std::vector<unsigned char> seen;
  Coverage(int m, int n, int s) : M(m), N(n), splits(s), seen((size_t)m * n * s, 0) {}
  void mark(int split, int row, int col) {
    if (row < 0 || row >= M || col < 0 || col >= N || split < 0 || split >= splits)
      bad("store outside the output: slice %d row %d col %d of %d x %d", split, row, col, M, N);
    unsigned char& c = seen[((size_t)split * M + row) * N + col];
    if (c) bad("output element (%d, %d) of slice %d stored twice", row, col, split);
    c = 1;
  }
  void complete() const {
    for (size_t i = 0; i < seen.size(); ++i)
      if (!seen[i]) bad("output element %zu (of %d x %d x %d slices) never stored", i, M, N, splits);
  }
};

struct ColsumCoverage {
  int M, splits;
  std::vector<unsigned char> seen;
  ColsumCoverage(int m, int s) : M(m), splits(s), seen((size_t)m * s, 0) {}
  void mark(int split, int row) {
    if (row < 0 || row >= M) bad("column sum %d outside [0, %d)", row, M);
    unsigned char& c = seen[(size_t)split * M + row];
    if (c) bad("column sum %d of slice %d written twice", row, split);
    c = 1;
  }
  void complete() const {
    for (size_t i = 0; i < seen.size(); ++i)
      if (!seen[i]) bad("column sum %zu never written", i);
  }
};

// ---- what every kernel has in common ----------------------------------------------------------------
void check_params(const GemmParams& p, bool a_kc, bool b_kc) {
  if (p.M <= 0 || p.N <= 0 || p.K < 0) bad("empty problem reached a launch");
  if (p.tiles_m <= 0 || p.tiles_n <= 0) bad("tiles %d x %d", p.tiles_m, p.tiles_n);
  if (p.split_k < 1) bad("split_k = %d", p.split_k);
  if (p.lda < (a_kc ? p.K : p.M) || p.ldb < (b_kc ? p.K : p.N) || p.ldc < p.N)
    bad("a leading dimension is smaller than its row");
  if (p.split_k > 1) {
    if (!p.ws) bad("split contraction without a workspace");
    if (p.ws_colsum != p.ws + (size_t)p.split_k * p.M * p.N) bad("column sums do not follow the partial products");
  }
}

// the slices of a contraction cover its K steps exactly once (DMA kernels: whole steps by DMA + the tail)
void check_dma_k_cover(const GemmParams& p) {
  if (p.k_reserve != 0 && p.k_reserve != 1) bad("k_reserve = %d", p.k_reserve);
  const int nk_all = dma_whole_steps(p.K, p.k_reserve);
  int next = 0, tails = 0;
  for (int s = 0; s < p.split_k; ++s) {
    const DmaSteps ks = dma_k_steps(p.K, p.split_k, p.steps_per_split, s, p.k_reserve);
    if (ks.nk_dma < 0) bad("slice %d has %d K steps", s, ks.nk_dma);
    if (ks.nk_dma > 0 && ks.kt0 != next) bad("slice %d starts at step %d, expected %d", s, ks.kt0, next);
    if (ks.nk_dma > 0) next = ks.kt0 + ks.nk_dma;
    if (ks.nk_dma == 0 && !ks.k_tail && p.split_k > 1) bad("slice %d of %d is empty", s, p.split_k);
    tails += ks.k_tail ? 1 : 0;
  }
  if (next != nk_all) bad("the slices cover %d of %d whole K steps", next, nk_all);
  if (p.K - nk_all * BK < 0 || p.K - nk_all * BK > BK) bad("a K remainder of %d indices", p.K - nk_all * BK);
  if (tails != (p.K > nk_all * BK ? 1 : 0)) bad("the K remainder is multiplied %d times", tails);
}
void check_staged_k_cover(const GemmParams& p) {
  const int nk_all = (p.K + BK - 1) / BK;
  int next = 0;
  for (int s = 0; s < p.split_k; ++s) {
    const StagedSteps ks = staged_k_steps(p.K, p.split_k, p.steps_per_split, s);
    if (ks.kt0 != next) bad("slice %d starts at step %d, expected %d", s, ks.kt0, next);
    if (ks.nk <= ks.kt0 && nk_all > 0) bad("slice %d of %d is empty", s, p.split_k);
    next = ks.nk;
  }
  if (next != nk_all) bad("the slices cover %d of %d K steps", next, nk_all);
}

// ---- epilogue of one wavefront block (write_block<TM, TN>) ------------------------------------------------
// live != NULL: the kernel skips the MFMAs of fragments beyond live->rows x live->cols, so nothing that
// is stored may sit in one of those
void check_write_block(const GemmParams& p, int tm, int tn, int row0, int col0, int split, Coverage& cov,
                       const LiveFragments* live = nullptr) {
  const size_t c_limit = (size_t)(p.M - 1) * (size_t)p.ldc + (size_t)p.N;
  const size_t mask_limit = (size_t)(p.M - 1) * (size_t)p.ldmask + (size_t)p.N;
  const bool interior = block_is_interior(p, row0, col0, tm, tn);
  const bool sliced = p.split_k > 1;
  // a slice stores raw partial products [M][N] at ws + slice offset, whatever the epilogue
  const long ld_out = sliced ? (long)p.N : p.ldc;
  const size_t out_limit = sliced ? (size_t)p.M * (size_t)p.N : c_limit;
  if (sliced && ws_slice_offset(p, split) + (size_t)p.M * p.N > (size_t)p.split_k * p.M * p.N)
    bad("slice %d ends beyond the partial-product area", split);
  const bool uses_interior_path = interior && (sliced || p.epilogue != 3 /*EPI_DIVIDE*/ || p.divisor_reciprocal != 0.0);
  for (int lane = 0; lane < 64; ++lane) {
    const int lr = lane & 15, lk = lane >> 4;
    if (uses_interior_path) {
      const uint32_t off32 = interior_lane_offset<uint32_t>(lk, lr, ld_out);
      const uint64_t off64 = interior_lane_offset<uint64_t>(lk, lr, ld_out);
      if (off32 != off64) bad("interior store offset wraps 32 bits (ld %ld)", ld_out);
      const uint32_t m32 = interior_lane_offset<uint32_t>(lk, lr, p.ldmask);
      const uint64_t m64 = interior_lane_offset<uint64_t>(lk, lr, p.ldmask);
      if (!sliced && p.epilogue == 4 /*EPI_MASK*/ && m32 != m64) bad("interior mask offset wraps 32 bits");
    }
    for (int i = 0; i < tm; ++i)
      for (int r = 0; r < 4; ++r)
        for (int j = 0; j < tn; ++j) {
          const int row = acc_row(row0, i, r, lk), col = acc_col(col0, j, lr);
          if (uses_interior_path) {
            // wave-uniform row pointer (row0 + 16 i + 4 r, col0) + lane offset + 128 j bytes
            const size_t elem = (size_t)acc_row(row0, i, r, 0) * (size_t)ld_out + (size_t)col0 +
                                interior_lane_offset<uint64_t>(lk, lr, ld_out) / 8 + (size_t)16 * j;
            if (elem != (size_t)row * (size_t)ld_out + (size_t)col) bad("interior store address does not name (row, col)");
            in_range("interior store", elem, 1, out_limit);
            if (live && (i >= live->rows || j >= live->cols)) bad("a stored element sits in a fragment whose MFMAs are skipped");
            cov.mark(split, row, col);
            if (!sliced && p.epilogue == 4) {
              const size_t me = (size_t)acc_row(row0, i, r, 0) * (size_t)p.ldmask + (size_t)col0 +
                                interior_lane_offset<uint64_t>(lk, lr, p.ldmask) / 8 + (size_t)16 * j;
              in_range("interior mask read", me, 1, mask_limit);
            }
          } else {
            // general path: clamped loads, predicated stores
            const int rc = row < p.M ? row : p.M - 1, cc = col < p.N ? col : p.N - 1;
            if (rc < 0 || cc < 0) bad("clamped epilogue index is negative");
            if (!sliced && p.epilogue == 4) in_range("mask read", (size_t)rc * p.ldmask + cc, 1, mask_limit);
            if (!sliced && p.sgd_parm) in_range("parameter read", (size_t)rc * p.ldc + cc, 1, c_limit);
            if (!sliced && (p.epilogue == 1 || p.epilogue == 2)) in_range("bias read", (size_t)cc, 1, (size_t)p.N);
            if (row < p.M && col < p.N) {
              in_range("store", (size_t)row * (size_t)ld_out + (size_t)col, 1, out_limit);
              if (live && (i >= live->rows || j >= live->cols)) bad("a stored element sits in a fragment whose MFMAs are skipped");
              cov.mark(split, row, col);
            }
          }
        }
  }
}

// column sums (bias gradient) by the workgroups of tile column 0: thread t owns row t % BM
void check_colsum(const GemmParams& p, bool a_kc, int bm, int threads, int m0, int tile_n, int split,
                  ColsumCoverage* cov) {
  if (a_kc || !p.colsum || tile_n != 0 || !cov) return;
  if (threads % bm != 0) bad("column-sum threads %d do not split over %d rows", threads, bm);
  for (int e = 0; e < bm; ++e)
    if (m0 + e < p.M) cov->mark(split, m0 + e);
}

// ---- tile-DMA kernels -------------------------------------------------------------------------------
enum class OcKind { k128, k64 };

// one operand tile of a DMA kernel: every lane of every chunk, first and last K step
void check_dma_operand(const char* name, const double* base, bool kc, OcKind oc, int ext_tile, int chunks, int o0,
                       int ext, int K, long ld, int kt0, int nk_dma, bool aligned) {
  const size_t limit = footprint(kc, ext, K, ld);
  const size_t origin = kc ? (size_t)o0 * (size_t)ld : (size_t)o0;
  const size_t step = (size_t)dma_k_step_bytes(kc, ld) / 8;
  const int stage = kc ? ext_tile * BK : (oc == OcKind::k128 ? BK * (ext_tile + 16) : ext_tile * BK);
  if (o0 < 0 || o0 >= ext) bad("%s tile origin %d outside [0, %d)", name, o0, ext);
  if (ld >= (1L << 22)) bad("%s leading dimension %ld is too long for the 32-bit DMA lane offsets", name, ld);
  for (int c = 0; c < chunks; ++c)
    for (int lane = 0; lane < 64; ++lane) {
      uint32_t o32;
      uint64_t o64;
      int lds;
      if (kc) {
        o32 = dma_offset_kc<uint32_t>(c, lane, o0, ext, ld);
        o64 = dma_offset_kc<uint64_t>(c, lane, o0, ext, ld);
        lds = dma_lds_chunk_kc(c);
      } else if (oc == OcKind::k128) {
        o32 = dma_offset_oc128<uint32_t>(c, lane, o0, ext, ld);
        o64 = dma_offset_oc128<uint64_t>(c, lane, o0, ext, ld);
        lds = dma_lds_chunk_oc128(c, ext_tile);
      } else {
        o32 = dma_offset_oc64<uint32_t>(c, lane, o0, ext, ld);
        o64 = dma_offset_oc64<uint64_t>(c, lane, o0, ext, ld);
        lds = dma_lds_chunk_oc64(c);
      }
      if (o32 != o64) bad("%s DMA lane offset wraps 32 bits: %u vs %" PRIu64, name, o32, o64);
      if (o64 % (aligned ? 16 : 8) != 0) bad("%s DMA lane offset %" PRIu64 " is not a multiple of %d", name, o64, aligned ? 16 : 8);
      {
        // an element that exists is fetched from its own place: the clamps only move pairs that lie
        // wholly beyond the extent (rows of a contraction-contiguous tile, columns of the other kind)
        const uint64_t d = o64 / 8;
        if (kc) {
          const int row = 8 * c + (lane >> 3), k = 2 * ((lane & 7) ^ (row & 7));
          if (o0 + row < ext && d != (uint64_t)row * (uint64_t)ld + (uint64_t)k) bad("%s DMA: row %d pair %d displaced", name, row, k);
        } else {
          const int krow = oc == OcKind::k128 ? c : 2 * c + (lane >> 5);
          const int e = oc == OcKind::k128 ? 2 * lane : 2 * ((lane & 31) ^ (8 * (c & 3)));
          if (o0 + e < ext && d != (uint64_t)krow * (uint64_t)ld + (uint64_t)e) bad("%s DMA: k row %d column %d displaced", name, krow, e);
        }
      }
      if (lds < 0 || lds + 2 * lane + 2 > stage) bad("%s DMA chunk %d lane %d lands outside its LDS stage", name, c, lane);
      if (nk_dma > 0) {
        const size_t first = origin + (size_t)kt0 * step + o64 / 8;
        const size_t last = origin + (size_t)(kt0 + nk_dma - 1) * step + o64 / 8;
        in_range(name, first, 2, limit);
        in_range(name, last, 2, limit);
        if (aligned) {
          aligned16(name, base, 8 * first);
          aligned16(name, base, 8 * last);
        }
      }
    }
}

// the LDS slot a fragment read takes for (e, pair) holds what the DMA put there for (e, pair)
void check_lds_layout(bool kc, OcKind oc, int ext_tile, int chunks) {
  const int stage = kc ? ext_tile * BK : (oc == OcKind::k128 ? BK * (ext_tile + 16) : ext_tile * BK);
  // slot (in doubles) -> e * 16 + k of the element the DMA stores there; the global address of the
  // lane decides which element that is: recover (row, k) from the offset with ld = 1 << 12
  const long ld = 1L << 12;
  std::vector<int> holds((size_t)stage, -1);
  for (int c = 0; c < chunks; ++c)
    for (int lane = 0; lane < 64; ++lane) {
      uint64_t off;
      int lds;
      if (kc) { off = dma_offset_kc<uint64_t>(c, lane, 0, ext_tile, ld) / 8; lds = dma_lds_chunk_kc(c); }
      else if (oc == OcKind::k128) { off = dma_offset_oc128<uint64_t>(c, lane, 0, ext_tile, ld) / 8; lds = dma_lds_chunk_oc128(c, ext_tile); }
      else { off = dma_offset_oc64<uint64_t>(c, lane, 0, ext_tile, ld) / 8; lds = dma_lds_chunk_oc64(c); }
      const int major = (int)(off / ld), minor = (int)(off % ld);
      for (int d = 0; d < 2; ++d) {
        const int e = kc ? major : minor + d, k = kc ? minor + d : major;
        if (e >= ext_tile || k >= BK) bad("DMA lane fetches (e=%d, k=%d) outside the tile", e, k);
        if (holds[lds + 2 * lane + d] != -1) bad("two DMA lanes land on LDS double %d", lds + 2 * lane + d);
        holds[lds + 2 * lane + d] = e * BK + k;
      }
    }
  for (int e = 0; e < ext_tile; ++e)
    for (int pr = 0; pr < BK / 2; ++pr) {
      int first, second;
      if (kc) { first = frag_lds_kc(e, pr); second = first + 1; }
      else if (oc == OcKind::k128) { first = frag_lds_oc128(e, pr, ext_tile); second = first + (ext_tile + 16); }
      else { first = frag_lds_oc64(e, pr); second = first + 64; }
      if (first < 0 || second >= stage) bad("fragment read of (e=%d, pair=%d) leaves the stage", e, pr);
      if (kc && first % 2 != 0) bad("128-bit fragment read at an odd double");
      if (holds[first] != e * BK + 2 * pr || holds[second] != e * BK + 2 * pr + 1)
        bad("fragment read of (e=%d, pair=%d) finds element %d / %d", e, pr, holds[first], holds[second]);
    }
}

template <int EXT, bool KC>
void check_tail_tile(const char* name, const double* base, int threads, long ld, int o0, int ext, int K, int k_reserve,
                     bool aligned) {
  // the masked remainder tile: load_tile<EXT, KC, VEC = aligned, TAIL = true>
  const size_t limit = footprint(KC, ext, K, ld);
  const int k0 = dma_whole_steps(K, k_reserve) * BK;
  const int pairs = EXT * BK / 2;
  if (pairs % threads != 0) bad("%s: %d pairs do not split over %d threads", name, pairs, threads);
  for (int q = 0; q < pairs; ++q) {
    const PairSource s = aligned ? staged_pair_source<EXT, KC, true, true>(q, ld, o0, ext, k0, K)
                                 : staged_pair_source<EXT, KC, false, true>(q, ld, o0, ext, k0, K);
    {
      // what is kept is the element the pair slot stands for
      const int e = KC ? o0 + (q >> 3) : o0 + 2 * (q % (EXT / 2));
      const int k = KC ? k0 + 2 * (q & 7) : k0 + q / (EXT / 2);
      if (KC) {
        if (e < ext && s.keep_first && s.first != (size_t)e * (size_t)ld + (size_t)k) bad("%s: (%d, %d) displaced", name, e, k);
        if (e < ext && s.keep_second && s.second != (size_t)e * (size_t)ld + (size_t)k + 1) bad("%s: (%d, %d) displaced", name, e, k + 1);
        if (s.keep_first != (k < K) || s.keep_second != (k + 1 < K)) bad("%s: the K mask of pair %d is wrong", name, q);
      } else {
        if (e < ext && s.keep_first && s.first != (size_t)k * (size_t)ld + (size_t)e) bad("%s: (%d, %d) displaced", name, e, k);
        if (e + 1 < ext && s.keep_second && s.second != (size_t)k * (size_t)ld + (size_t)e + 1) bad("%s: (%d, %d) displaced", name, e + 1, k);
        if (s.keep_first != (k < K) || s.keep_second != (k < K)) bad("%s: the K mask of pair %d is wrong", name, q);
      }
    }
    in_range(name, s.first, 1, limit);
    in_range(name, s.second, 1, limit);
    if (s.vec) {
      if (s.second != s.first + 1) bad("%s: a vector pair is not adjacent", name);
      aligned16(name, base, 8 * s.first);
    }
  }
}

// what a launch on the tile DMA promises about its operands
void check_dma_promises(const GemmParams& p, bool a_kc, bool b_kc) {
  if (p.M < 2 || p.N < 2) bad("the pair clamps need extents of at least 2");
  if ((reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B)) % 8) bad("operands are not 8-byte aligned");
  if (p.unaligned != 0 && p.unaligned != 1) bad("unaligned = %d", p.unaligned);
  if (!p.unaligned) {
    if ((reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B)) % 16) bad("operands promised 16-byte aligned are not");
    if (p.lda % 2 || p.ldb % 2) bad("odd leading dimension on operands promised aligned");
    if ((a_kc ? p.K : p.M) % 2 || (b_kc ? p.K : p.N) % 2) bad("odd contiguous extent on operands promised aligned");
  }
  // an output-contiguous operand of odd extent: its last K row must not travel by DMA
  const bool reach_behind = (!a_kc && p.M % 2) || (!b_kc && p.N % 2);
  if (reach_behind && p.k_reserve != 1) bad("an odd output-contiguous extent without the last K row kept back");
}

// all workgroups of one problem on 128x128 direct-to-LDS tiles (8 wavefronts of 64x32)
void check_dma128_problem(const GemmParams& p, bool a_kc, bool b_kc, long long blocks, bool ragged = false) {
  g_context = std::string("dma128 ") + describe(p, a_kc, b_kc);
  check_params(p, a_kc, b_kc);
  if (p.tiles_m != (p.M + 127) / 128 || p.tiles_n != (p.N + 127) / 128) bad("tile counts do not match 128x128 tiles");
  if (blocks != (long long)p.tiles_m * p.tiles_n * p.split_k) bad("%lld workgroups for %d x %d tiles x %d slices", blocks, p.tiles_m, p.tiles_n, p.split_k);
  check_dma_promises(p, a_kc, b_kc);
  const bool aligned = p.unaligned == 0;
  check_dma_k_cover(p);
  check_lds_layout(a_kc, OcKind::k128, 128, 16);
  check_lds_layout(b_kc, OcKind::k128, 128, 16);
  Coverage cov(p.M, p.N, p.split_k);
  ColsumCoverage colsums(p.M, p.split_k);
  const bool want_colsum = !a_kc && p.colsum;
  std::vector<unsigned char> visited((size_t)blocks, 0);
  for (long long b = 0; b < blocks; ++b) {
    const TileCoord tc = tile_of_block(p.tiles_m, p.tiles_n, (int)b);
    if (tc.split < 0 || tc.split >= p.split_k || tc.tile_m < 0 || tc.tile_m >= p.tiles_m || tc.tile_n < 0 || tc.tile_n >= p.tiles_n)
      bad("workgroup %lld maps to slice %d tile (%d, %d)", b, tc.split, tc.tile_m, tc.tile_n);
    const size_t id = ((size_t)tc.split * p.tiles_m + tc.tile_m) * p.tiles_n + tc.tile_n;
    if (visited[id]) bad("tile (%d, %d) of slice %d has two workgroups", tc.tile_m, tc.tile_n, tc.split);
    visited[id] = 1;
    const int m0 = tc.tile_m * 128, n0 = tc.tile_n * 128;
    const DmaSteps ks = dma_k_steps(p.K, p.split_k, p.steps_per_split, tc.split, p.k_reserve);
    check_dma_operand("A tile DMA", p.A, a_kc, OcKind::k128, 128, 16, m0, p.M, p.K, p.lda, ks.kt0, ks.nk_dma, aligned);
    check_dma_operand("B tile DMA", p.B, b_kc, OcKind::k128, 128, 16, n0, p.N, p.K, p.ldb, ks.kt0, ks.nk_dma, aligned);
    if (ks.k_tail) {
      if (a_kc) check_tail_tile<128, true>("A remainder tile", p.A, 512, p.lda, m0, p.M, p.K, p.k_reserve, aligned);
      else check_tail_tile<128, false>("A remainder tile", p.A, 512, p.lda, m0, p.M, p.K, p.k_reserve, aligned);
      if (b_kc) check_tail_tile<128, true>("B remainder tile", p.B, 512, p.ldb, n0, p.N, p.K, p.k_reserve, aligned);
      else check_tail_tile<128, false>("B remainder tile", p.B, 512, p.ldb, n0, p.N, p.K, p.k_reserve, aligned);
    }
    for (int wave = 0; wave < 8; ++wave) {
      const int wm = wave / 4, wn = wave % 4;
      const LiveFragments live = live_fragments(p.M, p.N, m0 + wm * 64, n0 + wn * 32, 4, 2);
      check_write_block(p, 4, 2, m0 + wm * 64, n0 + wn * 32, tc.split, cov, ragged ? &live : nullptr);
    }
    check_colsum(p, a_kc, 128, 512, m0, tc.tile_n, tc.split, want_colsum ? &colsums : nullptr);
  }
  cov.complete();
  if (want_colsum) colsums.complete();
}

void check_dma64_problem(const GemmParams& p, bool b_kc, long long blocks) {
  const bool a_kc = true;
  g_context = std::string("dma64 ") + describe(p, a_kc, b_kc);
  check_params(p, a_kc, b_kc);
  if (p.tiles_m != (p.M + 63) / 64 || p.tiles_n != (p.N + 63) / 64) bad("tile counts do not match 64x64 tiles");
  if (blocks != (long long)p.tiles_m * p.tiles_n * p.split_k) bad("%lld workgroups for %d x %d tiles x %d slices", blocks, p.tiles_m, p.tiles_n, p.split_k);
  check_dma_promises(p, a_kc, b_kc);
  const bool aligned = p.unaligned == 0;
  check_dma_k_cover(p);
  check_lds_layout(true, OcKind::k64, 64, 8);
  check_lds_layout(b_kc, OcKind::k64, 64, 8);
  Coverage cov(p.M, p.N, p.split_k);
  std::vector<unsigned char> visited((size_t)blocks, 0);
  for (long long b = 0; b < blocks; ++b) {
    const TileCoord tc = tile_of_block(p.tiles_m, p.tiles_n, (int)b);
    if (tc.split < 0 || tc.split >= p.split_k || tc.tile_m < 0 || tc.tile_m >= p.tiles_m || tc.tile_n < 0 || tc.tile_n >= p.tiles_n)
      bad("workgroup %lld maps to slice %d tile (%d, %d)", b, tc.split, tc.tile_m, tc.tile_n);
    const size_t id = ((size_t)tc.split * p.tiles_m + tc.tile_m) * p.tiles_n + tc.tile_n;
    if (visited[id]) bad("tile (%d, %d) of slice %d has two workgroups", tc.tile_m, tc.tile_n, tc.split);
    visited[id] = 1;
    const int m0 = tc.tile_m * 64, n0 = tc.tile_n * 64;
    const DmaSteps ks = dma_k_steps(p.K, p.split_k, p.steps_per_split, tc.split, p.k_reserve);
    check_dma_operand("A tile DMA", p.A, true, OcKind::k64, 64, 8, m0, p.M, p.K, p.lda, ks.kt0, ks.nk_dma, aligned);
    check_dma_operand("B tile DMA", p.B, b_kc, OcKind::k64, 64, 8, n0, p.N, p.K, p.ldb, ks.kt0, ks.nk_dma, aligned);
    if (ks.k_tail) {
      check_tail_tile<64, true>("A remainder tile", p.A, 256, p.lda, m0, p.M, p.K, p.k_reserve, aligned);
      if (b_kc) check_tail_tile<64, true>("B remainder tile", p.B, 256, p.ldb, n0, p.N, p.K, p.k_reserve, aligned);
      else check_tail_tile<64, false>("B remainder tile", p.B, 256, p.ldb, n0, p.N, p.K, p.k_reserve, aligned);
    }
    for (int wave = 0; wave < 4; ++wave) check_write_block(p, 2, 2, m0 + (wave >> 1) * 32, n0 + (wave & 1) * 32, tc.split, cov);
  }
  cov.complete();
}

// ---- register-staged kernels -------------------------------------------------------------------------
template <int EXT, bool KC, bool VEC>
void check_staged_operand(const char* name, const double* base, long ld, int o0, int ext, int K, const StagedSteps& ks) {
  const size_t limit = footprint(KC, ext, K, ld);
  if (o0 < 0 || o0 >= ext) bad("%s tile origin %d outside [0, %d)", name, o0, ext);
  if (VEC && (reinterpret_cast<uintptr_t>(base) % 16 || ld % 2 || (ext % 2 && !KC) || (K % 2 && KC)))
    bad("%s: 16-byte loads on an operand that does not promise aligned pairs", name);
  const int steps[3] = {ks.kt0, (ks.nk < ks.nk_full ? ks.nk : ks.nk_full) - 1, ks.nk > ks.nk_full ? ks.nk_full : -1};
  for (int which = 0; which < 3; ++which) {
    const int kt = steps[which];
    if (kt < ks.kt0 || kt >= ks.nk) continue;
    const bool tail = kt >= ks.nk_full;
    for (int q = 0; q < EXT * BK / 2; ++q) {
      const PairSource s = tail ? staged_pair_source<EXT, KC, VEC, true>(q, ld, o0, ext, kt * BK, K)
                                : staged_pair_source<EXT, KC, VEC, false>(q, ld, o0, ext, kt * BK, K);
      in_range(name, s.first, 1, limit);
      in_range(name, s.second, 1, limit);
      if (s.vec) {
        if (s.second != s.first + 1) bad("%s: a vector pair is not adjacent", name);
        aligned16(name, base, 8 * s.first);
      }
    }
  }
}

template <int EXT>
void check_staged_operand_rt(const char* name, bool kc, bool vec, const double* base, long ld, int o0, int ext, int K,
                             const StagedSteps& ks) {
  if (kc && vec) check_staged_operand<EXT, true, true>(name, base, ld, o0, ext, K, ks);
  else if (kc) check_staged_operand<EXT, true, false>(name, base, ld, o0, ext, K, ks);
  else if (vec) check_staged_operand<EXT, false, true>(name, base, ld, o0, ext, K, ks);
  else check_staged_operand<EXT, false, false>(name, base, ld, o0, ext, K, ks);
}

void check_staged_problem(const GemmParams& p, int bm, int bn, int wgm, int wgn, bool a_kc, bool b_kc, bool vec,
                          long long blocks) {
  char head[64];
  std::snprintf(head, sizeof(head), "staged %dx%d vec=%d ", bm, bn, (int)vec);
  g_context = std::string(head) + describe(p, a_kc, b_kc);
  check_params(p, a_kc, b_kc);
  if (bm != bn || (bm != 32 && bm != 128)) bad("unexpected tile %d x %d", bm, bn);
  if (p.tiles_m != (p.M + bm - 1) / bm || p.tiles_n != (p.N + bn - 1) / bn) bad("tile counts do not match the tile size");
  if (blocks != (long long)p.tiles_m * p.tiles_n * p.split_k) bad("%lld workgroups for %d x %d tiles x %d slices", blocks, p.tiles_m, p.tiles_n, p.split_k);
  check_staged_k_cover(p);
  const int wm_rows = bm / wgm, wn_cols = bn / wgn;
  const int tm = wm_rows / 16, tn = wn_cols / 16;
  Coverage cov(p.M, p.N, p.split_k);
  ColsumCoverage colsums(p.M, p.split_k);
  const bool want_colsum = !a_kc && p.colsum;
  std::vector<unsigned char> visited((size_t)blocks, 0);
  for (long long b = 0; b < blocks; ++b) {
    const TileCoord tc = tile_of_block(p.tiles_m, p.tiles_n, (int)b);
    if (tc.split < 0 || tc.split >= p.split_k || tc.tile_m < 0 || tc.tile_m >= p.tiles_m || tc.tile_n < 0 || tc.tile_n >= p.tiles_n)
      bad("workgroup %lld maps to slice %d tile (%d, %d)", b, tc.split, tc.tile_m, tc.tile_n);
    const size_t id = ((size_t)tc.split * p.tiles_m + tc.tile_m) * p.tiles_n + tc.tile_n;
    if (visited[id]) bad("tile (%d, %d) of slice %d has two workgroups", tc.tile_m, tc.tile_n, tc.split);
    visited[id] = 1;
    const int m0 = tc.tile_m * bm, n0 = tc.tile_n * bn;
    const StagedSteps ks = staged_k_steps(p.K, p.split_k, p.steps_per_split, tc.split);
    if (p.K > 0) {
      switch (bm) {
        case 32:
          check_staged_operand_rt<32>("A tile load", a_kc, vec, p.A, p.lda, m0, p.M, p.K, ks);
          check_staged_operand_rt<32>("B tile load", b_kc, vec, p.B, p.ldb, n0, p.N, p.K, ks);
          break;
        default:
          check_staged_operand_rt<128>("A tile load", a_kc, vec, p.A, p.lda, m0, p.M, p.K, ks);
          check_staged_operand_rt<128>("B tile load", b_kc, vec, p.B, p.ldb, n0, p.N, p.K, ks);
          break;
      }
    }
    for (int wave = 0; wave < wgm * wgn; ++wave)
      check_write_block(p, tm, tn, m0 + (wave / wgn) * wm_rows, n0 + (wave % wgn) * wn_cols, tc.split, cov);
    check_colsum(p, a_kc, bm, wgm * wgn * 64, m0, tc.tile_n, tc.split, want_colsum ? &colsums : nullptr);
  }
  cov.complete();
  if (want_colsum) colsums.complete();
}

// ---- reduction of the slices ---------------------------------------------------------------------------------
void check_split_reduce(const GemmParams& p, long long blocks) {
  g_context = std::string("split_reduce ") + describe(p, false, false);
  const size_t mn = (size_t)p.M * p.N;
  if (p.split_k < 2) bad("reduction of an unsplit contraction");
  if ((size_t)blocks * 256 < mn) bad("%lld workgroups of 256 threads for %zu outputs", blocks, mn);
  if (p.colsum && (size_t)blocks * 256 < (size_t)p.M) bad("too few threads for %d column sums", p.M);
  // thread i adds ws[i + s * mn], s < split_k, and stores C[row, col]
  in_range("slice read", (mn - 1) + (size_t)(p.split_k - 1) * mn, 1, (size_t)p.split_k * mn);
  if (p.colsum) {
    if (p.ws_colsum != p.ws + (size_t)p.split_k * mn) bad("column sums do not follow the partial products");
    in_range("slice column-sum read", (size_t)(p.M - 1) + (size_t)(p.split_k - 1) * p.M, 1, (size_t)p.split_k * p.M);
  }
  const size_t c_limit = (size_t)(p.M - 1) * (size_t)p.ldc + (size_t)p.N;
  in_range("reduced store", (size_t)(p.M - 1) * p.ldc + (p.N - 1), 1, c_limit);
}

// the workspace regions of the members of a group: inside the capacity, pairwise disjoint
void check_group_workspace(const GemmGroup& g) {
  const double* base = nullptr;
  for (int i = 0; i < g.count; ++i)
    if (g.p[i].split_k > 1 && (!base || g.p[i].ws < base)) base = g.p[i].ws;
  std::vector<std::pair<size_t, size_t>> regions;
  for (int i = 0; i < g.count; ++i) {
    const GemmParams& p = g.p[i];
    if (p.split_k <= 1) continue;
    const size_t first = (size_t)(p.ws - base);
    const size_t size = (size_t)p.split_k * ((size_t)p.M * p.N + (size_t)p.M);
    if (first + size > p.ws_capacity) bad("member %d's slices end at %zu of a workspace of %zu doubles", i, first + size, p.ws_capacity);
    for (auto& r : regions)
      if (first < r.first + r.second && r.first < first + size) bad("members share workspace doubles");
    regions.push_back({first, size});
  }
}

void check_group_blocks(const GemmGroup& g, const int* first, long long blocks) {
  if (g.count < 1 || g.count > kMaxGroup) bad("a group of %d", g.count);
  if (first[0] != 0 || first[g.count] != blocks) bad("the members' workgroup ranges do not tile the grid");
  for (int i = 0; i < g.count; ++i)
    if (first[i + 1] < first[i]) bad("workgroup ranges are not monotonic");
  for (long long b = 0; b < blocks; ++b) {
    const int i = group_member_of_block(first, g.count, (int)b);
    if (b < first[i] || b >= first[i + 1]) bad("workgroup %lld is assigned to member %d outside its range", b, i);
  }
}

std::string key_of(const GemmLaunch& l) {
  std::string k((const char*)&l.kernel, sizeof(l.kernel));
  auto add = [&](const void* p, size_t n) { k.append((const char*)p, n); };
  add(&l.bm, sizeof(int)); add(&l.wgm, sizeof(int)); add(&l.a_kc, 1); add(&l.b_kc, 1); add(&l.vec, 1);
  add(&l.blocks, sizeof(l.blocks)); add(&l.first_blocks, sizeof(int));
  auto add_params = [&](const GemmParams& p) {
    // the pointers matter only through their alignment
    const long fields[] = {p.M, p.N, p.K, p.lda, p.ldb, p.ldc, p.epilogue, p.ldmask, p.tiles_m, p.tiles_n, p.split_k,
                           p.steps_per_split, (long)(reinterpret_cast<uintptr_t>(p.A) % 16), (long)(reinterpret_cast<uintptr_t>(p.B) % 16),
                           p.colsum != nullptr, p.sgd_parm != nullptr, p.divisor_reciprocal != 0.0, (long)p.ws_capacity,
                           p.mask != nullptr, p.bias != nullptr};
    add(fields, sizeof(fields));
  };
  if (l.p) add_params(*l.p);
  if (l.p2) add_params(*l.p2);
  if (l.group) {
    add(&l.group->count, sizeof(int));
    add(l.group->first_block, sizeof(l.group->first_block));
    add(l.group->layout, sizeof(l.group->layout));
    for (int i = 0; i < l.group->count; ++i) {
      add_params(l.group->p[i]);
      const long off = (long)(l.group->p[i].ws - l.group->p[0].ws);
      add(&off, sizeof(off));
    }
  }
  return k;
}

}  // namespace

void observe_gemm_launch(const GemmLaunch& l) {
  if (l.blocks <= 0 || l.blocks > 0x7fffffffLL) {
    g_context = kernel_name(l.kernel);
    bad("grid of %lld workgroups", l.blocks);
  }
  if (!g_seen.insert(key_of(l)).second) {  // verified before: the model is a pure function of these
    ++g_skipped_repeats;
    return;
  }
  switch (l.kernel) {
    case GemmKernel::kStaged:
      check_staged_problem(*l.p, l.bm, l.bn, l.wgm, l.wgn, l.a_kc, l.b_kc, l.vec, l.blocks);
      ++g_staged_by_tile[l.bm == 32 ? 0 : 1];
      break;
    case GemmKernel::kDma128:
      check_dma128_problem(*l.p, l.a_kc, l.b_kc, l.blocks);
      break;
    case GemmKernel::kDma64:
      check_dma64_problem(*l.p, l.b_kc, l.blocks);
      break;
    case GemmKernel::kSplitReduce:
      check_split_reduce(*l.p, l.blocks);
      break;
    case GemmKernel::kDma128Pair: {
      g_context = "dma128_pair";
      const long long b1 = l.first_blocks, b2 = l.blocks - l.first_blocks;
      if (b1 <= 0 || b2 < b1) bad("pair of %lld + %lld workgroups", b1, b2);
      std::vector<unsigned char> seen1((size_t)b1, 0), seen2((size_t)b2, 0);
      for (long long b = 0; b < l.blocks; ++b) {
        const PairSlot s = pair_slot_of_block((int)b, (int)b1);
        std::vector<unsigned char>& seen = s.problem == 0 ? seen1 : seen2;
        if (s.block < 0 || (size_t)s.block >= seen.size()) bad("workgroup %lld maps to block %d of problem %d", b, s.block, s.problem);
        if (seen[s.block]) bad("block %d of problem %d has two workgroups", s.block, s.problem);
        seen[s.block] = 1;
        // the XCD-aware tile walk relies on a workgroup's number mod 8 being its XCD
        if ((s.block & 7) != (b & 7)) bad("workgroup %lld runs block %d: another XCD than the tile walk assumes", b, s.block);
      }
      if (l.p->split_k != 1 || l.p2->split_k != 1) bad("a paired product is split");
      check_dma128_problem(*l.p, true, false, b1);
      check_dma128_problem(*l.p2, false, false, b2);
      break;
    }
    case GemmKernel::kDma128Group: {
      g_context = "dma128_group";
      check_group_blocks(*l.group, l.group->first_block, l.blocks);
      check_group_workspace(*l.group);
      for (int i = 0; i < l.group->count; ++i)
        check_dma128_problem(l.group->p[i], false, false, l.group->first_block[i + 1] - l.group->first_block[i], true);
      break;
    }
    case GemmKernel::kStagedGroup:
    case GemmKernel::kStagedMixedGroup: {
      g_context = kernel_name(l.kernel);
      check_group_blocks(*l.group, l.group->first_block, l.blocks);
      check_group_workspace(*l.group);
      for (int i = 0; i < l.group->count; ++i) {
        const bool a_kc = l.kernel == GemmKernel::kStagedMixedGroup ? (l.group->layout[i] & 1) != 0 : l.a_kc;
        const bool b_kc = l.kernel == GemmKernel::kStagedMixedGroup ? (l.group->layout[i] & 2) != 0 : l.b_kc;
        check_staged_problem(l.group->p[i], 32, 32, 2, 2, a_kc, b_kc, l.group->p[i].unaligned == 0,
                             l.group->first_block[i + 1] - l.group->first_block[i]);
      }
      break;
    }
    case GemmKernel::kSplitReduceGroup: {
      g_context = "split_reduce_group";
      check_group_blocks(*l.group, l.group->first_reduce_block, l.blocks);
      for (int i = 0; i < l.group->count; ++i) {
        const long long nb = l.group->first_reduce_block[i + 1] - l.group->first_reduce_block[i];
        if (l.group->p[i].split_k > 1) check_split_reduce(l.group->p[i], nb);
        else if (nb != 0) bad("an unsplit member has %lld reduction workgroups", nb);
      }
      break;
    }
  }
  ++g_checked[(int)l.kernel];
  if (l.p && l.p->split_k > 1) ++g_sliced[(int)l.kernel];
  if (l.p && (l.kernel == GemmKernel::kDma128 || l.kernel == GemmKernel::kDma64 || l.kernel == GemmKernel::kDma128Pair) &&
      (l.p->unaligned || (l.p2 && l.p2->unaligned))) {
    ++g_unaligned[(int)l.kernel];
    if (l.p->k_reserve || (l.p2 && l.p2->k_reserve)) ++g_reserved[(int)l.kernel];
  }
  if (l.group) {
    bool any = false, reserved = false;
    for (int i = 0; i < l.group->count; ++i) {
      any = any || l.group->p[i].unaligned;
      reserved = reserved || l.group->p[i].k_reserve;
    }
    if (any) ++g_unaligned[(int)l.kernel];
    if (reserved) ++g_reserved[(int)l.kernel];
  }
}

}  // namespace rst

// ---- what the drivers read -------------------------------------------------------------------------------
extern "C" long address_model_checked(int kernel) { return kernel >= 0 && kernel < 16 ? rst::g_checked[kernel] : 0; }
extern "C" long address_model_staged_checked(int tile) { return rst::g_staged_by_tile[tile == 32 ? 0 : 1]; }
extern "C" long address_model_sliced(int kernel) { return kernel >= 0 && kernel < 16 ? rst::g_sliced[kernel] : 0; }
extern "C" long address_model_unaligned(int kernel) { return kernel >= 0 && kernel < 16 ? rst::g_unaligned[kernel] : 0; }
extern "C" long address_model_reserved(int kernel) { return kernel >= 0 && kernel < 16 ? rst::g_reserved[kernel] : 0; }
extern "C" long address_model_repeats() { return rst::g_skipped_repeats; }
extern "C" long long address_model_lane_checks() { return rst::g_lane_checks; }
extern "C" const char* address_model_kernel_name(int kernel) { return rst::kernel_name((rst::GemmKernel)kernel); }
