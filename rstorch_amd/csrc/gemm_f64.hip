// FP64 contraction kernels for gfx950 built on v_mfma_f64_16x16x4_f64.
//
// One kernel template covers the three products of a Linear layer
//   forward        Z[B,N]  = X[B,K] . W[N,K]^T        (A and B contraction-contiguous)
//   weight grad    dW[N,K] = G[B,N]^T . X[B,K]        (A and B output-contiguous)
//   input grad     dX[B,K] = G[B,N] . W[N,K]          (A contraction-contiguous, B output-contiguous)
// without materialising a transpose: the operand layout only changes how a tile is copied
// into LDS and which LDS stride the MFMA fragments are read with.
//
// Tiling: 256 threads = 4 wavefronts in a 2x2 grid, each owning a (BM/2)x(BN/2) block of
// 16x16 MFMA tiles held in registers; K advances in steps of 16 through two LDS stages, the
// global loads of step k+1 are in flight while step k is multiplied.
//
// MFMA register layout (64 lanes): A fragment lane l holds A[l%16][l/16], B fragment lane l
// holds B[l/16][l%16], and accumulator register r of lane l holds D[4*r + l/16][l%16].
#include "common.h"

namespace rst {
namespace {

typedef double v4d __attribute__((ext_vector_type(4)));
typedef double v2d __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;
constexpr int BK = 16;

struct GemmParams {
  const double* A;
  const double* B;
  double* C;
  int M, N, K;
  long lda, ldb, ldc;
  int epilogue;
  const double* bias;
  double divisor;
  const double* mask;
  long ldmask;
  int a_vec, b_vec;  // 16-byte global loads are legal for the operand
  int tiles_m, tiles_n;
};

// LDS geometry of one operand tile of EXT rows/cols by BK contraction steps.
//   contraction-contiguous: [EXT][BK + 2]   (stride 18 doubles: fragment reads hit 32 distinct
//                                            8-byte banks per half wave)
//   output-contiguous:      [BK][EXT + 16]  (stride = 16 mod 32 doubles, same property)
template <int EXT, bool KC>
struct TileGeom {
  static constexpr int stride = KC ? (BK + 2) : (EXT + 16);
  static constexpr int size = KC ? EXT * (BK + 2) : BK * (EXT + 16);
  static constexpr int loads = EXT * BK / 2 / kThreads;  // v2d loads per thread per tile
  static_assert(EXT * BK / 2 % kThreads == 0, "tile must split evenly over the block");
};

// Copy one operand tile global -> registers.  `ext0` is the first row/col of the tile along
// the output dimension (limit `ext_n`), `k0` the first contraction index (limit `k_n`).
template <int EXT, bool KC>
__device__ __forceinline__ void load_tile(v2d* __restrict__ reg,
                                          const double* __restrict__ base, long ld, int ext0,
                                          int ext_n, int k0, int k_n, int vec, int tid) {
  constexpr int L = TileGeom<EXT, KC>::loads;
#pragma unroll
  for (int u = 0; u < L; ++u) {
    const int q = tid + u * kThreads;
    int e, k;        // element coordinates of the first of the two doubles
    bool contiguous_is_k = KC;
    if (KC) {
      e = ext0 + (q >> 3);           // BK/2 = 8 pairs per row
      k = k0 + 2 * (q & 7);
    } else {
      k = k0 + q / (EXT / 2);
      e = ext0 + 2 * (q % (EXT / 2));
    }
    v2d v = {0.0, 0.0};
    if (contiguous_is_k) {
      if (e < ext_n) {
        const double* p = base + (size_t)e * ld + k;
        if (vec) {
          if (k + 1 < k_n) v = *reinterpret_cast<const v2d*>(p);
          else if (k < k_n) v.x = p[0];
        } else {
          if (k < k_n) v.x = p[0];
          if (k + 1 < k_n) v.y = p[1];
        }
      }
    } else {
      if (k < k_n) {
        const double* p = base + (size_t)k * ld + e;
        if (vec) {
          if (e + 1 < ext_n) v = *reinterpret_cast<const v2d*>(p);
          else if (e < ext_n) v.x = p[0];
        } else {
          if (e < ext_n) v.x = p[0];
          if (e + 1 < ext_n) v.y = p[1];
        }
      }
    }
    reg[u] = v;
  }
}

// Registers -> LDS stage.
template <int EXT, bool KC>
__device__ __forceinline__ void store_tile(double* __restrict__ lds,
                                           const v2d* __restrict__ reg, int tid) {
  constexpr int L = TileGeom<EXT, KC>::loads;
  constexpr int S = TileGeom<EXT, KC>::stride;
#pragma unroll
  for (int u = 0; u < L; ++u) {
    const int q = tid + u * kThreads;
    int off;
    if (KC) off = (q >> 3) * S + 2 * (q & 7);
    else off = (q / (EXT / 2)) * S + 2 * (q % (EXT / 2));
    *reinterpret_cast<v2d*>(lds + off) = reg[u];
  }
}

// LDS -> MFMA fragment: element (e, k) of the tile, e = output index inside the tile.
template <int EXT, bool KC>
__device__ __forceinline__ double read_frag(const double* __restrict__ lds, int e, int k) {
  constexpr int S = TileGeom<EXT, KC>::stride;
  return KC ? lds[e * S + k] : lds[k * S + e];
}

template <int BM, int BN, bool A_KC, bool B_KC>
__global__ __launch_bounds__(kThreads, 2) void gemm_f64_mfma(const GemmParams p) {
  using GA = TileGeom<BM, A_KC>;
  using GB = TileGeom<BN, B_KC>;
  constexpr int WM = BM / 2, WN = BN / 2;    // per-wavefront block
  constexpr int TM = WM / 16, TN = WN / 16;  // MFMA tiles per wavefront
  static_assert(WM % 16 == 0 && WN % 16 == 0, "wave block must be whole MFMA tiles");

  __shared__ __attribute__((aligned(16))) double lds_a[2][GA::size];
  __shared__ __attribute__((aligned(16))) double lds_b[2][GB::size];

  // Workgroups are handed to the 8 XCDs round-robin; renumber them so that each XCD (and
  // its private L2) works on one compact patch of the tile grid, then walk the patch in
  // groups of 8 tile rows so that concurrently resident workgroups share operand panels.
  const int n_blocks = gridDim.x;
  int logical;
  {
    const int pid = blockIdx.x;
    const int xcd = pid & 7, local = pid >> 3;
    const int base = n_blocks >> 3, rem = n_blocks & 7;
    logical = xcd * base + (xcd < rem ? xcd : rem) + local;
  }
  int tile_m, tile_n;
  {
    constexpr int GROUP = 8;
    const int group_size = GROUP * p.tiles_n;
    const int group = logical / group_size;
    const int first_m = group * GROUP;
    const int gm = (p.tiles_m - first_m) < GROUP ? (p.tiles_m - first_m) : GROUP;
    const int in_group = logical - group * group_size;
    tile_m = first_m + in_group % gm;
    tile_n = in_group / gm;
  }
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int lr = lane & 15, lk = lane >> 4;

  v4d acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = (v4d){0.0, 0.0, 0.0, 0.0};

  v2d ra[GA::loads], rb[GB::loads];
  const int nk = (p.K + BK - 1) / BK;

  load_tile<BM, A_KC>(ra, p.A, p.lda, m0, p.M, 0, p.K, p.a_vec, tid);
  load_tile<BN, B_KC>(rb, p.B, p.ldb, n0, p.N, 0, p.K, p.b_vec, tid);
  store_tile<BM, A_KC>(lds_a[0], ra, tid);
  store_tile<BN, B_KC>(lds_b[0], rb, tid);
  __syncthreads();

  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    const bool more = kt + 1 < nk;
    if (more) {
      load_tile<BM, A_KC>(ra, p.A, p.lda, m0, p.M, (kt + 1) * BK, p.K, p.a_vec, tid);
      load_tile<BN, B_KC>(rb, p.B, p.ldb, n0, p.N, (kt + 1) * BK, p.K, p.b_vec, tid);
    }
    const double* __restrict__ sa = lds_a[cur];
    const double* __restrict__ sb = lds_b[cur];
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
    if (more) {
      store_tile<BM, A_KC>(lds_a[cur ^ 1], ra, tid);
      store_tile<BN, B_KC>(lds_b[cur ^ 1], rb, tid);
    }
    __syncthreads();
  }

  // Epilogue: accumulator register r of this lane is row 4*r + lk, column lr of its tile.
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = n0 + wn * WN + j * 16 + lr;
      if (col >= p.N) continue;
      double bias = 0.0;
      if (p.epilogue == EPI_BIAS || p.epilogue == EPI_BIAS_RELU) bias = p.bias[col];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = m0 + wm * WM + i * 16 + 4 * r + lk;
        if (row >= p.M) continue;
        double v = acc[i][j][r];
        switch (p.epilogue) {
          case EPI_BIAS: v = v + bias; break;
          case EPI_BIAS_RELU: v = fmax(v + bias, 0.0); break;
          case EPI_RELU: v = fmax(v, 0.0); break;
          case EPI_DIVIDE: v = v / p.divisor; break;
          case EPI_MASK: v = v * (p.mask[(size_t)row * p.ldmask + col] > 0.0 ? 1.0 : 0.0); break;
          default: break;
        }
        p.C[(size_t)row * p.ldc + col] = v;
      }
    }
  }
}

template <int BM, int BN, bool A_KC, bool B_KC>
int launch_one(hipStream_t stream, GemmParams p) {
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const long long blocks = (long long)p.tiles_m * p.tiles_n;
  if (blocks > 0x7fffffffLL) return fail(RST_ERR_UNSUPPORTED, "contraction grid too large");
  hipLaunchKernelGGL((gemm_f64_mfma<BM, BN, A_KC, B_KC>), dim3((unsigned)blocks), dim3(kThreads), 0,
                     stream, p);
  RST_HIP(hipGetLastError());
  return RST_OK;
}

template <bool A_KC, bool B_KC>
int launch_layout(hipStream_t stream, const GemmParams& p) {
  // Largest tile that still gives the 256 compute units about two workgroups each; small
  // problems fall through to smaller tiles for parallelism.
  auto tiles = [&](int bm, int bn) {
    return (long long)((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn);
  };
  if (tiles(128, 128) >= 256) return launch_one<128, 128, A_KC, B_KC>(stream, p);
  if (tiles(64, 64) >= 256) return launch_one<64, 64, A_KC, B_KC>(stream, p);
  return launch_one<32, 32, A_KC, B_KC>(stream, p);
}

}  // namespace

int launch_gemm(hipStream_t stream, const GemmDesc& d) {
  if (d.M <= 0 || d.N <= 0) return RST_OK;
  GemmParams p;
  p.A = d.A; p.B = d.B; p.C = d.C;
  p.M = d.M; p.N = d.N; p.K = d.K;
  p.lda = d.lda; p.ldb = d.ldb; p.ldc = d.ldc;
  p.epilogue = d.epilogue;
  p.bias = d.bias; p.divisor = d.divisor; p.mask = d.mask; p.ldmask = d.ldmask;
  auto vec_ok = [](const double* ptr, long ld, int contiguous_extent) {
    return (reinterpret_cast<uintptr_t>(ptr) % 16 == 0) && (ld % 2 == 0) &&
           (contiguous_extent % 2 == 0);
  };
  p.a_vec = vec_ok(d.A, d.lda, d.a_kc ? d.K : d.M) ? 1 : 0;
  p.b_vec = vec_ok(d.B, d.ldb, d.b_kc ? d.K : d.N) ? 1 : 0;
  p.tiles_m = p.tiles_n = 0;
  if (d.a_kc && d.b_kc) return launch_layout<true, true>(stream, p);
  if (!d.a_kc && !d.b_kc) return launch_layout<false, false>(stream, p);
  if (d.a_kc && !d.b_kc) return launch_layout<true, false>(stream, p);
  return launch_layout<false, true>(stream, p);
}

}  // namespace rst
