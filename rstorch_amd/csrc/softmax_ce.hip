// Row softmax and the fused softmax + cross-entropy forward/gradient kernel.
//
// Arithmetic follows the reference literally (src/module/activation/softmax.rs:45-53,
// src/loss/cross_entropy.rs:34-47): m = max of the row folded from the lowest finite double,
// e = exp(z - m), s = sum e, p = e / s (a true division), loss term = truth * ln(p),
// gradient = -(truth - p).  Where truth is exactly 0 the term is 0 unless p is 0 or NaN
// (0 * -inf = NaN in the reference), so ln is only evaluated where truth is non-zero.
//
// Rows of up to 2048 logits are kept in registers between the three phases, so each logit and
// each truth value is read once and each gradient written once: 24 bytes per logit.  Wider rows
// are walked twice (running maximum and sum first, then the probabilities); the second walk goes
// backwards so that the most recently read part of the row is still in L2.
#include <cfloat>

#include "argmax.h"
#include "common.h"

namespace rst {
namespace {

typedef double v2d __attribute__((ext_vector_type(2)));

// the fused classifier head: the most classes it takes
constexpr int kHeadCols = 16;

struct MaxOp {
  __device__ static double apply(double a, double b) { return a < b ? b : a; }
};
struct SumOp {
  __device__ static double apply(double a, double b) { return a + b; }
};

// Reduction over the TPR consecutive threads that share a row.  Every thread of the group
// receives the same bits.  `scratch` needs TPR/64 doubles per row group when TPR > 64.
template <int TPR, class Op>
__device__ __forceinline__ double group_reduce(double v, double* scratch) {
  constexpr int W = TPR < 64 ? TPR : 64;
#pragma unroll
  for (int off = W / 2; off > 0; off >>= 1) v = Op::apply(v, __shfl_xor(v, off));
  if (TPR > 64) {
    constexpr int NW = TPR / 64;
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) scratch[wave] = v;
    __syncthreads();
    double r = scratch[0];
#pragma unroll 1
    for (int w = 1; w < NW; ++w) r = Op::apply(r, scratch[w]);
    v = r;
  }
  return v;
}

// The thread that finishes a loss also stores it, the NaN flag and (if counted) the arg-max hits in
// pinned host memory: in plain words (read after a stream synchronisation) and, when the launch has
// a ticket, in the 16-byte records that the host polls (see store_result_slot).
__device__ __forceinline__ void publish(const LossMirror& mirror, double loss, int nan_flag, bool counted,
                                        unsigned long long hits) {
  if (mirror.loss) {
    mirror.loss[0] = loss;
    mirror.flags[1] = nan_flag;
  }
  if (counted) mirror.hits[0] = hits;
  if (mirror.slots) {
    if (counted) store_result_slot(mirror.slots + 1, (double)0, hits, true, 0u, mirror.ticket);
    store_result_slot(mirror.slots, loss, 0ull, false, (unsigned)nan_flag, mirror.ticket);
  }
}

__device__ __forceinline__ double loss_term(double truth, double p) {
  if (truth == 0.0) return p > 0.0 ? 0.0 : __builtin_nan("");
  return truth * log(p);
}

// Register-resident rows: TPR threads per row, IPT vectors of VEC doubles per thread, BLOCK / TPR
// rows per workgroup.  SOLO: the whole batch (at most 64 rows) sits in one workgroup of 1024
// threads, which then also finishes the loss the way loss_reduce_kernel would (same order of
// additions, same bits), so that a small batch needs one launch instead of two.
// ACC (rows of at most 64 threads): the kernel also counts the rows whose first arg-max agrees between
// logits and truth (utils.rs:44-65), which a training loop asks for right after the loss - one launch
// and one round trip instead of two.  With SOLO the count goes out with the loss; otherwise every
// workgroup leaves its count in mirror.group_hits[its number] and loss_reduce_kernel adds them up
// (one word per workgroup: thousands of additions to one word would queue up behind each other).
template <int TPR, int IPT, int VEC, bool CE, int BLOCK = 256, bool SOLO = false, bool ACC = false>
__global__ __launch_bounds__(BLOCK) void softmax_rows_kernel(
    const double* __restrict__ z, const double* __restrict__ truth, double* __restrict__ grad,
    double* __restrict__ prob, double* __restrict__ row_loss, double* __restrict__ loss,
    int* __restrict__ flags, size_t rows, size_t cols, LossMirror mirror) {
  static_assert(BLOCK % TPR == 0 && (TPR <= 64 || BLOCK == TPR) && (!SOLO || (CE && BLOCK == 1024)) &&
                (!ACC || (CE && TPR <= 64)), "unsupported shape");
  constexpr int RPB = BLOCK / TPR;
  __shared__ double red[3][TPR > 64 ? TPR / 64 : 1];

  const int sub = threadIdx.x % TPR;
  const size_t row = (size_t)blockIdx.x * RPB + threadIdx.x / TPR;
  const bool row_ok = row < rows;
  const size_t base = row * cols;

  double x[IPT][VEC];
  bool saw_nan = false;
  double mx = -DBL_MAX;
  // (ACC) this thread's first maximum of the logits and of the truth row: value and column
  double best_z = 0.0, best_t = 0.0;
  unsigned arg_z = kNoIndex, arg_t = kNoIndex;
#pragma unroll
  for (int i = 0; i < IPT; ++i) {
    const size_t c = (size_t)(sub + i * TPR) * VEC;
    const bool ok = row_ok && c < cols;
    if (VEC == 2) {
      v2d v = {0.0, 0.0};
      if (ok) v = __builtin_nontemporal_load(reinterpret_cast<const v2d*>(z + base + c));
      x[i][0] = v.x;
      x[i][VEC - 1] = v.y;
    } else {
      x[i][0] = ok ? z[base + c] : 0.0;
    }
    if (ok) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        saw_nan |= (x[i][e] != x[i][e]);
        mx = MaxOp::apply(mx, x[i][e]);
        if (ACC) argmax_step(best_z, arg_z, x[i][e], c + e);
      }
    }
  }
  mx = group_reduce<TPR, MaxOp>(mx, red[0]);

  double s = 0.0;
#pragma unroll
  for (int i = 0; i < IPT; ++i) {
    const size_t c = (size_t)(sub + i * TPR) * VEC;
    const bool ok = row_ok && c < cols;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      double ev = ok ? exp(x[i][e] - mx) : 0.0;
      x[i][e] = ev;
      s += ev;
    }
  }
  s = group_reduce<TPR, SumOp>(s, red[1]);

  double lsum = 0.0;
#pragma unroll
  for (int i = 0; i < IPT; ++i) {
    const size_t c = (size_t)(sub + i * TPR) * VEC;
    const bool ok = row_ok && c < cols;
    if (!ok) continue;
    double p[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) p[e] = x[i][e] / s;
    if (CE) {
      double t[VEC];
      if (VEC == 2) {
        v2d tv = __builtin_nontemporal_load(reinterpret_cast<const v2d*>(truth + base + c));
        t[0] = tv.x;
        t[VEC - 1] = tv.y;
      } else {
        t[0] = truth[base + c];
      }
      double g[VEC];
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        lsum += loss_term(t[e], p[e]);
        g[e] = -(t[e] - p[e]);
        if (ACC) argmax_step(best_t, arg_t, t[e], c + e);
      }
      if (VEC == 2) {
        v2d gv = {g[0], g[VEC - 1]};
        __builtin_nontemporal_store(gv, reinterpret_cast<v2d*>(grad + base + c));
      } else {
        grad[base + c] = g[0];
      }
    }
    if (prob) {
      if (VEC == 2) {
        v2d pv = {p[0], p[VEC - 1]};
        *reinterpret_cast<v2d*>(prob + base + c) = pv;
      } else {
        prob[base + c] = p[0];
      }
    }
  }
  if (CE && SOLO) {
    __shared__ double solo_sum[64];
    __shared__ int solo_nan;
    __shared__ unsigned solo_hits;
    lsum = group_reduce<TPR, SumOp>(lsum, red[2]);
    if (threadIdx.x < 64) solo_sum[threadIdx.x] = 0.0;
    if (threadIdx.x == 0) { solo_nan = 0; solo_hits = 0; }
    if (ACC) {  // the TPR threads of a row (one wavefront or part of one) agree on the two columns
      constexpr int W = TPR < 64 ? TPR : 64;
#pragma unroll
      for (int off = W / 2; off > 0; off >>= 1) {
        argmax_combine(best_z, arg_z, __shfl_xor(best_z, off), __shfl_xor(arg_z, off));
        argmax_combine(best_t, arg_t, __shfl_xor(best_t, off), __shfl_xor(arg_t, off));
      }
    }
    __syncthreads();
    if (sub == 0 && row_ok) solo_sum[row] = lsum;
    if (saw_nan) atomicOr(&solo_nan, 1);
    if (ACC && sub == 0 && row_ok && arg_z == arg_t) atomicAdd(&solo_hits, 1u);  // (an integer count: any order)
    __syncthreads();
    if (threadIdx.x < 64) {
      // loss_reduce_kernel on at most 64 rows: one value per lane of wavefront 0, the butterfly
      // of group_reduce, then the (zero) sums of the other fifteen wavefronts
      double v = solo_sum[threadIdx.x];
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) v = SumOp::apply(v, __shfl_xor(v, off));
      if (threadIdx.x == 0) {
        v = v + 0.0;
        const double l = -v / (double)rows;
        loss[0] = l;
        flags[1] = solo_nan;
        publish(mirror, l, solo_nan, ACC, solo_hits);
      }
    }
  } else if (CE) {
    lsum = group_reduce<TPR, SumOp>(lsum, red[2]);
    if (sub == 0 && row_ok) row_loss[row] = lsum;
    if (saw_nan) atomicOr(&flags[0], 1);
    if (ACC) {
      constexpr int W = TPR < 64 ? TPR : 64;
#pragma unroll
      for (int off = W / 2; off > 0; off >>= 1) {
        argmax_combine(best_z, arg_z, __shfl_xor(best_z, off), __shfl_xor(arg_z, off));
        argmax_combine(best_t, arg_t, __shfl_xor(best_t, off), __shfl_xor(arg_t, off));
      }
      __shared__ unsigned group_count;
      if (threadIdx.x == 0) group_count = 0;
      __syncthreads();
      const unsigned long long agreeing = __ballot(sub == 0 && row_ok && arg_z == arg_t);
      if ((threadIdx.x & 63) == 0 && agreeing != 0ull) atomicAdd(&group_count, (unsigned)__popcll(agreeing));
      __syncthreads();
      if (threadIdx.x == 0) mirror.group_hits[blockIdx.x] = group_count;
    }
  } else {
    if (saw_nan) atomicOr(&flags[2], 1);
  }
}

template <int VEC>
__device__ __forceinline__ void load_vec(const double* p, double (&v)[VEC]) {
  if (VEC == 2) {
    const v2d t = *reinterpret_cast<const v2d*>(p);
    v[0] = t.x;
    v[VEC - 1] = t.y;
  } else {
    v[0] = *p;
  }
}
template <int VEC>
__device__ __forceinline__ void load_vec_nt(const double* p, double (&v)[VEC]) {
  if (VEC == 2) {
    const v2d t = __builtin_nontemporal_load(reinterpret_cast<const v2d*>(p));
    v[0] = t.x;
    v[VEC - 1] = t.y;
  } else {
    v[0] = __builtin_nontemporal_load(p);
  }
}
template <int VEC>
__device__ __forceinline__ void store_vec_nt(double* p, const double (&v)[VEC]) {
  if (VEC == 2) {
    const v2d t = {v[0], v[VEC - 1]};
    __builtin_nontemporal_store(t, reinterpret_cast<v2d*>(p));
  } else {
    __builtin_nontemporal_store(v[0], p);
  }
}

// Rows wider than 2048 logits: one workgroup of BLOCK threads per row, several workgroups per
// compute unit (128 registers per thread), so that the arithmetic of one row overlaps the memory
// traffic of another.  First walk: every thread folds its share of the row into a running
// maximum m and the sum s of exp(z - m), rescaling s when m grows; the workgroup then agrees on
// the row maximum M and the row sum S = sum of s * exp(m - M).  Second walk, backwards: p =
// exp(z - M) / S with the same operations as the register kernel, then the loss term and the
// gradient.  S differs from a left-to-right sum only by rounding (relative 1e-16).  The first
// PARK chunks of the row (PARK * 4 * BLOCK vectors, 32 KiB with 256 threads, 64 KiB with 512)
// wait in LDS between the walks instead of being read again.
template <int BLOCK, int VEC, bool CE>
__global__ __launch_bounds__(BLOCK) __attribute__((amdgpu_waves_per_eu(4, 4))) void softmax_wide_rows_kernel(
    const double* __restrict__ z, const double* __restrict__ truth, double* __restrict__ grad,
    double* __restrict__ prob, double* __restrict__ row_loss, int* __restrict__ flags, size_t cols) {
  constexpr int UNR = 4;
  constexpr int PARK = 2;
  constexpr size_t CHUNK = (size_t)UNR * BLOCK;
  __shared__ double red[3][BLOCK / 64];
  __shared__ __attribute__((aligned(16))) double park[PARK * UNR * BLOCK * VEC];
  const size_t row = blockIdx.x;
  const size_t base = row * cols;
  const double* zr = z + base;
  const size_t units = cols / VEC;
  const size_t nchunk = units / CHUNK;
  const size_t full = nchunk * CHUNK;

  bool saw_nan = false;
  double m = -DBL_MAX, s = 0.0;
  for (size_t c = 0; c < nchunk; ++c) {
    double v[UNR][VEC];
    const double* src = zr + (c * CHUNK + threadIdx.x) * VEC;
    if (c < PARK) {
#pragma unroll
      for (int i = 0; i < UNR; ++i) load_vec_nt<VEC>(src + (size_t)i * BLOCK * VEC, v[i]);
#pragma unroll
      for (int i = 0; i < UNR; ++i) {
        double* slot = park + ((c * UNR + i) * BLOCK + threadIdx.x) * VEC;
#pragma unroll
        for (int e = 0; e < VEC; ++e) slot[e] = v[i][e];
      }
    } else {
#pragma unroll
      for (int i = 0; i < UNR; ++i) load_vec<VEC>(src + (size_t)i * BLOCK * VEC, v[i]);
    }
    double cm = m;
#pragma unroll
    for (int i = 0; i < UNR; ++i) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        saw_nan |= (v[i][e] != v[i][e]);
        cm = MaxOp::apply(cm, v[i][e]);
      }
    }
    if (cm > m) {
      s *= exp(m - cm);
      m = cm;
    }
#pragma unroll
    for (int i = 0; i < UNR; ++i) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) s += exp(v[i][e] - m);
    }
  }
  for (size_t u = full + threadIdx.x; u < units; u += BLOCK) {
    double v[VEC];
    load_vec<VEC>(zr + u * VEC, v);
    double cm = m;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      saw_nan |= (v[e] != v[e]);
      cm = MaxOp::apply(cm, v[e]);
    }
    if (cm > m) {
      s *= exp(m - cm);
      m = cm;
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) s += exp(v[e] - m);
  }
  const double M = group_reduce<BLOCK, MaxOp>(m, red[0]);
  s *= exp(m - M);
  const double S = group_reduce<BLOCK, SumOp>(s, red[1]);

  double lsum = 0.0;
  auto finish = [&](size_t u, const double (&v)[VEC], const double (&t)[VEC]) {
    double p[VEC], g[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      p[e] = exp(v[e] - M) / S;
      if (CE) {
        lsum += loss_term(t[e], p[e]);
        g[e] = -(t[e] - p[e]);
      }
    }
    if (CE) store_vec_nt<VEC>(grad + base + u * VEC, g);
    if (prob) store_vec_nt<VEC>(prob + base + u * VEC, p);
  };
  for (size_t u = full + threadIdx.x; u < units; u += BLOCK) {
    double v[VEC], t[VEC] = {};
    load_vec<VEC>(zr + u * VEC, v);
    if (CE) load_vec_nt<VEC>(truth + base + u * VEC, t);
    finish(u, v, t);
  }
  for (size_t c = nchunk; c > 0; --c) {
    const size_t cc = c - 1;
    const size_t ub = cc * CHUNK + threadIdx.x;
    double v[UNR][VEC], t[UNR][VEC] = {};
    if (cc < PARK) {
#pragma unroll
      for (int i = UNR - 1; i >= 0; --i) {
        const double* slot = park + ((cc * UNR + i) * BLOCK + threadIdx.x) * VEC;
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[i][e] = slot[e];
      }
    } else {
#pragma unroll
      for (int i = UNR - 1; i >= 0; --i) load_vec<VEC>(zr + (ub + (size_t)i * BLOCK) * VEC, v[i]);
    }
    if (CE) {
#pragma unroll
      for (int i = UNR - 1; i >= 0; --i) load_vec_nt<VEC>(truth + base + (ub + (size_t)i * BLOCK) * VEC, t[i]);
    }
#pragma unroll
    for (int i = UNR - 1; i >= 0; --i) finish(ub + (size_t)i * BLOCK, v[i], t[i]);
  }
  if (CE) {
    lsum = group_reduce<BLOCK, SumOp>(lsum, red[2]);
    if (threadIdx.x == 0) row_loss[row] = lsum;
    if (saw_nan) atomicOr(&flags[0], 1);
  } else {
    if (saw_nan) atomicOr(&flags[2], 1);
  }
}

// Second (tiny) launch of a cross entropy: loss = -(sum of the per-row sums) / rows in a fixed
// order, one workgroup.  It also latches the NaN flag of the launch into flags[1] and re-arms
// flags[0], so no reset launch is needed.  hit_groups > 0: the row kernel left the arg-max agreements of
// its workgroups in mirror.group_hits[0 .. hit_groups); their sum goes out with the loss.
__global__ __launch_bounds__(1024) void loss_reduce_kernel(const double* __restrict__ row_loss,
                                                          double* __restrict__ loss,
                                                          int* __restrict__ flags, size_t rows,
                                                          LossMirror mirror, unsigned hit_groups) {
  __shared__ double red[1024 / 64];
  __shared__ unsigned hit_total;
  if (hit_groups > 0) {
    if (threadIdx.x == 0) hit_total = 0;
    __syncthreads();
    unsigned mine = 0;
    for (unsigned g = threadIdx.x; g < hit_groups; g += 1024) mine += mirror.group_hits[g];
    if (mine != 0) atomicAdd(&hit_total, mine);  // (an integer count: any order)
  }
  // thread t adds rows t, t + 1024, ... in that order; eight of its loads are in flight at a time (the
  // row sums were written by other XCDs: every load is a trip to memory)
  double s = 0.0;
  size_t r = threadIdx.x;
  for (; r + 7 * 1024 < rows; r += 8 * 1024) {
    double t[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) t[j] = row_loss[r + (size_t)j * 1024];
#pragma unroll
    for (int j = 0; j < 8; ++j) s += t[j];
  }
  for (; r < rows; r += 1024) s += row_loss[r];
  s = group_reduce<1024, SumOp>(s, red);
  if (threadIdx.x == 0) {
    const double l = -s / (double)rows;
    const int nan_seen = flags[0];
    loss[0] = l;
    flags[1] = nan_seen;
    flags[0] = 0;
    // (group_reduce above ends in a barrier of the whole workgroup: every addition to hit_total is in)
    publish(mirror, l, nan_seen, hit_groups > 0, hit_groups > 0 ? (unsigned long long)hit_total : 0ull);
  }
}

// The classifier head of a training step in one launch: the last Linear's forward
// (src/module/linear.rs:44-58), the cross entropy on its logits with the gradient
// (src/loss/cross_entropy.rs:34-47), that Linear's input gradient (linear.rs:68) with the mask of a
// preceding ReLU (src/module/activation/relu.rs:25-28), and the loss itself, finished by the
// workgroup that arrives last.  For heads of at most kHeadCols classes on a few hundred inputs,
// where the four launches this replaces are each over before the next one has started.
//
// A workgroup of BLOCK threads takes BLOCK / 16 rows at a time, 16 lanes to a row.  Lane j of a row
// keeps inputs j, j + 16, ... of that row in registers (KI of them at most) and the whole weight
// matrix sits in LDS.  Logits: the lane adds up its share of every class's dot product in ascending
// k, an exchange over the 16 lanes completes the sums, and lane c goes on with class c through the
// softmax with the arithmetic of softmax_rows_kernel.  Input gradient: the lanes of a row exchange
// their gradient entries, and lane j computes elements j, j + 16, ... as sums over the classes in
// ascending order, masked by the inputs it still holds.
// The loss: each workgroup adds its rows' terms up in row order, and the workgroup that arrives last
// adds the workgroups' sums up in a fixed order (thread t sums t, t + BLOCK, ...; a butterfly over each
// wavefront; the wavefronts in turn), so the result does not depend on which one came last.
//
// HID: the Linear in front of the head (at most 112 inputs and outputs) runs in the same launch, so
// that two more launches - its forward and its input gradient - disappear.  Its weights sit in LDS
// as well; a workgroup (512 threads) takes 16 rows at a time - one MFMA fragment - and walks over
// the batch with a stride of the grid (the weights are fetched once per workgroup): hidden forward
// on the matrix cores (wavefront w computes output fragment w), the head as above on the result (the
// first four wavefronts), hidden input gradient on the matrix cores.
struct HeadParams {
  const double* h;      // [rows, K] inputs of the Linear (contiguous rows)
  const double* w;      // [N, K]
  const double* bias;   // [N]
  const double* truth;  // [rows, N]
  double* logits;       // [rows, N]
  double* grad;         // [rows, N]  -(truth - p)
  double* dx;           // [rows, K] or NULL
  double* partial;      // one sum per workgroup
  unsigned long long* arrivals;  // zero between launches
  double* loss;
  int* flags;
  size_t rows;
  int N, K;
  LossMirror mirror;
  // HID
  const double* h1;     // [rows, K1] inputs of the hidden Linear
  const double* w2;     // [K, K1] its weights
  const double* b2;     // [K]
  double* h_out;        // [rows, K] its outputs (what `h` is otherwise)
  double* dx1;          // [rows, K1] the gradient with respect to h1, or NULL
  int K1;
  int mask1;            // dx1 is zeroed where h1 <= 0
};

typedef double v4d_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void lds_barrier() {
  // A workgroup barrier for data exchanged through LDS: this wavefront's LDS accesses are over, then
  // everybody meets.  Unlike __syncthreads() it does not wait for the stores to global memory that
  // are still on their way (nobody in the workgroup reads those back), which take a microsecond or two.
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
__device__ __forceinline__ double lds_read_f64(uint32_t byte_address) {
  double v;
  asm volatile("ds_read_b64 %0, %1" : "=v"(v) : "v"(byte_address) : "memory");
  return v;
}
// One 16 x 16 MFMA product chain out of LDS: c += sum over steps s of A[.][4 s + lk] x B[4 s + lk][.],
// a (resp. b) pointing at this lane's element of step 0 and moving by a_step (b_step) doubles per
// step; `steps` is a multiple of four.  The reads are inline assembly, so that their place in the
// instruction stream is fixed and the waits can name how many younger reads may still be
// outstanding: the operands of four steps are in registers or on their way at any time, in two sets
// of two steps, and a set's four reads go out as soon as the MFMAs that used its registers have been
// issued.  Each of the four steps of a round adds up in an accumulator of its own (an MFMA that
// continues the sum of the one issued just before it would wait for its result); they are added
// together at the end.  After the last step the requests fetch the last operands again; nobody uses them.
__device__ __forceinline__ v4d_t mfma_chain(const double* a, int a_step, const double* b, int b_step, int steps) {
  uint32_t pa = (uint32_t)(uintptr_t)a, pb = (uint32_t)(uintptr_t)b;
  const uint32_t da = 8u * (uint32_t)a_step, db = 8u * (uint32_t)b_step;
  double xa0 = lds_read_f64(pa), xb0 = lds_read_f64(pb);
  double xa1 = lds_read_f64(pa + da), xb1 = lds_read_f64(pb + db);
  double ya0 = lds_read_f64(pa + 2 * da), yb0 = lds_read_f64(pb + 2 * db);
  double ya1 = lds_read_f64(pa + 3 * da), yb1 = lds_read_f64(pb + 3 * db);
  v4d_t c0 = {0.0, 0.0, 0.0, 0.0}, c1 = c0, c2 = c0, c3 = c0;
  for (int s = 0; s < steps; s += 4) {
    const bool more = s + 4 < steps;
    pa += more ? 4 * da : 0;
    pb += more ? 4 * db : 0;
    asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(xa0), "+v"(xb0), "+v"(xa1), "+v"(xb1));
    c0 = __builtin_amdgcn_mfma_f64_16x16x4f64(xa0, xb0, c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f64_16x16x4f64(xa1, xb1, c1, 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    xa0 = lds_read_f64(pa);
    xb0 = lds_read_f64(pb);
    xa1 = lds_read_f64(pa + da);
    xb1 = lds_read_f64(pb + db);
    asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(ya0), "+v"(yb0), "+v"(ya1), "+v"(yb1));
    c2 = __builtin_amdgcn_mfma_f64_16x16x4f64(ya0, yb0, c2, 0, 0, 0);
    c3 = __builtin_amdgcn_mfma_f64_16x16x4f64(ya1, yb1, c3, 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    ya0 = lds_read_f64(pa + 2 * da);
    yb0 = lds_read_f64(pb + 2 * db);
    ya1 = lds_read_f64(pa + 3 * da);
    yb1 = lds_read_f64(pb + 3 * db);
  }
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(xa0), "+v"(xb0), "+v"(xa1), "+v"(xb1), "+v"(ya0), "+v"(yb0), "+v"(ya1), "+v"(yb1));
  return (c0 + c1) + (c2 + c3);
}

// (two wavefronts per SIMD as the floor of the register budget: with the whole register file to itself
// the compiler would park the MFMA accumulators in the accumulation registers and copy them back and
// forth around every instruction of the chain)
template <int KI, int NC, bool MASK, int BLOCK, bool HID = false>
__global__ __launch_bounds__(BLOCK, 2) void head_ce_kernel(HeadParams p) {
  // rows per workgroup and pass (HID: one 16-row MFMA fragment; the wavefronts beyond the first four
  // only take part in the matrix-core phases and in the copies)
  constexpr int ROWS = HID ? 16 : BLOCK / 16;
  constexpr int NW = BLOCK / 64;
  static_assert(NC == 4 || NC == 8 || NC == 16, "the class sums are exchanged by halving");
  static_assert(!HID || (BLOCK == 512 && KI == 8), "the hidden layer: eight wavefronts, one output fragment each");
  // the weights, transposed: [16 * KI][P], the NC classes of one input side by side, zero from class N
  // and from input K on; with P = NC + 2 the 16 lanes of a row, which read 16 consecutive inputs, hit
  // different banks
  extern __shared__ __attribute__((aligned(16))) double head_ws[];
  constexpr int P = NC + 2;
  // HID: behind them the hidden layer's weights [n][k] (rows of P1 doubles, zero past its extents), the
  // 16 input rows [m][k] (P1) and a [16][PH] panel that first holds the hidden layer's output and
  // then the gradient with respect to it
  constexpr int PH = 16 * KI + 2;
  const int K = p.K, N = p.N, K1 = HID ? p.K1 : 0;
  const int KP1 = (K1 + 15) / 16 * 16, P1 = KP1 + 2;  // (MFMA steps in fours)
  const int NF2 = HID ? (K + 15) / 16 : 0, NF1 = (K1 + 15) / 16;
  double* const w2s = head_ws + 16 * KI * P;
  double* const h1s = w2s + (size_t)NF2 * 16 * P1 + 16;
  double* const hg = h1s + 16 * P1;
  __shared__ double wave_sum[BLOCK / 64];
  __shared__ double row_sum[ROWS];
  __shared__ int nan_here, last_nan;
  __shared__ bool is_last;
  const int t = threadIdx.x;
  if (t == 0) nan_here = 0;
  const int r = t >> 4, j = t & 15;
  const bool head_thread = r < ROWS;
  const int lane = t & 63, wave = t >> 6, lr = lane & 15, lk = lane >> 4;
  const size_t passes_all = (p.rows + ROWS - 1) / ROWS;

  // the weights: every global load of a batch is issued before the first one is waited for
  for (int k = t; k < 16 * KI; k += BLOCK) {  // (at most two rounds)
    double v[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) v[c] = (c < N && k < K) ? p.w[(size_t)c * K + k] : 0.0;
#pragma unroll
    for (int c = 0; c < NC; c += 2) *reinterpret_cast<v2d*>(head_ws + k * P + c) = v2d{v[c], v[c + 1]};
  }
  if (HID) {
    // a wavefront takes every eighth row of the padded matrix, a lane one pair of columns
    constexpr int U = 14;
    const int kp = 2 * lane;
    for (int n0 = wave; n0 < NF2 * 16; n0 += NW * U) {
      double v[U][2];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int n = n0 + NW * u;
        const bool row_in = n < K;
        v[u][0] = (row_in && kp < K1) ? p.w2[(size_t)n * K1 + kp] : 0.0;
        v[u][1] = (row_in && kp + 1 < K1) ? p.w2[(size_t)n * K1 + kp + 1] : 0.0;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int n = n0 + NW * u;
        if (n < NF2 * 16 && kp < P1) *reinterpret_cast<v2d*>(w2s + n * P1 + kp) = v2d{v[u][0], v[u][1]};
      }
    }
  }

  // HID: the 16 input rows of a pass travel through registers
  constexpr int RU = 16 / NW > 0 ? 16 / NW : 1;
  double h1v[RU][2];
  auto fetch_inputs = [&](size_t pass) {
    const size_t first = pass * ROWS;
    const int kp = 2 * lane;
#pragma unroll
    for (int u = 0; u < RU; ++u) {
      const int m = wave + NW * u;
      const bool in = m < 16 && first + m < p.rows;
      h1v[u][0] = (in && kp < K1) ? p.h1[(first + m) * (size_t)K1 + kp] : 0.0;
      h1v[u][1] = (in && kp + 1 < K1) ? p.h1[(first + m) * (size_t)K1 + kp + 1] : 0.0;
    }
  };
  if (HID) fetch_inputs(blockIdx.x);

  double mine = 0.0;  // (thread 0) the workgroup's loss terms so far
  unsigned long long old = 0;
  unsigned long long* const partial = reinterpret_cast<unsigned long long*>(p.partial);
  for (size_t pass = blockIdx.x; pass < passes_all; pass += gridDim.x) {
    const bool last_pass = pass + gridDim.x >= passes_all;
    const size_t row0 = pass * ROWS;
    const size_t row = row0 + r;
    const bool row_ok = row < p.rows;
    double hv[KI];
    if (!HID) {
      const double* hr = p.h + row * (size_t)K;
#pragma unroll
      for (int i = 0; i < KI; ++i) {
        const int k = j + 16 * i;
        hv[i] = (row_ok && k < K) ? hr[k] : 0.0;
      }
    } else {
      // (the previous pass is done with the input rows and the panel)
      if (pass != blockIdx.x) lds_barrier();
      // the 16 input rows, requested during the previous pass: a wavefront takes every eighth row, a
      // lane a pair of columns
#pragma unroll
      for (int u = 0; u < RU; ++u)
        if (wave + NW * u < 16 && 2 * lane < P1)
          *reinterpret_cast<v2d*>(h1s + (wave + NW * u) * P1 + 2 * lane) = v2d{h1v[u][0], h1v[u][1]};
      fetch_inputs(pass + gridDim.x);  // (for the next pass; beyond the batch: zeros, unused)
    }
    const double bias = (head_thread && j < N) ? p.bias[j] : 0.0;
    const double tv = (head_thread && row_ok && j < N) ? p.truth[row * N + j] : 0.0;
    const double b2v = (HID && wave * 16 + lr < K) ? p.b2[wave * 16 + lr] : 0.0;
    lds_barrier();

    if (HID) {
      // The hidden Linear (src/module/linear.rs:44-58) on the 16 rows: wavefront w computes the 16-column
      // fragment w of the output with FP64 MFMAs, four contraction indices a step, both
      // operands from LDS; bias and ReLU as in the contraction kernels' epilogue; the result goes to
      // memory (the head's weight gradient reads it) and into the panel for the head below.
      if (wave < NF2) {
        const v4d_t c = mfma_chain(h1s + lr * P1 + lk, 4, w2s + (wave * 16 + lr) * P1 + lk, 4, KP1 / 4);
        const int col = wave * 16 + lr;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int m = 4 * q + lk;
          double v = c[q] + b2v;
          if (MASK) v = fmax(v, 0.0);
          if (col >= K) v = 0.0;
          hg[m * PH + col] = v;
          if (row0 + m < p.rows && col < K) p.h_out[(row0 + m) * (size_t)K + col] = v;
        }
      }
      lds_barrier();
#pragma unroll
      for (int i = 0; i < KI; ++i) {
        const int k = j + 16 * i;
        hv[i] = (head_thread && k < NF2 * 16) ? hg[r * PH + k] : 0.0;
      }
    }

    // logits.  No branch in the loop (a branch would have every LDS read waited for on its own): inputs
    // and weights past the row's end are zero; the weights of the next input are on their way while
    // those of this one are used.
    const v2d* const wj = reinterpret_cast<const v2d*>(head_ws + j * P);  // input j + 16 i: wj + i * 8 P
    double g = 0.0;  // this lane's entry of the loss gradient
    if (head_thread) {
    double acc[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[c] = 0.0;
    {
      v2d w2[2][NC / 2];
#pragma unroll
      for (int c = 0; c < NC / 2; ++c) w2[0][c] = wj[c];
#pragma unroll
      for (int i = 0; i < KI; ++i) {
        if (i + 1 < KI) {
#pragma unroll
          for (int c = 0; c < NC / 2; ++c) w2[(i + 1) & 1][c] = wj[(i + 1) * 8 * P + c];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < NC / 2; ++c) {
          acc[2 * c] = fma(hv[i], w2[i & 1][c].x, acc[2 * c]);
          acc[2 * c + 1] = fma(hv[i], w2[i & 1][c].y, acc[2 * c + 1]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // The 16 lanes of a row add their shares up by halving: with offset 8, 4, 2, 1 in turn a lane keeps
    // the classes whose index has the lane's bit at that position and receives its partner's share of
    // them, so that lane j ends with the whole sum of class j (lanes from NC on: a class below NC again).
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) {
      if (off < NC) {
        const bool upper = (j & off) != 0;
#pragma unroll
        for (int i = 0; i < off; ++i) {
          const double lo = acc[i], hi = acc[i + off < NC ? i + off : i];
          const double got = __shfl_xor(upper ? lo : hi, off);
          acc[i] = (upper ? hi : lo) + got;
        }
      } else {  // fewer classes than 2 * off: every lane keeps all of them
#pragma unroll
        for (int c = 0; c < NC; ++c) acc[c] = acc[c] + __shfl_xor(acc[c], off);
      }
    }
    double z = acc[0];
    const bool col_ok = j < N, ok = row_ok && col_ok;
    z = z + bias;
    const bool saw_nan = ok && z != z;
    double mx = col_ok ? MaxOp::apply(-DBL_MAX, z) : -DBL_MAX;
    mx = group_reduce<kHeadCols, MaxOp>(mx, nullptr);
    const double ev = col_ok ? exp(z - mx) : 0.0;
    const double s = group_reduce<kHeadCols, SumOp>(ev, nullptr);
    double lsum = 0.0;
    if (ok) {
      const double pr = ev / s;
      lsum = loss_term(tv, pr);
      g = -(tv - pr);
      p.grad[row * N + j] = g;
      p.logits[row * N + j] = z;
    }
    lsum = group_reduce<kHeadCols, SumOp>(lsum, nullptr);
    if (j == 0) row_sum[r] = row_ok ? lsum : 0.0;
    if (saw_nan) nan_here = 1;  // (every writer writes the same value)
    }
    lds_barrier();

    // The loss.  Thread 0 hands this workgroup's sum over with an atomic exchange, which is carried out
    // where every workgroup of the device sees it, and only then - the exchange's return value is an
    // operand of the addition - counts the workgroup in at `arrivals` (low word: workgroups, high word:
    // those that met a NaN logit).  Whoever counts in last therefore finds every other sum in place and
    // reads them with atomic loads.  No fence is involved: a device-wide release would have every
    // workgroup write the whole L2 back.  The exchange travels while the input gradients are computed.
    if (t == 0) {
#pragma unroll
      for (int i = 0; i < ROWS; ++i) mine += row_sum[i];
      if (last_pass) old = atomicExch(partial + blockIdx.x, (unsigned long long)__double_as_longlong(mine));
    }

    if (p.dx && head_thread) {
      double gc[NC];
#pragma unroll
      for (int c = 0; c < NC; ++c) gc[c] = __shfl(g, c, 16);  // (zero from class N on)
      double* const dr = p.dx + row * (size_t)K;
      v2d w2[2][NC / 2];
#pragma unroll
      for (int c = 0; c < NC / 2; ++c) w2[0][c] = wj[c];
#pragma unroll
      for (int i = 0; i < KI; ++i) {
        const int k = j + 16 * i;
        if (i + 1 < KI) {
#pragma unroll
          for (int c = 0; c < NC / 2; ++c) w2[(i + 1) & 1][c] = wj[(i + 1) * 8 * P + c];
        }
        __builtin_amdgcn_sched_barrier(0);
        double a = 0.0;
#pragma unroll
        for (int c = 0; c < NC / 2; ++c) {
          a = fma(gc[2 * c], w2[i & 1][c].x, a);
          a = fma(gc[2 * c + 1], w2[i & 1][c].y, a);
        }
        if (MASK) a = a * (hv[i] > 0.0 ? 1.0 : 0.0);
        if (row_ok && k < K) dr[k] = a;
        if (HID) hg[r * PH + k] = k < K ? a : 0.0;  // (every lane took its inputs from the panel before the last barrier)
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (HID && p.dx1) {
      // The hidden Linear's input gradient (linear.rs:68): [16, K] x [K, K1] from the panel and the
      // weights in LDS, fragment by fragment as above, zeroed where the ReLU in front of it was off.
      lds_barrier();
      if (wave < NF1) {
        const v4d_t c = mfma_chain(hg + lr * PH + lk, 4, w2s + lk * P1 + wave * 16 + lr, 4 * P1, NF2 * 4);
        const int col = wave * 16 + lr;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int m = 4 * q + lk;
          double v = c[q];
          if (p.mask1) v = v * ((col < K1 ? h1s[m * P1 + col] : 0.0) > 0.0 ? 1.0 : 0.0);
          if (row0 + m < p.rows && col < K1) p.dx1[(row0 + m) * (size_t)K1 + col] = v;
        }
      }
    }
  }

  if (t == 0) {
    // the addition below is issued only when the exchange has returned: its result is an input of this
    // (empty) statement, which no memory access may cross
    asm volatile("" : "+v"(old) : : "memory");
    const unsigned long long inc = 1ull + ((unsigned long long)nan_here << 32) + (old & 0ull);
    const unsigned long long seen = atomicAdd(p.arrivals, inc) + inc;
    last_nan = (int)((seen >> 32) != 0);
    is_last = (unsigned)seen == gridDim.x;
  }
  __syncthreads();
  if (!is_last) return;
  double sum = 0.0;
  for (unsigned base = t; base < gridDim.x; base += BLOCK * 4) {  // four loads in flight
    unsigned long long v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const unsigned at = base + BLOCK * i < gridDim.x ? base + BLOCK * i : 0;
      v[i] = __hip_atomic_load(partial + at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (base + BLOCK * i < gridDim.x) sum += __longlong_as_double((long long)v[i]);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum = sum + __shfl_xor(sum, off);
  if ((t & 63) == 0) wave_sum[t >> 6] = sum;
  __syncthreads();
  if (t == 0) {
    double total = wave_sum[0];
#pragma unroll
    for (int w = 1; w < BLOCK / 64; ++w) total += wave_sum[w];
    const double l = -total / (double)p.rows;
    p.loss[0] = l;
    p.flags[1] = last_nan;
    __hip_atomic_store(p.arrivals, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // re-armed for the next launch
    publish(p.mirror, l, last_nan, false, 0);
  }
}

// softmax down the columns (Softmax::with_axis(0), src/module/activation/softmax.rs:23-28):
// one thread per column walks the rows three times; a rarely used orientation, kept simple.
__global__ __launch_bounds__(256) void softmax_columns_kernel(const double* __restrict__ z,
                                                             double* __restrict__ out,
                                                             int* __restrict__ flags, size_t rows,
                                                             size_t cols) {
  const size_t c = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (c >= cols) return;
  double mx = -DBL_MAX;
  bool saw_nan = false;
  for (size_t r = 0; r < rows; ++r) {
    const double v = z[r * cols + c];
    saw_nan |= (v != v);
    mx = MaxOp::apply(mx, v);
  }
  double s = 0.0;
  for (size_t r = 0; r < rows; ++r) {
    const double e = exp(z[r * cols + c] - mx);
    out[r * cols + c] = e;
    s += e;
  }
  for (size_t r = 0; r < rows; ++r) out[r * cols + c] = out[r * cols + c] / s;
  if (saw_nan) atomicOr(&flags[2], 1);
}

// jacobian fix-up of the Softmax module's backward (softmax.rs:64-69): off-diagonal entries of
// out^T.out are negated, a diagonal entry d becomes d * (1 - d).
__global__ __launch_bounds__(256) void softmax_jacobian_kernel(double* __restrict__ jac, size_t cols) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= cols * cols) return;
  const size_t r = i / cols, c = i - r * cols;
  const double v = jac[i];
  jac[i] = (r == c) ? v * (1.0 - v) : -v;
}

template <int TPR, int IPT, int VEC>
int launch_rows(hipStream_t s, const double* z, const double* t, double* grad, double* prob,
                double* row_loss, double* loss, int* flags, size_t rows, size_t cols, bool ce,
                LossMirror mirror, bool* loss_done, bool* hits_done, unsigned* hit_groups) {
  constexpr int BLOCK = 256;
  constexpr int RPB = BLOCK / TPR;
  size_t blocks = (rows + RPB - 1) / RPB;
  if (blocks > 0x7fffffffull) return fail(RST_ERR_UNSUPPORTED, "too many rows for one launch");
  // (rows that span several wavefronts reduce through per-row scratch that exists once per workgroup)
  if constexpr (TPR <= 64) {
    if (ce && rows * TPR <= 1024) {
      if (mirror.hits) {
        hipLaunchKernelGGL((softmax_rows_kernel<TPR, IPT, VEC, true, 1024, true, true>), dim3(1), dim3(1024), 0, s,
                           z, t, grad, prob, row_loss, loss, flags, rows, cols, mirror);
        *hits_done = true;
      } else {
        hipLaunchKernelGGL((softmax_rows_kernel<TPR, IPT, VEC, true, 1024, true>), dim3(1), dim3(1024), 0, s,
                           z, t, grad, prob, row_loss, loss, flags, rows, cols, mirror);
      }
      *loss_done = true;
      RST_HIP(hipGetLastError());
      return RST_OK;
    }
  }
  if constexpr (TPR <= 64) {
    if (ce && mirror.hits && mirror.group_hits) {  // counted per workgroup; the reduction launch publishes the sum with the loss
      hipLaunchKernelGGL((softmax_rows_kernel<TPR, IPT, VEC, true, BLOCK, false, true>), dim3((unsigned)blocks),
                         dim3(BLOCK), 0, s, z, t, grad, prob, row_loss, loss, flags, rows, cols, mirror);
      *hits_done = true;
      *hit_groups = (unsigned)blocks;
      RST_HIP(hipGetLastError());
      return RST_OK;
    }
  }
  if (ce)
    hipLaunchKernelGGL((softmax_rows_kernel<TPR, IPT, VEC, true>), dim3((unsigned)blocks),
                       dim3(BLOCK), 0, s, z, t, grad, prob, row_loss, loss, flags, rows, cols, mirror);
  else
    hipLaunchKernelGGL((softmax_rows_kernel<TPR, IPT, VEC, false>), dim3((unsigned)blocks),
                       dim3(BLOCK), 0, s, z, t, grad, prob, row_loss, loss, flags, rows, cols, mirror);
  RST_HIP(hipGetLastError());
  return RST_OK;
}

template <int BLOCK, int VEC>
int launch_wide(hipStream_t s, const double* z, const double* t, double* grad, double* prob,
                double* row_loss, int* flags, size_t rows, size_t cols, bool ce) {
  if (rows > 0x7fffffffull) return fail(RST_ERR_UNSUPPORTED, "too many rows for one launch");
  if (ce)
    hipLaunchKernelGGL((softmax_wide_rows_kernel<BLOCK, VEC, true>), dim3((unsigned)rows), dim3(BLOCK), 0,
                       s, z, t, grad, prob, row_loss, flags, cols);
  else
    hipLaunchKernelGGL((softmax_wide_rows_kernel<BLOCK, VEC, false>), dim3((unsigned)rows), dim3(BLOCK), 0,
                       s, z, t, grad, prob, row_loss, flags, cols);
  RST_HIP(hipGetLastError());
  return RST_OK;
}

template <int VEC>
int dispatch(hipStream_t s, const double* z, const double* t, double* grad, double* prob,
             double* row_loss, double* loss, int* flags, size_t rows, size_t cols, bool ce,
             LossMirror mirror, bool* loss_done, bool* hits_done, unsigned* hit_groups) {
  const size_t units = cols / VEC;  // vectors per row
  if (units <= 16 * 2) return launch_rows<16, 2, VEC>(s, z, t, grad, prob, row_loss, loss, flags, rows, cols, ce, mirror, loss_done, hits_done, hit_groups);
  if (units <= 64 * 4) return launch_rows<64, 4, VEC>(s, z, t, grad, prob, row_loss, loss, flags, rows, cols, ce, mirror, loss_done, hits_done, hit_groups);
  if (units <= 256 * 4) return launch_rows<256, 4, VEC>(s, z, t, grad, prob, row_loss, loss, flags, rows, cols, ce, mirror, loss_done, hits_done, hit_groups);
  // measured on 32 Mi logits: 256 threads per row are ahead below about 12 Ki columns, 512 above
  if (cols < 12288) return launch_wide<256, VEC>(s, z, t, grad, prob, row_loss, flags, rows, cols, ce);
  return launch_wide<512, VEC>(s, z, t, grad, prob, row_loss, flags, rows, cols, ce);
}

inline bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

// The row kernel of a softmax or cross entropy; *loss_done tells whether it finished the loss too.
int launch_row_kernel(hipStream_t s, const double* z, const double* t, double* grad_out, double* prob_out,
                      double* row_loss, double* loss, int* flags, size_t rows, size_t cols,
                      LossMirror mirror, bool* loss_done, bool* hits_done, unsigned* hit_groups) {
  const bool ce = grad_out != nullptr;
  const bool vec = cols % 2 == 0 && aligned16(z) && (!ce || (aligned16(t) && aligned16(grad_out))) &&
                   (!prob_out || aligned16(prob_out));
  *loss_done = false;
  if (vec) return dispatch<2>(s, z, t, grad_out, prob_out, row_loss, loss, flags, rows, cols, ce, mirror, loss_done, hits_done, hit_groups);
  return dispatch<1>(s, z, t, grad_out, prob_out, row_loss, loss, flags, rows, cols, ce, mirror, loss_done, hits_done, hit_groups);
}

}  // namespace

int launch_softmax_ce(hipStream_t s, const double* z, const double* t, double* grad_out,
                      double* prob_out, double* row_loss, double* loss, int* flags, size_t rows,
                      size_t cols, LossMirror mirror, bool* hits_done) {
  bool no_hits = false;
  if (!hits_done) {
    hits_done = &no_hits;
    mirror.hits = nullptr;
  }
  *hits_done = false;
  if (rows == 0 || cols == 0) return RST_OK;
  const bool ce = grad_out != nullptr;
  bool loss_done = false;
  unsigned hit_groups = 0;  // workgroups of the row kernel that left a hit count for the reduction launch
  RST_TRY(launch_row_kernel(s, z, t, grad_out, prob_out, row_loss, loss, flags, rows, cols, mirror, &loss_done, hits_done, &hit_groups));
  if (ce && !loss_done) {
    hipLaunchKernelGGL(loss_reduce_kernel, dim3(1), dim3(1024), 0, s, row_loss, loss, flags, rows, mirror, hit_groups);
    RST_HIP(hipGetLastError());
  }
  return RST_OK;
}

bool head_ce_supported(size_t cols, size_t in_features) {
  return cols >= 1 && cols <= (size_t)kHeadCols && in_features >= 1 && in_features <= 16 * 18;
}

namespace {
// LDS of the variant that also runs the hidden Linear: the head's weights, the hidden weights padded
// to whole fragments, 16 input rows and the [16][130] panel
size_t tail_lds_bytes(size_t cols, size_t hidden, size_t in_features) {
  const size_t nc = cols <= 4 ? 4 : cols <= 8 ? 8 : 16;
  const size_t p1 = (in_features + 15) / 16 * 16 + 2, nf2 = (hidden + 15) / 16;
  return (16 * 8 * (nc + 2) + nf2 * 16 * p1 + 16 + 16 * p1 + 16 * (16 * 8 + 2)) * sizeof(double);
}
}  // namespace

bool tail_ce_supported(size_t cols, size_t hidden, size_t in_features, size_t lds_limit) {
  return head_ce_supported(cols, hidden) && hidden <= 112 && in_features >= 1 && in_features <= 112 &&
         tail_lds_bytes(cols, hidden, in_features) <= lds_limit;
}

int launch_head_ce(hipStream_t s, const double* h, const double* w, const double* bias, const double* truth,
                   double* logits, double* grad, double* dx, bool mask, double* row_loss, double* loss,
                   int* flags, size_t rows, size_t cols, size_t in_features, LossMirror mirror,
                   const HiddenLayer* hidden) {
  if (!head_ce_supported(cols, in_features))
    return fail(RST_ERR_UNSUPPORTED, "fused head: %zu classes on %zu inputs do not fit", cols, in_features);
  if (hidden && (in_features > 112 || hidden->in_features > 112 || !dx))
    return fail(RST_ERR_UNSUPPORTED, "fused head with its hidden layer: %zu on %zu inputs do not fit",
                in_features, hidden->in_features);
  if (rows == 0) return RST_OK;
  // 16 rows to a workgroup while that leaves every compute unit with work, 32 beyond (each workgroup
  // pays a round trip to the one arrival counter); with the hidden layer 16 (one MFMA fragment) on 512 threads
  const int block_threads = (hidden || rows > 16 * 512 / 2) ? 512 : 256;
  const size_t rows_per_block = hidden ? 16 : block_threads / 16;
  const size_t blocks = (rows + rows_per_block - 1) / rows_per_block;
  if (blocks > 0x7fffffffull) return fail(RST_ERR_UNSUPPORTED, "too many rows for one launch");
  HeadParams p{};
  p.h = h; p.w = w; p.bias = bias; p.truth = truth;
  p.logits = logits; p.grad = grad; p.dx = dx;
  p.partial = row_loss;  // [rows] holds one word per workgroup
  p.arrivals = reinterpret_cast<unsigned long long*>(flags + 4);
  p.loss = loss; p.flags = flags;
  p.rows = rows; p.N = (int)cols; p.K = (int)in_features;
  p.mirror = mirror;
  p.mirror.hits = nullptr;  // the hit count is not taken here
  const bool masked = mask && dx;
  const int nc = cols <= 4 ? 4 : cols <= 8 ? 8 : 16;
  // (with the hidden layer: one workgroup per compute unit of the part at most - a constant, the grid
  // fixes the order in which the loss is summed - each walking over the batch)
  const dim3 grid((unsigned)(hidden && blocks > 256 ? 256 : blocks)), block(block_threads);
  if (hidden) {
    p.h1 = hidden->input; p.w2 = hidden->weight; p.b2 = hidden->bias;
    p.h_out = hidden->output; p.dx1 = hidden->input_grad;
    p.K1 = (int)hidden->in_features; p.mask1 = hidden->mask_input_grad ? 1 : 0;
    const size_t lds = tail_lds_bytes(cols, in_features, hidden->in_features);
#define RST_TAIL_LAUNCH(NC)                                                                          \
  do {                                                                                               \
    if (masked) hipLaunchKernelGGL((head_ce_kernel<8, NC, true, 512, true>), grid, block, lds, s, p); \
    else hipLaunchKernelGGL((head_ce_kernel<8, NC, false, 512, true>), grid, block, lds, s, p);      \
  } while (0)
    if (nc == 4) RST_TAIL_LAUNCH(4);
    else if (nc == 8) RST_TAIL_LAUNCH(8);
    else RST_TAIL_LAUNCH(16);
#undef RST_TAIL_LAUNCH
    RST_HIP(hipGetLastError());
    return RST_OK;
  }
  const size_t lds = (size_t)(nc + 2) * 16 * (in_features <= 16 * 8 ? 8 : 18) * sizeof(double);
#define RST_HEAD_LAUNCH3(KI, NC, M, B) hipLaunchKernelGGL((head_ce_kernel<KI, NC, M, B>), grid, block, lds, s, p)
#define RST_HEAD_LAUNCH(KI, NC)                                  \
  do {                                                           \
    if (block_threads == 256) {                                  \
      if (masked) RST_HEAD_LAUNCH3(KI, NC, true, 256);           \
      else RST_HEAD_LAUNCH3(KI, NC, false, 256);                 \
    } else {                                                     \
      if (masked) RST_HEAD_LAUNCH3(KI, NC, true, 512);           \
      else RST_HEAD_LAUNCH3(KI, NC, false, 512);                 \
    }                                                            \
  } while (0)
  if (in_features <= 16 * 8) {
    if (nc == 4) RST_HEAD_LAUNCH(8, 4);
    else if (nc == 8) RST_HEAD_LAUNCH(8, 8);
    else RST_HEAD_LAUNCH(8, 16);
  } else {
    if (nc == 4) RST_HEAD_LAUNCH(18, 4);
    else if (nc == 8) RST_HEAD_LAUNCH(18, 8);
    else RST_HEAD_LAUNCH(18, 16);
  }
#undef RST_HEAD_LAUNCH3
#undef RST_HEAD_LAUNCH
  RST_HIP(hipGetLastError());
  return RST_OK;
}

int launch_softmax_columns(hipStream_t s, const double* z, double* out, int* flags, size_t rows,
                           size_t cols) {
  if (rows == 0 || cols == 0) return RST_OK;
  hipLaunchKernelGGL(softmax_columns_kernel, dim3((unsigned)((cols + 255) / 256)), dim3(256), 0, s, z,
                     out, flags, rows, cols);
  RST_HIP(hipGetLastError());
  return RST_OK;
}

int launch_softmax_jacobian(hipStream_t s, double* jac, size_t cols) {
  if (cols == 0) return RST_OK;
  hipLaunchKernelGGL(softmax_jacobian_kernel, dim3((unsigned)((cols * cols + 255) / 256)), dim3(256),
                     0, s, jac, cols);
  RST_HIP(hipGetLastError());
  return RST_OK;
}

}  // namespace rst
