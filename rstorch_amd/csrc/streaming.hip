// HBM-bound streaming kernels: ReLU forward/backward (unfused form), fill, the bias-gradient
// column mean, SGD and row arg-max accuracy.  All of them move each byte exactly once with
// 16-byte accesses where alignment allows.
#include "argmax.h"
#include "common.h"

namespace rst {
namespace {

typedef double v2d __attribute__((ext_vector_type(2)));
constexpr int kBlock = 256;
// one wavefront per workgroup streams a few per cent faster for the wide element-wise passes
// (measured on MI355X for ReLU and SGD alike)
constexpr int kStreamBlock = 64;

inline bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

inline unsigned grid_for(size_t work_items, size_t per_block) {
  size_t blocks = (work_items + per_block - 1) / per_block;
  if (blocks < 1) blocks = 1;
  return (unsigned)blocks;
}

// ---- ReLU -----------------------------------------------------------------------------------
// forward: out = max(x, 0); fmax returns the non-NaN operand, like f64::max in the reference.
__global__ __launch_bounds__(kStreamBlock) void relu_forward_v2(const v2d* __restrict__ x,
                                                         v2d* __restrict__ out, size_t n2) {
  size_t i = (size_t)blockIdx.x * kStreamBlock + threadIdx.x;
  if (i < n2) {
    v2d v = __builtin_nontemporal_load(x + i);
    v.x = fmax(v.x, 0.0);
    v.y = fmax(v.y, 0.0);
    out[i] = v;
  }
}
__global__ __launch_bounds__(kBlock) void relu_forward_s(const double* __restrict__ x,
                                                        double* __restrict__ out, size_t n) {
  size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < n) out[i] = fmax(x[i], 0.0);
}
// backward: out = g * (x > 0 ? 1 : 0), a real multiply so that inf * 0 stays NaN.
__global__ __launch_bounds__(kStreamBlock) void relu_backward_v2(const v2d* __restrict__ g,
                                                          const v2d* __restrict__ x,
                                                          v2d* __restrict__ out, size_t n2) {
  size_t i = (size_t)blockIdx.x * kStreamBlock + threadIdx.x;
  if (i < n2) {
    v2d gv = __builtin_nontemporal_load(g + i);
    v2d xv = __builtin_nontemporal_load(x + i);
    v2d r;
    r.x = gv.x * (xv.x > 0.0 ? 1.0 : 0.0);
    r.y = gv.y * (xv.y > 0.0 ? 1.0 : 0.0);
    out[i] = r;
  }
}
__global__ __launch_bounds__(kBlock) void relu_backward_s(const double* __restrict__ g,
                                                         const double* __restrict__ x,
                                                         double* __restrict__ out, size_t n) {
  size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < n) out[i] = g[i] * (x[i] > 0.0 ? 1.0 : 0.0);
}

// ---- fill -----------------------------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void fill_kernel(double* __restrict__ dst, size_t n,
                                                     double value) {
  size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
  size_t stride = (size_t)gridDim.x * kBlock;
  for (; i < n; i += stride) dst[i] = value;
}

// ---- column mean (bias gradient) -----------------------------------------------------------
// 256 threads = 16 row groups x 16 columns; a thread adds rows rg, rg+16, ... of its column in
// order, the 16 partial sums are combined through LDS in a fixed order, then divided.
__global__ __launch_bounds__(kBlock) void column_mean_kernel(const double* __restrict__ g,
                                                            double* __restrict__ out, size_t rows,
                                                            size_t cols, double divisor) {
  __shared__ double part[16][17];
  const int c = threadIdx.x & 15, rg = threadIdx.x >> 4;
  const size_t col = (size_t)blockIdx.x * 16 + c;
  double s = 0.0;
  if (col < cols)
    for (size_t r = rg; r < rows; r += 16) s += g[r * cols + col];
  part[rg][c] = s;
  __syncthreads();
  if (rg == 0 && col < cols) {
    double t = 0.0;
#pragma unroll
    for (int k = 0; k < 16; ++k) t += part[k][c];
    out[col] = t / divisor;
  }
}

// ---- SGD --------------------------------------------------------------------------------------
// parm = parm - (lr * grad) with the two roundings of the reference: the product is rounded to
// f64, then the difference.  Contraction into a fused multiply-add is switched off here (and for
// the whole library on the compiler command line; the __dmul_rn intrinsic is a plain multiply
// that the compiler would be free to fuse).  Streaming loads and stores bypass temporal caching.
__device__ __forceinline__ double sgd_scalar(double w, double g, double lr) {
#pragma clang fp contract(off)
  const double step = lr * g;
  return w - step;
}

__device__ __forceinline__ v2d sgd_update(v2d w, v2d g, double lr) {
  v2d r;
  r.x = sgd_scalar(w.x, g.x, lr);
  r.y = sgd_scalar(w.y, g.y, lr);
  return r;
}

// One wavefront per workgroup: measured on MI355X, 64-thread workgroups stream about 4 % faster
// than 256-thread ones for this 2-reads-1-write pattern (6.70 vs 6.44 TB/s over 268 M parameters).
constexpr int kSgdBlock = 64;

__global__ __launch_bounds__(kSgdBlock) void sgd_flat_v2(v2d* __restrict__ w,
                                                        const v2d* __restrict__ g, size_t n2,
                                                        double lr) {
  size_t i = (size_t)blockIdx.x * kSgdBlock + threadIdx.x;
  if (i < n2) {
    v2d wv = __builtin_nontemporal_load(w + i);
    v2d gv = __builtin_nontemporal_load(g + i);
    __builtin_nontemporal_store(sgd_update(wv, gv, lr), w + i);
  }
}
__global__ __launch_bounds__(kBlock) void sgd_flat_s(double* __restrict__ w,
                                                    const double* __restrict__ g, size_t n,
                                                    double lr) {
  size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < n) w[i] = sgd_scalar(w[i], g[i], lr);
}

constexpr unsigned long long kSgdPerBlock = 2ull * kSgdBlock;  // doubles per workgroup

// One launch over many tensors: the workgroup finds its tensor by bisection over the block
// prefix in the descriptor table (uniform per workgroup, scalar loads).
__global__ __launch_bounds__(kSgdBlock) void sgd_multi_kernel(const SgdTensor* __restrict__ table,
                                                          int n_tensors, double lr) {
  const unsigned long long b = blockIdx.x;
  int lo = 0, hi = n_tensors - 1;
  while (lo < hi) {
    int mid = (lo + hi + 1) >> 1;
    if (table[mid].first_block <= b) lo = mid; else hi = mid - 1;
  }
  const SgdTensor t = table[lo];
  const unsigned long long first = (b - t.first_block) * kSgdPerBlock + 2ull * threadIdx.x;
  if (first >= t.count) return;
  double* w = t.parm + first;
  const double* g = t.grad + first;
  const bool pair = first + 1 < t.count;
  if (pair && ((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(g)) % 16 == 0)) {
    v2d wv = __builtin_nontemporal_load(reinterpret_cast<v2d*>(w));
    v2d gv = __builtin_nontemporal_load(reinterpret_cast<const v2d*>(g));
    __builtin_nontemporal_store(sgd_update(wv, gv, lr), reinterpret_cast<v2d*>(w));
  } else {
    w[0] = sgd_scalar(w[0], g[0], lr);
    if (pair) w[1] = sgd_scalar(w[1], g[1], lr);
  }
}

// ---- accuracy -----------------------------------------------------------------------------------
// One wavefront per row: every lane scans a strided part keeping its first maximum, then the
// lanes are combined preferring the larger value and, on ties, the smaller column - which is
// the reference's "first maximum wins" (strict > replacement).  NaN never replaces.
__device__ __forceinline__ unsigned row_argmax(const double* __restrict__ row, size_t cols,
                                               int lane) {
  // the reference starts from element 0 and replaces only when e > acc
  double v = 0.0;
  unsigned idx = kNoIndex;
  for (size_t c = lane; c < cols; c += 64) argmax_step(v, idx, row[c], c);
  for (int off = 32; off > 0; off >>= 1) {
    double ov = __shfl_xor(v, off);
    unsigned oidx = __shfl_xor(idx, off);
    argmax_combine(v, idx, ov, oidx);
  }
  return idx;
}

__global__ __launch_bounds__(kBlock) void accuracy_kernel(const double* __restrict__ pred,
                                                         const double* __restrict__ truth,
                                                         size_t rows, size_t cols,
                                                         unsigned long long* hits) {
  const int lane = threadIdx.x & 63;
  const size_t row = (size_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  if (row >= rows) return;
  unsigned a = row_argmax(pred + row * cols, cols, lane);
  unsigned b = row_argmax(truth + row * cols, cols, lane);
  if (lane == 0 && a == b) atomicAdd(hits, 1ull);
}

// Narrow rows (up to kNarrowCols columns: the ten classes of the README network): a thread per row
// instead of a wavefront - a wavefront on ten columns leaves 54 lanes idle and a batch of 8192 rows
// takes 12 us.  The scan is the reference's own (ascending columns, first maximum wins).
constexpr size_t kNarrowCols = 32;
__global__ __launch_bounds__(kBlock) void accuracy_narrow_kernel(const double* __restrict__ pred,
                                                                const double* __restrict__ truth,
                                                                size_t rows, size_t cols,
                                                                unsigned long long* hits) {
  const size_t row = (size_t)blockIdx.x * kBlock + threadIdx.x;
  bool hit = false;
  if (row < rows) {
    const double* p = pred + row * cols;
    const double* t = truth + row * cols;
    double pv = 0.0, tv = 0.0;
    unsigned pi = kNoIndex, ti = kNoIndex;
    for (size_t c = 0; c < cols; ++c) {
      argmax_step(pv, pi, p[c], c);
      argmax_step(tv, ti, t[c], c);
    }
    hit = pi == ti;
  }
  const unsigned long long agreeing = __ballot(hit);
  if ((threadIdx.x & 63) == 0 && agreeing != 0ull) atomicAdd(hits, (unsigned long long)__popcll(agreeing));
}

// Wide rows (a 32768-logit row is 256 KiB): one workgroup of 256 threads per row, 16-byte loads,
// eight of them in flight per thread and array; a wavefront per row leaves a row's 512 KiB to 64
// lanes and the chip to a thousand wavefronts (measured 0.48 ms on 1024 x 32768, 1.1 TB/s).
__device__ __forceinline__ unsigned wide_row_argmax(const double* __restrict__ row, size_t cols, unsigned* scratch_idx,
                                                    double* scratch_v) {
  constexpr int UNR = 8;
  double v = 0.0;
  unsigned idx = kNoIndex;
  const size_t pairs = cols / 2;
  const v2d* row2 = reinterpret_cast<const v2d*>(row);
  size_t p = threadIdx.x;
  for (; p + (size_t)(UNR - 1) * kBlock < pairs; p += (size_t)UNR * kBlock) {
    v2d t[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) t[u] = __builtin_nontemporal_load(row2 + p + (size_t)u * kBlock);
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const size_t c = 2 * (p + (size_t)u * kBlock);
      argmax_step(v, idx, t[u].x, c);
      argmax_step(v, idx, t[u].y, c + 1);
    }
  }
  for (; p < pairs; p += kBlock) {
    const v2d t = row2[p];
    argmax_step(v, idx, t.x, 2 * p);
    argmax_step(v, idx, t.y, 2 * p + 1);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) argmax_combine(v, idx, __shfl_xor(v, off), __shfl_xor(idx, off));
  const int wave = threadIdx.x >> 6;
  __syncthreads();  // (the scratch may still be read from the previous row array)
  if ((threadIdx.x & 63) == 0) { scratch_v[wave] = v; scratch_idx[wave] = idx; }
  __syncthreads();
  v = scratch_v[0];
  idx = scratch_idx[0];
#pragma unroll
  for (int w = 1; w < kBlock / 64; ++w) argmax_combine(v, idx, scratch_v[w], scratch_idx[w]);
  return idx;
}

__global__ __launch_bounds__(kBlock) void accuracy_wide_kernel(const double* __restrict__ pred,
                                                              const double* __restrict__ truth, size_t cols,
                                                              unsigned long long* hits) {
  __shared__ double scratch_v[kBlock / 64];
  __shared__ unsigned scratch_idx[kBlock / 64];
  const size_t row = blockIdx.x;
  const unsigned a = wide_row_argmax(pred + row * cols, cols, scratch_idx, scratch_v);
  const unsigned b = wide_row_argmax(truth + row * cols, cols, scratch_idx, scratch_v);
  if (threadIdx.x == 0 && a == b) atomicAdd(hits, 1ull);
}

__global__ void zero_hits_kernel(unsigned long long* hits) { hits[0] = 0ull; }

}  // namespace

int launch_relu_forward(hipStream_t s, const double* x, double* out, size_t n) {
  if (n == 0) return RST_OK;
  if (n % 2 == 0 && aligned16(x) && aligned16(out)) {
    hipLaunchKernelGGL(relu_forward_v2, dim3(grid_for(n / 2, kStreamBlock)), dim3(kStreamBlock), 0, s,
                       reinterpret_cast<const v2d*>(x), reinterpret_cast<v2d*>(out), n / 2);
  } else {
    hipLaunchKernelGGL(relu_forward_s, dim3(grid_for(n, kBlock)), dim3(kBlock), 0, s, x, out, n);
  }
  RST_HIP(hipGetLastError());
  return RST_OK;
}

int launch_relu_backward(hipStream_t s, const double* g, const double* x, double* out, size_t n) {
  if (n == 0) return RST_OK;
  if (n % 2 == 0 && aligned16(g) && aligned16(x) && aligned16(out)) {
    hipLaunchKernelGGL(relu_backward_v2, dim3(grid_for(n / 2, kStreamBlock)), dim3(kStreamBlock), 0, s,
                       reinterpret_cast<const v2d*>(g), reinterpret_cast<const v2d*>(x),
                       reinterpret_cast<v2d*>(out), n / 2);
  } else {
    hipLaunchKernelGGL(relu_backward_s, dim3(grid_for(n, kBlock)), dim3(kBlock), 0, s, g, x, out, n);
  }
  RST_HIP(hipGetLastError());
  return RST_OK;
}

int launch_fill(hipStream_t s, double* dst, size_t n, double value) {
  if (n == 0) return RST_OK;
  size_t blocks = (n + kBlock - 1) / kBlock;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(fill_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, s, dst, n, value);
  RST_HIP(hipGetLastError());
  return RST_OK;
}

int launch_column_mean(hipStream_t s, const double* g, double* out, size_t rows, size_t cols,
                       double divisor) {
  if (cols == 0) return RST_OK;
  hipLaunchKernelGGL(column_mean_kernel, dim3(grid_for(cols, 16)), dim3(kBlock), 0, s, g, out, rows,
                     cols, divisor);
  RST_HIP(hipGetLastError());
  return RST_OK;
}

int launch_sgd_flat(hipStream_t s, double* parm, const double* grad, size_t n, double lr) {
  if (n == 0) return RST_OK;
  if (aligned16(parm) && aligned16(grad)) {
    size_t n2 = n / 2;
    if (n2) {
      if ((n2 + kSgdBlock - 1) / kSgdBlock > 0x7fffffffull)
        return fail(RST_ERR_UNSUPPORTED, "parameter range too large for one launch");
      hipLaunchKernelGGL(sgd_flat_v2, dim3(grid_for(n2, kSgdBlock)), dim3(kSgdBlock), 0, s,
                         reinterpret_cast<v2d*>(parm), reinterpret_cast<const v2d*>(grad), n2, lr);
    }
    if (n & 1)
      hipLaunchKernelGGL(sgd_flat_s, dim3(1), dim3(kBlock), 0, s, parm + (n - 1), grad + (n - 1),
                         (size_t)1, lr);
  } else {
    hipLaunchKernelGGL(sgd_flat_s, dim3(grid_for(n, kBlock)), dim3(kBlock), 0, s, parm, grad, n, lr);
  }
  RST_HIP(hipGetLastError());
  return RST_OK;
}

unsigned long long sgd_blocks_for(unsigned long long count) {
  return (count + kSgdPerBlock - 1) / kSgdPerBlock;
}

int launch_sgd_multi(hipStream_t s, const SgdTensor* device_table, size_t n_tensors,
                     unsigned long long total_blocks, double lr) {
  if (n_tensors == 0 || total_blocks == 0) return RST_OK;
  if (total_blocks > 0x7fffffffull)
    return fail(RST_ERR_UNSUPPORTED, "too many parameters for one launch");
  hipLaunchKernelGGL(sgd_multi_kernel, dim3((unsigned)total_blocks), dim3(kSgdBlock), 0, s,
                     device_table, (int)n_tensors, lr);
  RST_HIP(hipGetLastError());
  return RST_OK;
}

// Small inputs: one workgroup of 16 wavefronts counts every row (wavefront w takes rows w, w+16,
// ...), adds the sixteen counts in order and stores the total in the device word and in its host
// mirror - one launch, no atomics, nothing to copy back.
__global__ __launch_bounds__(1024) void accuracy_small_kernel(const double* __restrict__ pred,
                                                             const double* __restrict__ truth,
                                                             size_t rows, size_t cols,
                                                             unsigned long long* hits,
                                                             unsigned long long* hits_mirror,
                                                             ResultSlot* slots, unsigned ticket) {
  __shared__ unsigned counts[16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  unsigned mine = 0;
  for (size_t row = wave; row < rows; row += 16) {
    const unsigned a = row_argmax(pred + row * cols, cols, lane);
    const unsigned b = row_argmax(truth + row * cols, cols, lane);
    mine += a == b ? 1u : 0u;
  }
  if (lane == 0) counts[wave] = mine;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long total = 0;
    for (int w = 0; w < 16; ++w) total += counts[w];
    hits[0] = total;
    if (hits_mirror) hits_mirror[0] = total;
    if (slots) store_result_slot(slots + 1, 0.0, total, true, 0u, ticket);
  }
}

// The count of a multi-workgroup accuracy launch, from the device word into its host mirror and the
// pinned result record (with the launch's ticket): the host then waits for exactly this result by
// polling instead of copying it back and synchronising the stream - work that a caller has put on the
// stream behind the accuracy (the input gradients of a coming backward pass) is not waited for.
__global__ void publish_hits_kernel(const unsigned long long* __restrict__ hits, unsigned long long* hits_mirror,
                                    ResultSlot* slots, unsigned ticket) {
  const unsigned long long total = hits[0];
  hits_mirror[0] = total;
  store_result_slot(slots + 1, 0.0, total, true, 0u, ticket);
}

int launch_accuracy(hipStream_t s, const double* pred, const double* truth, size_t rows,
                    size_t cols, unsigned long long* hits, unsigned long long* hits_mirror,
                    bool* mirrored, ResultSlot* slots, unsigned ticket) {
  if (mirrored) *mirrored = false;
  if (hits_mirror && mirrored && rows * cols <= (size_t)1 << 16) {
    hipLaunchKernelGGL(accuracy_small_kernel, dim3(1), dim3(1024), 0, s, pred, truth, rows, cols, hits,
                       hits_mirror, slots, ticket);
    RST_HIP(hipGetLastError());
    *mirrored = true;
    return RST_OK;
  }
  hipLaunchKernelGGL(zero_hits_kernel, dim3(1), dim3(1), 0, s, hits);
  if (rows && cols) {
    if (cols >= 4096 && cols % 2 == 0 && aligned16(pred) && aligned16(truth) && rows <= 0x7fffffffull)
      hipLaunchKernelGGL(accuracy_wide_kernel, dim3((unsigned)rows), dim3(kBlock), 0, s, pred, truth, cols, hits);
    else if (cols <= kNarrowCols && rows >= 1024)
      hipLaunchKernelGGL(accuracy_narrow_kernel, dim3(grid_for(rows, kBlock)), dim3(kBlock), 0, s, pred, truth, rows,
                         cols, hits);
    else
      hipLaunchKernelGGL(accuracy_kernel, dim3(grid_for(rows, kBlock / 64)), dim3(kBlock), 0, s, pred,
                         truth, rows, cols, hits);
  }
  RST_HIP(hipGetLastError());
  if (hits_mirror && mirrored && slots) {
    hipLaunchKernelGGL(publish_hits_kernel, dim3(1), dim3(1), 0, s, hits, hits_mirror, slots, ticket);
    RST_HIP(hipGetLastError());
    *mirrored = true;
  }
  return RST_OK;
}

}  // namespace rst
