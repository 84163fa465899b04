// Counter-based synthetic data and initialisers.  value(seed, stream, index) is a pure function
// (a splitmix64 finaliser over a per-tensor key), so results do not depend on launch geometry.
// The reference initialises with ndarray-rand's unseedable thread RNG (src/module/init/he.rs:13);
// these kernels provide the same distributions reproducibly.
#include "common.h"

namespace rst {
namespace {

constexpr int kBlock = 256;

__host__ __device__ inline uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ULL;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
  return z ^ (z >> 31);
}

__host__ __device__ inline uint64_t tensor_key(uint64_t seed, uint64_t stream) {
  return mix64(mix64(seed) ^ (stream * 0xD1342543DE82EF95ULL));
}

__device__ inline uint64_t draw(uint64_t key, uint64_t index) {
  return mix64(key + index * 0x9E3779B97F4A7C15ULL);
}

__global__ __launch_bounds__(kBlock) void uniform_kernel(double* __restrict__ dst, size_t n,
                                                        uint64_t key, double lo, double hi) {
  size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
  size_t stride = (size_t)gridDim.x * kBlock;
  for (; i < n; i += stride) {
    double u = (double)(draw(key, i) >> 11) * 0x1.0p-53;
    dst[i] = lo + (hi - lo) * u;
  }
}

// Box-Muller, one normal per index from draws 2i and 2i+1.
__global__ __launch_bounds__(kBlock) void normal_kernel(double* __restrict__ dst, size_t n,
                                                       uint64_t key, double mean, double std) {
  const double two_pi = 6.283185307179586476925286766559;
  size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
  size_t stride = (size_t)gridDim.x * kBlock;
  for (; i < n; i += stride) {
    double u1 = ((double)(draw(key, 2 * i) >> 11) + 1.0) * 0x1.0p-53;  // (0, 1]
    double u2 = (double)(draw(key, 2 * i + 1) >> 11) * 0x1.0p-53;      // [0, 1)
    dst[i] = mean + std * (sqrt(-2.0 * log(u1)) * cos(two_pi * u2));
  }
}

__global__ __launch_bounds__(kBlock) void one_hot_kernel(double* __restrict__ dst, size_t rows,
                                                        size_t cols, uint64_t key) {
  size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
  size_t stride = (size_t)gridDim.x * kBlock;
  const size_t n = rows * cols;
  for (; i < n; i += stride) {
    size_t r = i / cols, c = i - r * cols;
    size_t label = (size_t)(draw(key, r) % (uint64_t)cols);
    dst[i] = (c == label) ? 1.0 : 0.0;
  }
}

inline unsigned blocks_for(size_t n) {
  size_t b = (n + kBlock - 1) / kBlock;
  if (b > 16384) b = 16384;
  if (b < 1) b = 1;
  return (unsigned)b;
}

}  // namespace

int launch_fill_uniform(hipStream_t s, double* dst, size_t n, uint64_t seed, uint64_t stream,
                        double lo, double hi) {
  if (n == 0) return RST_OK;
  hipLaunchKernelGGL(uniform_kernel, dim3(blocks_for(n)), dim3(kBlock), 0, s, dst, n,
                     tensor_key(seed, stream), lo, hi);
  RST_HIP(hipGetLastError());
  return RST_OK;
}

int launch_fill_normal(hipStream_t s, double* dst, size_t n, uint64_t seed, uint64_t stream,
                       double mean, double std) {
  if (n == 0) return RST_OK;
  hipLaunchKernelGGL(normal_kernel, dim3(blocks_for(n)), dim3(kBlock), 0, s, dst, n,
                     tensor_key(seed, stream), mean, std);
  RST_HIP(hipGetLastError());
  return RST_OK;
}

int launch_fill_one_hot(hipStream_t s, double* dst, size_t rows, size_t cols, uint64_t seed,
                        uint64_t stream) {
  if (rows == 0 || cols == 0) return RST_OK;
  hipLaunchKernelGGL(one_hot_kernel, dim3(blocks_for(rows * cols)), dim3(kBlock), 0, s, dst, rows,
                     cols, tensor_key(seed, stream));
  RST_HIP(hipGetLastError());
  return RST_OK;
}

}  // namespace rst
