// First-maximum-wins arg-max of a row (src/utils.rs:44-53: the accumulator starts at element 0 and is
// replaced only when e > acc), shared by the accuracy kernels and the cross entropy that counts hits.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>

namespace rst {

constexpr unsigned kNoIndex = 0xffffffffu;

// One more element x at column c into a thread's running (v, idx).  A NaN never wins a strict
// comparison, so it only counts when it is element 0 (the reference's initial accumulator), where
// it also can never be replaced.
__device__ __forceinline__ void argmax_step(double& v, unsigned& idx, double x, size_t c) {
  if (x != x && c != 0) return;
  if (idx == kNoIndex) { v = x; idx = (unsigned)c; }
  else if (x > v) { v = x; idx = (unsigned)c; }
}

// Two partial results: the larger value wins and, on ties, the smaller column.
__device__ __forceinline__ void argmax_combine(double& v, unsigned& idx, double ov, unsigned oidx) {
  if (oidx != kNoIndex && (idx == kNoIndex || ov > v || (ov == v && oidx < idx))) {
    v = ov;
    idx = oidx;
  }
}

// One result record in pinned host memory, written with a single 16-byte store so that the ticket
// and the value it announces arrive together: {value or count (8 bytes), flags, ticket}.
typedef unsigned v4u __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store_result_slot(void* slot, double value, unsigned long long count, bool is_count,
                                                  unsigned flags, unsigned ticket) {
  const unsigned long long bits = is_count ? count : (unsigned long long)__double_as_longlong(value);
  v4u record;
  record.x = (unsigned)(bits & 0xffffffffull);
  record.y = (unsigned)(bits >> 32);
  record.z = flags;
  record.w = ticket;
  __builtin_nontemporal_store(record, reinterpret_cast<v4u*>(slot));
}

}  // namespace rst
