// Helpers shared by the layer-list decoders' kernels: activations are either bf16 (raw 16-bit
// patterns, common.h) or fp32, selected by a template parameter; all arithmetic is fp32.
#pragma once
#include "common.h"

namespace k8sllm {

template <typename T>
__device__ __forceinline__ float ldf(const T* p);
template <>
__device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p) { return bf2f(*p); }

template <typename T>
__device__ __forceinline__ void stf(T* p, float v);
template <>
__device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void stf<bf16_t>(bf16_t* p, float v) { *p = f2bf(v); }

// element i of a tensor whose dtype is only known at run time: 1 = bf16, 2 = fp32
__device__ __forceinline__ float ld_any(const void* p, int dt, long i) {
  return dt == 2 ? reinterpret_cast<const float*>(p)[i] : bf2f(reinterpret_cast<const bf16_t*>(p)[i]);
}

__device__ __forceinline__ float silu_f(float z) { return z / (1.f + __expf(-z)); }

// the segment that holds row r: largest s with cu[s] <= r (cu has S + 1 entries, cu[0] = 0)
__device__ __forceinline__ int find_segment(const int* __restrict__ cu, int S, int r) {
  int lo = 0, hi = S - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu[mid] <= r) lo = mid; else hi = mid - 1;
  }
  return lo;
}

}  // namespace k8sllm
