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

// 8 consecutive elements (16-byte aligned for bf16, 32-byte for fp32) as floats, and back
__device__ __forceinline__ void load8(const bf16_t* p, float* f) { unpack8(*reinterpret_cast<const uint4*>(p), f); }
__device__ __forceinline__ void load8(const float* p, float* f) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w;
  f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}
__device__ __forceinline__ void store8(bf16_t* p, const float* f) { *reinterpret_cast<uint4*>(p) = pack8(f); }
__device__ __forceinline__ void store8(float* p, const float* f) {
  *reinterpret_cast<float4*>(p) = make_float4(f[0], f[1], f[2], f[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(f[4], f[5], f[6], f[7]);
}
__device__ __forceinline__ void load8_any(const void* p, int dt, long i, float* f) {
  if (dt == 2) load8(reinterpret_cast<const float*>(p) + i, f);
  else load8(reinterpret_cast<const bf16_t*>(p) + i, f);
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
