// Windowed grouped-query attention with a softmax sink over a paged cache (any head size).
//   qk_norm_cache             whole-projection RMSNorm of q and of k in place, k / v -> pages
//   window_attention_prefill  one wave per (chunk row, query head)
//   window_attention_decode   one wave per (sequence, query head)
// Pages: k_cache [blocks][BS][G*dk], v_cache [blocks][BS][G*dv]; a sequence's page list is a row of
// block_tables.  Row at position p sees positions max(0, p - window + 1) .. p (window 0: 0 .. p).
// The sink is one more softmax term with score 0 and no value: the running maximum starts at 0 and
// the running denominator at 1.  Scores, weights and the output accumulation are fp32.
#include "hy_common.h"

namespace k8sllm {

constexpr int kMaxVC = 4;  // output dims per lane: dv <= 64 * kMaxVC
constexpr int kMaxDK = 512;

template <typename T>
__global__ __launch_bounds__(256) void qk_norm_cache_kernel(T* __restrict__ qkv, long stride,
                                                            const float* __restrict__ qw,
                                                            const float* __restrict__ kw, float eps, int nq, int nk,
                                                            int nv, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                            const int* __restrict__ slots) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  T* row = qkv + t * stride;
  float sq = 0.f, sk = 0.f;
  for (int c = threadIdx.x; c < nq; c += 256) {
    const float x = ldf(row + c);
    sq += x * x;
  }
  for (int c = threadIdx.x; c < nk; c += 256) {
    const float x = ldf(row + nq + c);
    sk += x * x;
  }
  sq = block_sum<256>(sq, red);
  sk = block_sum<256>(sk, red);
  const float iq = 1.0f / sqrtf(sq / (float)nq + eps), ik = 1.0f / sqrtf(sk / (float)nk + eps);
  const long slot = (slots != nullptr && k_cache != nullptr) ? slots[t] : -1;
  for (int c = threadIdx.x; c < nq; c += 256) stf(row + c, ldf(row + c) * iq * qw[c]);
  for (int c = threadIdx.x; c < nk; c += 256) {
    stf(row + nq + c, ldf(row + nq + c) * ik * kw[c]);
    if (slot >= 0) k_cache[slot * nk + c] = row[nq + c];
  }
  if (slot >= 0)
    for (int c = threadIdx.x; c < nv; c += 256) v_cache[slot * nv + c] = row[nq + nk + c];
}

// One wave: query q (dk values at q_row) against cached positions [lo, hi) of one kv head.
template <typename T>
__device__ __forceinline__ void attend_wave(T* __restrict__ out_row, const T* __restrict__ q_row,
                                            const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                            const int* __restrict__ bt, int lo, int hi, int g, int G, int dk, int dv,
                                            int bs, float scale, int sink, float* q_s, float* p_s) {
  const int lane = threadIdx.x & 63;
  for (int c = lane; c < dk; c += 64) q_s[c] = ldf(q_row + c) * scale;
  __syncthreads();  // one wave per workgroup: orders the LDS writes before the other lanes' reads
  float m = sink ? 0.f : -INFINITY, l = sink ? 1.f : 0.f;
  float acc[kMaxVC];
#pragma unroll
  for (int c = 0; c < kMaxVC; ++c) acc[c] = 0.f;
  const long krow = (long)G * dk, vrow = (long)G * dv;
  for (int j0 = lo; j0 < hi; j0 += 64) {
    const int j = j0 + lane;
    float s = -INFINITY;
    if (j < hi) {
      const T* kp = k_cache + ((long)bt[j / bs] * bs + j % bs) * krow + (long)g * dk;
      float a = 0.f;
      for (int c = 0; c < dk; ++c) a += q_s[c] * ldf(kp + c);
      s = a;
    }
    const float mt = fmaxf(m, wave_max(s));
    const float p = j < hi ? expf(s - mt) : 0.f;
    const float alpha = expf(m - mt);  // m = -inf only before the first key (no sink): exp(-inf) = 0
    l = l * alpha + wave_sum(p);
    m = mt;
    __syncthreads();  // the previous tile's reads of p_s are done
    p_s[lane] = p;
    __syncthreads();
    const int n = min(64, hi - j0);
#pragma unroll
    for (int c = 0; c < kMaxVC; ++c) {
      const int dcol = lane + 64 * c;
      float a = acc[c] * alpha;
      if (dcol < dv)
        for (int i = 0; i < n; ++i) {
          const int jj = j0 + i;
          a += p_s[i] * ldf(v_cache + ((long)bt[jj / bs] * bs + jj % bs) * vrow + (long)g * dv + dcol);
        }
      acc[c] = a;
    }
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int c = 0; c < kMaxVC; ++c) {
    const int dcol = lane + 64 * c;
    if (dcol < dv) stf(out_row + dcol, acc[c] * inv);
  }
}

template <typename T>
__global__ __launch_bounds__(64) void window_prefill_kernel(T* __restrict__ out, const T* __restrict__ qkv,
                                                            long q_stride, const T* __restrict__ k_cache,
                                                            const T* __restrict__ v_cache,
                                                            const int* __restrict__ cu, const int* __restrict__ ctx,
                                                            const int* __restrict__ block_tables, int bt_stride, int S,
                                                            int Hq, int G, int dk, int dv, int bs, float scale,
                                                            int window, int sink) {
  __shared__ float q_s[kMaxDK];
  __shared__ float p_s[64];
  const int r = blockIdx.x, h = blockIdx.y;
  const int s = find_segment(cu, S, r);
  const int p = ctx[s] + r - cu[s];
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  attend_wave<T>(out + (long)r * Hq * dv + (long)h * dv, qkv + (long)r * q_stride + (long)h * dk, k_cache, v_cache,
                 block_tables + (long)s * bt_stride, lo, p + 1, h / (Hq / G), G, dk, dv, bs, scale, sink, q_s, p_s);
}

template <typename T>
__global__ __launch_bounds__(64) void window_decode_kernel(T* __restrict__ out, const T* __restrict__ qkv,
                                                           long q_stride, const T* __restrict__ k_cache,
                                                           const T* __restrict__ v_cache,
                                                           const int* __restrict__ block_tables, int bt_stride,
                                                           const int* __restrict__ seq_lens, int Hq, int G, int dk,
                                                           int dv, int bs, float scale, int window, int sink) {
  __shared__ float q_s[kMaxDK];
  __shared__ float p_s[64];
  const int b = blockIdx.x, h = blockIdx.y;
  const int n = seq_lens[b];
  T* o = out + (long)b * Hq * dv + (long)h * dv;
  if (n <= 0) {  // padding row of a decode bucket
    for (int c = threadIdx.x; c < dv; c += 64) stf(o + c, 0.f);
    return;
  }
  const int lo = window > 0 ? max(0, n - window) : 0;
  attend_wave<T>(o, qkv + (long)b * q_stride + (long)h * dk, k_cache, v_cache, block_tables + (long)b * bt_stride, lo,
                 n, h / (Hq / G), G, dk, dv, bs, scale, sink, q_s, p_s);
}

}  // namespace k8sllm

using namespace k8sllm;

extern "C" {

int k8sllm_hy_qk_norm_cache(void* qkv, long stride, const float* qw, const float* kw, float eps, long T, int nq,
                            int nk, int nv, void* k_cache, void* v_cache, const int* slots, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (f32)
    hipLaunchKernelGGL(qk_norm_cache_kernel<float>, dim3(T), dim3(256), 0, s, (float*)qkv, stride, qw, kw, eps, nq, nk,
                       nv, (float*)k_cache, (float*)v_cache, slots);
  else
    hipLaunchKernelGGL(qk_norm_cache_kernel<bf16_t>, dim3(T), dim3(256), 0, s, (bf16_t*)qkv, stride, qw, kw, eps, nq,
                       nk, nv, (bf16_t*)k_cache, (bf16_t*)v_cache, slots);
  return (int)hipGetLastError();
}

int k8sllm_hy_window_prefill(void* out, const void* qkv, long q_stride, const void* k_cache, const void* v_cache,
                             const int* cu, const int* ctx, const int* block_tables, int bt_stride, int S, long T,
                             int Hq, int G, int dk, int dv, int bs, float scale, int window, int sink, int f32,
                             hipStream_t s) {
  if (T <= 0 || S <= 0) return 0;
  if (dk > kMaxDK || dv > 64 * kMaxVC || G < 1 || Hq % G) return -1;
  if (f32)
    hipLaunchKernelGGL(window_prefill_kernel<float>, dim3(T, Hq), dim3(64), 0, s, (float*)out, (const float*)qkv,
                       q_stride, (const float*)k_cache, (const float*)v_cache, cu, ctx, block_tables, bt_stride, S, Hq,
                       G, dk, dv, bs, scale, window, sink);
  else
    hipLaunchKernelGGL(window_prefill_kernel<bf16_t>, dim3(T, Hq), dim3(64), 0, s, (bf16_t*)out, (const bf16_t*)qkv,
                       q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, cu, ctx, block_tables, bt_stride, S,
                       Hq, G, dk, dv, bs, scale, window, sink);
  return (int)hipGetLastError();
}

int k8sllm_hy_window_decode(void* out, const void* qkv, long q_stride, const void* k_cache, const void* v_cache,
                            const int* block_tables, int bt_stride, const int* seq_lens, int B, int Hq, int G, int dk,
                            int dv, int bs, float scale, int window, int sink, int f32, hipStream_t s) {
  if (B <= 0) return 0;
  if (dk > kMaxDK || dv > 64 * kMaxVC || G < 1 || Hq % G) return -1;
  if (f32)
    hipLaunchKernelGGL(window_decode_kernel<float>, dim3(B, Hq), dim3(64), 0, s, (float*)out, (const float*)qkv,
                       q_stride, (const float*)k_cache, (const float*)v_cache, block_tables, bt_stride, seq_lens, Hq, G,
                       dk, dv, bs, scale, window, sink);
  else
    hipLaunchKernelGGL(window_decode_kernel<bf16_t>, dim3(B, Hq), dim3(64), 0, s, (bf16_t*)out, (const bf16_t*)qkv,
                       q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, bt_stride, seq_lens, Hq,
                       G, dk, dv, bs, scale, window, sink);
  return (int)hipGetLastError();
}
}
