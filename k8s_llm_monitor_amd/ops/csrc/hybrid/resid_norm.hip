// fp32 residual stream of the layer-list decoders.
//   embed_pos         x[t] = embed[id] + pos[position]            (fp32 rows)
//   add_norm          residual += a0 + a1 + a2 + vec;  out = residual / rms(residual) * (w | 1 + w)
//   gated_group_norm  out = group_rms_norm(y * silu(z)) * w       (y fp32, groups of equal size)
//   swiglu            out = silu(gu[:, :f]) * gu[:, f:]
#include "hy_common.h"

namespace k8sllm {

template <typename T>
__global__ __launch_bounds__(256) void embed_pos_kernel(float* __restrict__ out, const int* __restrict__ ids,
                                                        const int* __restrict__ positions, const T* __restrict__ emb,
                                                        const T* __restrict__ pos, const int* __restrict__ src,
                                                        const int* __restrict__ prev, int d, int vocab, int max_pos) {
  const long t = blockIdx.x;
  int id = ids[t];
  if (src != nullptr && src[t] >= 0) id = prev[src[t]];
  id = min(max(id, 0), vocab - 1);
  const T* e = emb + (long)id * d;
  const T* p = nullptr;
  if (pos != nullptr) p = pos + (long)min(max(positions[t], 0), max_pos - 1) * d;
  for (int c = threadIdx.x; c < d; c += 256) out[t * d + c] = ldf(e + c) + (p != nullptr ? ldf(p + c) : 0.f);
}

template <typename T>
__global__ __launch_bounds__(256) void add_norm_kernel(T* __restrict__ out, float* __restrict__ residual,
                                                       const void* a0, int t0, const void* a1, int t1, const void* a2,
                                                       int t2, const float* __restrict__ vec,
                                                       const float* __restrict__ w, int d, float eps, int one_plus) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  float* r = residual + row * d;
  float ss = 0.f;
  if ((d & 7) == 0) {  // 8 columns per thread and trip, 16 / 32-byte accesses
    for (int c = threadIdx.x * 8; c < d; c += 2048) {
      float x[8], a[8];
      load8(r + c, x);
      if (t0) {
        load8_any(a0, t0, row * d + c, a);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] += a[i];
      }
      if (t1) {
        load8_any(a1, t1, row * d + c, a);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] += a[i];
      }
      if (t2) {
        load8_any(a2, t2, row * d + c, a);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] += a[i];
      }
      if (vec != nullptr) {
        load8(vec + c, a);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] += a[i];
      }
      store8(r + c, x);
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += x[i] * x[i];
    }
    ss = block_sum<256>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)d + eps);
    for (int c = threadIdx.x * 8; c < d; c += 2048) {  // each thread re-reads what it wrote
      float x[8], g[8];
      load8(r + c, x);
      load8(w + c, g);
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] *= inv * (one_plus ? 1.f + g[i] : g[i]);
      store8(out + row * d + c, x);
    }
    return;
  }
  for (int c = threadIdx.x; c < d; c += 256) {
    float x = r[c];
    if (t0) x += ld_any(a0, t0, row * d + c);
    if (t1) x += ld_any(a1, t1, row * d + c);
    if (t2) x += ld_any(a2, t2, row * d + c);
    if (vec != nullptr) x += vec[c];
    r[c] = x;
    ss += x * x;
  }
  ss = block_sum<256>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += 256) {  // each thread re-reads what it wrote
    const float g = one_plus ? 1.f + w[c] : w[c];
    stf(out + row * d + c, r[c] * inv * g);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(T* __restrict__ out, const float* __restrict__ y,
                                                               const T* __restrict__ z, long z_stride,
                                                               const float* __restrict__ w, int n, int groups,
                                                               float eps) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  const int g = blockIdx.y, gs = n / groups;
  const float* yr = y + row * n + (long)g * gs;
  const T* zr = z + row * z_stride + (long)g * gs;
  float ss = 0.f;
  for (int c = threadIdx.x; c < gs; c += 256) {
    const float v = yr[c] * silu_f(ldf(zr + c));
    ss += v * v;
  }
  ss = block_sum<256>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)gs + eps);
  for (int c = threadIdx.x; c < gs; c += 256) {
    const float v = yr[c] * silu_f(ldf(zr + c));
    stf(out + row * n + (long)g * gs + c, v * inv * w[(long)g * gs + c]);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void swiglu_kernel(T* __restrict__ out, const T* __restrict__ gu, long rows, int f) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * f) return;
  const long r = i / f;
  const int c = (int)(i - r * f);
  stf(out + i, silu_f(ldf(gu + r * 2 * f + c)) * ldf(gu + r * 2 * f + f + c));
}

}  // namespace k8sllm

using namespace k8sllm;

extern "C" {

int k8sllm_hy_embed_pos(float* out, const int* ids, const int* positions, const void* emb, const void* pos,
                        const int* src, const int* prev, long T, int d, int vocab, int max_pos, int f32,
                        hipStream_t s) {
  if (T <= 0) return 0;
  if (f32)
    hipLaunchKernelGGL(embed_pos_kernel<float>, dim3(T), dim3(256), 0, s, out, ids, positions, (const float*)emb,
                       (const float*)pos, src, prev, d, vocab, max_pos);
  else
    hipLaunchKernelGGL(embed_pos_kernel<bf16_t>, dim3(T), dim3(256), 0, s, out, ids, positions, (const bf16_t*)emb,
                       (const bf16_t*)pos, src, prev, d, vocab, max_pos);
  return (int)hipGetLastError();
}

int k8sllm_hy_add_norm(void* out, float* residual, const void* a0, int t0, const void* a1, int t1, const void* a2,
                       int t2, const float* vec, const float* w, long rows, int d, float eps, int one_plus, int f32,
                       hipStream_t s) {
  if (rows <= 0) return 0;
  if (f32)
    hipLaunchKernelGGL(add_norm_kernel<float>, dim3(rows), dim3(256), 0, s, (float*)out, residual, a0, t0, a1, t1, a2,
                       t2, vec, w, d, eps, one_plus);
  else
    hipLaunchKernelGGL(add_norm_kernel<bf16_t>, dim3(rows), dim3(256), 0, s, (bf16_t*)out, residual, a0, t0, a1, t1,
                       a2, t2, vec, w, d, eps, one_plus);
  return (int)hipGetLastError();
}

int k8sllm_hy_gated_group_norm(void* out, const float* y, const void* z, long z_stride, const float* w, long rows,
                               int n, int groups, float eps, int f32, hipStream_t s) {
  if (rows <= 0) return 0;
  if (groups < 1 || n % groups) return -1;
  if (f32)
    hipLaunchKernelGGL(gated_group_norm_kernel<float>, dim3(rows, groups), dim3(256), 0, s, (float*)out, y,
                       (const float*)z, z_stride, w, n, groups, eps);
  else
    hipLaunchKernelGGL(gated_group_norm_kernel<bf16_t>, dim3(rows, groups), dim3(256), 0, s, (bf16_t*)out, y,
                       (const bf16_t*)z, z_stride, w, n, groups, eps);
  return (int)hipGetLastError();
}

int k8sllm_hy_swiglu(void* out, const void* gu, long rows, int f, int f32, hipStream_t s) {
  const long n = rows * f;
  if (n <= 0) return 0;
  const unsigned g = (unsigned)((n + 255) / 256);
  if (f32)
    hipLaunchKernelGGL(swiglu_kernel<float>, dim3(g), dim3(256), 0, s, (float*)out, (const float*)gu, rows, f);
  else
    hipLaunchKernelGGL(swiglu_kernel<bf16_t>, dim3(g), dim3(256), 0, s, (bf16_t*)out, (const bf16_t*)gu, rows, f);
  return (int)hipGetLastError();
}
}
