// Latent (low-rank compressed) attention: what surrounds the attention kernels of window_attn.hip.
//   latent_prep     in place on the fused down-projections [T][q_rank | kv_rank | rot]: RMSNorm of the
//                   query latent; RMSNorm of the key/value latent and rotation of the shared key part,
//                   both written to the pages: key page row = [latent | rotated part], value page =
//                   the latent once more, dim-major ([blocks][1][kv_rank][BS])
//   latent_queries  per head [q_lat (unrotated query times the key expansion) | rotated query part]
// Rotation: entries i and i + n/2 of the first 2 * nf entries (nf frequencies, freq[i] given in fp32)
// turn by the angle position * freq[i]; angles, sine and cosine are fp32.
#include "hy_common.h"

namespace k8sllm {

template <typename T>
__global__ __launch_bounds__(256) void latent_prep_kernel(T* __restrict__ proj, long stride, int Q, int R, int dr,
                                                          const float* __restrict__ qw, const float* __restrict__ kw,
                                                          float eps, const int* __restrict__ positions,
                                                          const float* __restrict__ freq, int nf,
                                                          T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                          const int* __restrict__ slots, int bs) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  T* row = proj + t * stride;
  float sq = 0.f, sc = 0.f;
  for (int c = threadIdx.x; c < Q; c += 256) {
    const float v = ldf(row + c);
    sq += v * v;
  }
  sq = block_sum<256>(sq, red);
  const float iq = 1.0f / sqrtf(sq / (float)Q + eps);
  for (int c = threadIdx.x; c < Q; c += 256) stf(row + c, ldf(row + c) * iq * qw[c]);
  if (kw == nullptr) return;  // a layer that reads another layer's pages
  for (int c = threadIdx.x; c < R; c += 256) {
    const float v = ldf(row + Q + c);
    sc += v * v;
  }
  sc = block_sum<256>(sc, red);
  const float ic = 1.0f / sqrtf(sc / (float)R + eps);
  const long slot = (slots != nullptr && k_cache != nullptr) ? slots[t] : -1;
  T* kp = slot >= 0 ? k_cache + slot * (long)(R + dr) : nullptr;
  for (int c = threadIdx.x; c < R; c += 256) {
    T* e = row + Q + c;
    stf(e, ldf(e) * ic * kw[c]);
    if (kp != nullptr) {
      kp[c] = *e;
      v_cache[((slot / bs) * R + c) * bs + slot % bs] = *e;
    }
  }
  T* kr = row + Q + R;
  const float pos = (float)positions[t];
  for (int i = threadIdx.x; i < dr; i += 256) {
    if (i < nf) {  // this thread owns the pair (i, i + nf)
      float sn, cs;
      sincosf(pos * freq[i], &sn, &cs);
      const float u = ldf(kr + i), v = ldf(kr + i + nf);
      stf(kr + i, u * cs - v * sn);
      stf(kr + i + nf, v * cs + u * sn);
      if (kp != nullptr) {
        kp[R + i] = kr[i];
        kp[R + i + nf] = kr[i + nf];
      }
    } else if (i >= 2 * nf && kp != nullptr) {
      kp[R + i] = kr[i];
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void latent_queries_kernel(T* __restrict__ out, const T* __restrict__ q, long q_stride,
                                                             const T* __restrict__ q_lat, long T_rows, int H, int dn,
                                                             int dr, int R, const int* __restrict__ positions,
                                                             const float* __restrict__ freq, int nf) {
  const long t = blockIdx.x;
  const int w = R + dr;
  const float pos = (float)positions[t];
  T* o = out + t * (long)H * w;
  for (int c = threadIdx.x; c < H * w; c += 256) {
    const int h = c / w, j = c - h * w;
    if (j < R) {
      o[c] = q_lat[((long)h * T_rows + t) * R + j];
      continue;
    }
    const int i = j - R;
    const T* qr = q + t * q_stride + (long)h * (dn + dr) + dn;
    if (i >= 2 * nf) {
      o[c] = qr[i];
      continue;
    }
    const int f = i < nf ? i : i - nf;
    float sn, cs;
    sincosf(pos * freq[f], &sn, &cs);
    const float u = ldf(qr + f), v = ldf(qr + f + nf);
    stf(o + c, i < nf ? u * cs - v * sn : v * cs + u * sn);
  }
}

}  // namespace k8sllm

using namespace k8sllm;

extern "C" {

int k8sllm_hy_latent_prep(void* proj, long stride, long T, int Q, int R, int dr, const float* qw, const float* kw,
                          float eps, const int* positions, const float* freq, int nf, void* k_cache, void* v_cache,
                          const int* slots, int bs, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (2 * nf > dr) return -1;
  if (f32)
    hipLaunchKernelGGL(latent_prep_kernel<float>, dim3(T), dim3(256), 0, s, (float*)proj, stride, Q, R, dr, qw, kw, eps,
                       positions, freq, nf, (float*)k_cache, (float*)v_cache, slots, bs);
  else
    hipLaunchKernelGGL(latent_prep_kernel<bf16_t>, dim3(T), dim3(256), 0, s, (bf16_t*)proj, stride, Q, R, dr, qw, kw,
                       eps, positions, freq, nf, (bf16_t*)k_cache, (bf16_t*)v_cache, slots, bs);
  return (int)hipGetLastError();
}

int k8sllm_hy_latent_queries(void* out, const void* q, long q_stride, const void* q_lat, long T, int H, int dn, int dr,
                             int R, const int* positions, const float* freq, int nf, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (2 * nf > dr) return -1;
  if (f32)
    hipLaunchKernelGGL(latent_queries_kernel<float>, dim3(T), dim3(256), 0, s, (float*)out, (const float*)q, q_stride,
                       (const float*)q_lat, T, H, dn, dr, R, positions, freq, nf);
  else
    hipLaunchKernelGGL(latent_queries_kernel<bf16_t>, dim3(T), dim3(256), 0, s, (bf16_t*)out, (const bf16_t*)q,
                       q_stride, (const bf16_t*)q_lat, T, H, dn, dr, R, positions, freq, nf);
  return (int)hipGetLastError();
}
}
