// Windowed grouped-query attention with a softmax sink over a paged cache (any head size).
//   qk_norm_cache             whole-projection RMSNorm of q and of k in place, k / v -> pages
//   window_attention_prefill  one wave per (chunk row, query head)
//   window_attention_decode   one wave per (sequence, query head)
// Pages: k_cache [blocks][BS][G*dk] (a token's keys contiguous), v_cache [blocks][G][dv][BS] (a value
// dim's BS tokens contiguous: the layout the PV products read along); a sequence's page list is a row of
// block_tables.  Row at position p sees positions max(0, p - window + 1) .. p (window 0: 0 .. p).
// The sink is one more softmax term with no value and a fixed score - 0, or a learned unscaled logit
// per query head (sinks[h]): the running maximum starts at that score and the running denominator at 1.  Scores, weights and the output accumulation are fp32.
#include "hy_common.h"

namespace k8sllm {

constexpr int kMaxVC = 4;  // output dims per lane of the vector decode kernel: dv <= 64 * kMaxVC
constexpr int kMaxDK = 512;
constexpr int kGenVC = 8;  // the any-size kernels: dv <= 64 * kGenVC, dk <= kGenDK
constexpr int kGenDK = 1024;

template <typename T>
__global__ __launch_bounds__(256) void qk_norm_cache_kernel(T* __restrict__ qkv, long stride,
                                                            const float* __restrict__ qw,
                                                            const float* __restrict__ kw, float eps, int nq, int nk,
                                                            int nv, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                            const int* __restrict__ slots, int bs) {
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
    for (int c = threadIdx.x; c < nv; c += 256) v_cache[((slot / bs) * nv + c) * bs + slot % bs] = row[nq + nk + c];
}

// One wave: query q (dk values at q_row) against cached positions [lo, hi) of one kv head.
template <typename T>
__device__ __forceinline__ void attend_wave(T* __restrict__ out_row, const T* __restrict__ q_row,
                                            const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                            const int* __restrict__ bt, int lo, int hi, int g, int G, int dk, int dv,
                                            int bs, float scale, int sink, float sink_z, float* q_s, float* p_s) {
  const int lane = threadIdx.x & 63;
  for (int c = lane; c < dk; c += 64) q_s[c] = ldf(q_row + c) * scale;
  __syncthreads();  // one wave per workgroup: orders the LDS writes before the other lanes' reads
  float m = sink ? sink_z : -INFINITY, l = sink ? 1.f : 0.f;  // the sink: one term exp(sink_z - m)
  float acc[kGenVC];
#pragma unroll
  for (int c = 0; c < kGenVC; ++c) acc[c] = 0.f;
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
    const float mt = fmaxf(m, wave_max_dpp(s));
    const float p = j < hi ? expf(s - mt) : 0.f;
    const float alpha = expf(m - mt);  // m = -inf only before the first key (no sink): exp(-inf) = 0
    l = l * alpha + wave_sum_dpp(p);
    m = mt;
    __syncthreads();  // the previous tile's reads of p_s are done
    p_s[lane] = p;
    __syncthreads();
    const int n = min(64, hi - j0);
#pragma unroll
    for (int c = 0; c < kGenVC; ++c) {
      const int dcol = lane + 64 * c;
      float a = acc[c] * alpha;
      if (dcol < dv)
        for (int i = 0; i < n; ++i) {
          const int jj = j0 + i;
          a += p_s[i] * ldf(v_cache + ((long)bt[jj / bs] * vrow + (long)g * dv + dcol) * bs + jj % bs);
        }
      acc[c] = a;
    }
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int c = 0; c < kGenVC; ++c) {
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
                                                            int window, int sink, const float* __restrict__ sinks) {
  __shared__ float q_s[kGenDK];
  __shared__ float p_s[64];
  const int r = blockIdx.x, h = blockIdx.y;
  const int s = find_segment(cu, S, r);
  const int p = ctx[s] + r - cu[s];
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  attend_wave<T>(out + (long)r * Hq * dv + (long)h * dv, qkv + (long)r * q_stride + (long)h * dk, k_cache, v_cache,
                 block_tables + (long)s * bt_stride, lo, p + 1, h / (Hq / G), G, dk, dv, bs, scale, sink,
                 sinks != nullptr ? sinks[h] : 0.f, q_s, p_s);
}

template <typename T>
__global__ __launch_bounds__(64) void window_decode_kernel(T* __restrict__ out, const T* __restrict__ qkv,
                                                           long q_stride, const T* __restrict__ k_cache,
                                                           const T* __restrict__ v_cache,
                                                           const int* __restrict__ block_tables, int bt_stride,
                                                           const int* __restrict__ seq_lens, int Hq, int G, int dk,
                                                           int dv, int bs, float scale, int window, int sink,
                                                           const float* __restrict__ sinks) {
  __shared__ float q_s[kGenDK];
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
                 n, h / (Hq / G), G, dk, dv, bs, scale, sink, sinks != nullptr ? sinks[h] : 0.f, q_s, p_s);
}

// bf16 decode with 16-byte loads, 16-token pages: one workgroup (NW = 8 waves; 4 for 8 query heads
// per kv head, whose merge buffers would not fit otherwise) per (sequence, kv head) serves all
// R = Hq / G query heads of that kv head, so every cached key and value is read once.  The waves take
// the window's 64-key tiles (aligned to 64, i.e. four whole pages) in turn and their partial (maximum,
// denominator, output) triples are merged through LDS at the end; only wave 0 starts from the sink's
// (0, 1); scores carry log2 e so that every exponential is one v_exp_f32.  Scores: lane = key, the lane walks its key row in 8-element pieces against the R queries
// held in LDS (fp32).  Values: lane = value dim (+ 64 c); a page's 16 tokens of that dim are two
// 16-byte loads, 2 KiB contiguous per wave; the weights come back from LDS four at a time.
template <int R, int NW>
__global__ __launch_bounds__(64 * NW) void window_decode_vec_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ qkv,
                                                                long q_stride, const bf16_t* __restrict__ k_cache,
                                                                const bf16_t* __restrict__ v_cache,
                                                                const int* __restrict__ block_tables, int bt_stride,
                                                                const int* __restrict__ seq_lens, int Hq, int G, int dk,
                                                                int dv, float scale, int window, int sink,
                                                                const float* __restrict__ sinks) {
  constexpr int bs = 16;
  __shared__ __attribute__((aligned(16))) float q_s[R * kMaxDK];
  __shared__ __attribute__((aligned(16))) float p_s[NW][R][64];
  __shared__ float ml_s[NW][R][2];
  __shared__ float acc_s[NW][R][64 * kMaxVC];
  const int b = blockIdx.x, g = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = seq_lens[b];
  bf16_t* o = out + (long)b * Hq * dv + (long)g * R * dv;
  if (n <= 0) {  // padding row of a decode bucket
    for (int c = threadIdx.x; c < R * dv; c += 64 * NW) o[c] = 0;
    return;
  }
  const bf16_t* q = qkv + (long)b * q_stride + (long)g * R * dk;
  for (int c = threadIdx.x; c < R * dk; c += 64 * NW) q_s[(c / dk) * kMaxDK + c % dk] = bf2f(q[c]) * (scale * 1.44269504088896341f);  // base-2 scores
  __syncthreads();
  const int* bt = block_tables + (long)b * bt_stride;
  const int lo = window > 0 ? max(0, n - window) : 0;
  const bool first = sink && wave == 0;
  float m[R], l[R], acc[R][kMaxVC];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    // the sink's logit is not scaled; scores live in the base-2 domain
    m[r] = first ? (sinks != nullptr ? sinks[g * R + r] * 1.44269504088896341f : 0.f) : -INFINITY;
    l[r] = first ? 1.f : 0.f;
#pragma unroll
    for (int c = 0; c < kMaxVC; ++c) acc[r][c] = 0.f;
  }
  const long krs = (long)G * dk;
  for (int j0 = (lo & ~63) + 64 * wave; j0 < n; j0 += 64 * NW) {
    const int j = j0 + lane;
    const bool valid = j >= lo && j < n;
    float sc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) sc[r] = 0.f;
    if (valid) {
      const bf16_t* kp = k_cache + ((long)bt[j / bs] * bs + j % bs) * krs + (long)g * dk;
      for (int c0 = 0; c0 < dk; c0 += 64) {  // 8 pieces of the key row in flight at a time
        uint4 kq[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (c0 + 8 * u < dk) kq[u] = *reinterpret_cast<const uint4*>(kp + c0 + 8 * u);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int c = c0 + 8 * u;
          if (c < dk) {
            float kv[8];
            unpack8(kq[u], kv);
#pragma unroll
            for (int r = 0; r < R; ++r) {
              const float4 qa = *reinterpret_cast<const float4*>(&q_s[r * kMaxDK + c]);
              const float4 qb = *reinterpret_cast<const float4*>(&q_s[r * kMaxDK + c + 4]);
              sc[r] += kv[0] * qa.x + kv[1] * qa.y + kv[2] * qa.z + kv[3] * qa.w + kv[4] * qb.x + kv[5] * qb.y +
                       kv[6] * qb.z + kv[7] * qb.w;
            }
          }
        }
      }
    }
    // value loads of the tile's pages go out before the softmax arithmetic: 2 x 16 bytes per page and
    // 64 dims (pages at or past the sequence's end are not touched: their weights are zero)
    const int npg = min(4, (n - j0 + bs - 1) / bs);
    uint4 vq[4][kMaxVC][2];
#pragma unroll
    for (int pg = 0; pg < 4; ++pg)
      if (pg < npg) {
        const long base = ((long)bt[j0 / bs + pg] * G + g) * dv;
#pragma unroll
        for (int c = 0; c < kMaxVC; ++c)
          if (lane + 64 * c < dv) {
            const uint4* vp = reinterpret_cast<const uint4*>(v_cache + (base + lane + 64 * c) * bs);
            vq[pg][c][0] = vp[0];
            vq[pg][c][1] = vp[1];
          }
      }
    __builtin_amdgcn_wave_barrier();  // this wave's previous reads of its p_s rows come first
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float sv = valid ? sc[r] : -INFINITY;
      const float mt = fmaxf(m[r], wave_max_dpp(sv));  // the tile holds at least one live key, or m is the sink's
      const float pw = (valid && mt != -INFINITY) ? __builtin_amdgcn_exp2f(sv - mt) : 0.f;
      const float alpha = (m[r] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m[r] - mt);
      l[r] = l[r] * alpha + wave_sum_dpp(pw);
      m[r] = mt;
      p_s[wave][r][lane] = pw;
#pragma unroll
      for (int c = 0; c < kMaxVC; ++c) acc[r][c] *= alpha;
    }
    __builtin_amdgcn_wave_barrier();  // a wave's LDS instructions execute in issue order
#pragma unroll
    for (int pg = 0; pg < 4; ++pg)
      if (pg < npg) {
#pragma unroll
        for (int c = 0; c < kMaxVC; ++c)
          if (lane + 64 * c < dv) {
            float vv[16];
            unpack8(vq[pg][c][0], vv);
            unpack8(vq[pg][c][1], vv + 8);
#pragma unroll
            for (int r = 0; r < R; ++r) {
              float a = acc[r][c];
#pragma unroll
              for (int t4 = 0; t4 < 4; ++t4) {
                const float4 pq = *reinterpret_cast<const float4*>(&p_s[wave][r][16 * pg + 4 * t4]);
                a += pq.x * vv[4 * t4] + pq.y * vv[4 * t4 + 1] + pq.z * vv[4 * t4 + 2] + pq.w * vv[4 * t4 + 3];
              }
              acc[r][c] = a;
            }
          }
      }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
#pragma unroll
    for (int c = 0; c < kMaxVC; ++c)
      if (lane + 64 * c < dv) acc_s[wave][r][lane + 64 * c] = acc[r][c];
    if (lane == 0) {
      ml_s[wave][r][0] = m[r];
      ml_s[wave][r][1] = l[r];
    }
  }
  __syncthreads();
  for (int c = threadIdx.x; c < R * dv; c += 64 * NW) {
    const int r = c / dv, dcol = c - r * dv;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) M = fmaxf(M, ml_s[w][r][0]);
    float L = 0.f, val = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float f = ml_s[w][r][0] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ml_s[w][r][0] - M);
      L += ml_s[w][r][1] * f;
      val += acc_s[w][r][dcol] * f;
    }
    o[c] = f2bf(L > 0.f ? val / L : 0.f);
  }
}

// bf16 prefill on the matrix cores, head sizes that are multiples of 32 (keys) / 16 (values).
// One wave = 16 consecutive chunk rows of one sequence x one query head; key tiles of 16.
//   S^T[key][q]  = K Q^T      v_mfma_f32_16x16x32_bf16: A = K rows (16-byte loads straight from the
//                             pages), B = the wave's Q rows (held in registers for the whole loop)
//   O^T[d][q]   += V^T P^T    v_mfma_f32_16x16x16_bf16: B = the score accumulator itself (query on
//                             the lane, 4 keys per lane: the C layout of S^T IS the B layout of P^T),
//                             A = V^T, 8-byte loads from the d-major V page (tokens contiguous)
// With the query on the lane the running maximum, denominator and the rescale of O are lane-local
// (two xor-shuffles per reduction).  Scores, weights and sums are fp32 (base-2 exponentials: the
// scale carries log2 e); P is rounded to bf16 for the PV product.
template <int DK, int DV, int QT>
__global__ __launch_bounds__(64) void window_prefill_mfma_kernel(
    bf16_t* __restrict__ out, const bf16_t* __restrict__ qkv, long q_stride, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int* __restrict__ cu, const int* __restrict__ ctx,
    const int* __restrict__ block_tables, int bt_stride, int S, int Hq, int G, float scale, int window,
    int sink, const float* __restrict__ sinks) {
  // pages hold 16 tokens; scores live in the base-2 domain (scale * log2 e folded in) so that every
  // exponential is one v_exp_f32
  const float sc2 = scale * 1.44269504088896341f;
  constexpr int QB = 16 * QT;  // query rows per wave: QT tiles of 16 share every K and V^T fragment
  int tile = blockIdx.x, s = 0, n = 0;
  for (; s < S; ++s) {  // q-blocks are numbered segment by segment
    n = cu[s + 1] - cu[s];
    const int nt = (n + QB - 1) / QB;
    if (tile < nt) break;
    tile -= nt;
  }
  if (s >= S) return;
  const int q0 = tile * QB, nq = min(QB, n - q0);
  const int h = blockIdx.y, g = h / (Hq / G);
  const int lane = threadIdx.x, c16 = lane & 15, quad = lane >> 4;
  const int* bt = block_tables + (long)s * bt_stride;
  const int row0 = cu[s] + q0, p0 = ctx[s] + q0;
  int my_p[QT], my_lo[QT];
  bool q_live[QT];
  bf16x8 qf[QT][DK / 32];
  f32x4 oacc[QT][DV / 16];
  float m[QT], l[QT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    const int myq = min(16 * t + c16, nq - 1);
    my_p[t] = p0 + myq;
    my_lo[t] = window > 0 ? max(0, my_p[t] - window + 1) : 0;
    q_live[t] = 16 * t + c16 < nq;
    const bf16_t* qrow = qkv + (long)(row0 + myq) * q_stride + (long)h * DK;
#pragma unroll
    for (int ks = 0; ks < DK / 32; ++ks) qf[t][ks] = *reinterpret_cast<const bf16x8*>(qrow + 32 * ks + 8 * quad);
#pragma unroll
    for (int dt = 0; dt < DV / 16; ++dt) oacc[t][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    m[t] = sink ? (sinks != nullptr ? sinks[blockIdx.y] * 1.44269504088896341f : 0.f) : -INFINITY;
    l[t] = sink ? 1.f : 0.f;
  }
  const int lo_t = window > 0 ? max(0, p0 - window + 1) : 0, hi = p0 + nq;
  const long krs = (long)G * DK, vrs = (long)G * DV;
  // Register double buffer: while tile j0 is computed, the K and V^T fragments of tile j0 + 16 are
  // in flight, and the page id of tile j0 + 32 behind them (no load waits on a load issued in the
  // same iteration).  A key tile is one 16-token page: its V^T fragments (4 consecutive tokens of
  // one value dim per lane) are 8-byte loads straight from the d-major page, 512 contiguous bytes
  // per 16 dims - no LDS, no barrier.
  const bf16_t* kbase = k_cache + (long)g * DK + 8 * quad;
  const bf16_t* vbase = v_cache + ((long)g * DV + c16) * 16 + 4 * quad;
  const int jfirst = lo_t & ~15;
  int pg_n = bt[jfirst >> 4];
  bf16x8 kf_n[DK / 32];
  s16x4 vf_n[DV / 16];
  auto issue = [&](int j0) {  // loads of tile j0 from the page id in pg_n
    const bf16_t* krow = kbase + (((long)pg_n << 4) + (min(j0 + c16, hi - 1) & 15)) * krs;
#pragma unroll
    for (int ks = 0; ks < DK / 32; ++ks) kf_n[ks] = *reinterpret_cast<const bf16x8*>(krow + 32 * ks);
    const bf16_t* vpg = vbase + (long)pg_n * vrs * 16;
#pragma unroll
    for (int dt = 0; dt < DV / 16; ++dt) vf_n[dt] = *reinterpret_cast<const s16x4*>(vpg + dt * 256);
  };
  issue(jfirst);
  pg_n = bt[min(jfirst + 16, hi - 1) >> 4];
  for (int j0 = jfirst; j0 < hi; j0 += 16) {
    bf16x8 kf[DK / 32];
    s16x4 vf[DV / 16];
#pragma unroll
    for (int ks = 0; ks < DK / 32; ++ks) kf[ks] = kf_n[ks];
#pragma unroll
    for (int dt = 0; dt < DV / 16; ++dt) vf[dt] = vf_n[dt];
    if (j0 + 16 < hi) {
      issue(j0 + 16);
      pg_n = bt[min(j0 + 32, hi - 1) >> 4];
    }
    s16x4 pb[QT];
    float alpha[QT];
    bool rescale[QT];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      f32x4 sacc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < DK / 32; ++ks) sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[ks], qf[t][ks], sacc, 0, 0, 0);
      float sv[4], tmax = -INFINITY;
#pragma unroll
      for (int i = 0; i < 4; ++i) {  // sacc[i]: key j0 + 4 quad + i, query 16 t + c16
        const int j = j0 + 4 * quad + i;
        sv[i] = (q_live[t] && j >= my_lo[t] && j <= my_p[t]) ? sacc[i] * sc2 : -INFINITY;
        tmax = fmaxf(tmax, sv[i]);
      }
      tmax = xor32_max_f(xor16_max(tmax));
      const float mn = fmaxf(m[t], tmax);
      alpha[t] = m[t] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m[t] - mn);
      float ps = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pv = sv[i] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(sv[i] - mn);
        ps += pv;
        pb[t][i] = (short)f2bf(pv);
      }
      ps = xor32_sum_f(xor16_sum(ps));
      l[t] = l[t] * alpha[t] + ps;
      m[t] = mn;
      rescale[t] = __any(alpha[t] != 1.f);
    }
    // wave-uniform: once the running maxima settle, most tiles skip the rescale.  ONE block for a
    // row tile's whole accumulator: a branch around each value tile's four multiplies is flattened by
    // the compiler into multiplies on every tile
#pragma unroll
    for (int t = 0; t < QT; ++t)
      if (rescale[t]) {
#pragma unroll
        for (int dt = 0; dt < DV / 16; ++dt)
#pragma unroll
          for (int i = 0; i < 4; ++i) oacc[t][dt][i] *= alpha[t];
      }
#pragma unroll
    for (int dt = 0; dt < DV / 16; ++dt) {
      const s16x4 a = vf[dt];
#pragma unroll
      for (int t = 0; t < QT; ++t) oacc[t][dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, pb[t], oacc[t][dt], 0, 0, 0);
    }
  }
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    if (!q_live[t]) continue;  // oacc[t][dt][i] = O[q = 16 t + c16][d = 16 dt + 4 quad + i]
    const float inv = l[t] > 0.f ? 1.f / l[t] : 0.f;
    bf16_t* orow = out + (long)(row0 + 16 * t + c16) * Hq * DV + (long)h * DV;
#pragma unroll
    for (int dt = 0; dt < DV / 16; ++dt) {
      uint2 w;
      w.x = pack2(oacc[t][dt][0] * inv, oacc[t][dt][1] * inv);
      w.y = pack2(oacc[t][dt][2] * inv, oacc[t][dt][3] * inv);
      *reinterpret_cast<uint2*>(orow + 16 * dt + 4 * quad) = w;
    }
  }
}

}  // namespace k8sllm

using namespace k8sllm;

extern "C" {

int k8sllm_hy_qk_norm_cache(void* qkv, long stride, const float* qw, const float* kw, float eps, long T, int nq,
                            int nk, int nv, void* k_cache, void* v_cache, const int* slots, int bs, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (f32)
    hipLaunchKernelGGL(qk_norm_cache_kernel<float>, dim3(T), dim3(256), 0, s, (float*)qkv, stride, qw, kw, eps, nq, nk,
                       nv, (float*)k_cache, (float*)v_cache, slots, bs);
  else
    hipLaunchKernelGGL(qk_norm_cache_kernel<bf16_t>, dim3(T), dim3(256), 0, s, (bf16_t*)qkv, stride, qw, kw, eps, nq,
                       nk, nv, (bf16_t*)k_cache, (bf16_t*)v_cache, slots, bs);
  return (int)hipGetLastError();
}

int k8sllm_hy_window_prefill(void* out, const void* qkv, long q_stride, const void* k_cache, const void* v_cache,
                             const int* cu, const int* ctx, const int* block_tables, int bt_stride, int S, long T,
                             int Hq, int G, int dk, int dv, int bs, float scale, int window, int sink,
                             const float* sinks, int f32, int mfma, hipStream_t s) {
  if (T <= 0 || S <= 0) return 0;
  if (dk > kGenDK || dv > 64 * kGenVC || G < 1 || Hq % G) return -1;
  // bf16 with matrix-core head sizes and 16-byte aligned rows: the MFMA kernel
  if (!f32 && mfma && bs == 16 && q_stride % 8 == 0 && (dk == 64 || dk == 128) && (dv == 64 || dv == 128)) {
    // query rows per wave: 32 once the step is large enough to fill the chip that way (two row tiles
    // share every K / V^T fragment), else 16; mfma = 16 / 32 / 64 forces one (tests, measurements)
    const int qrows = mfma >= 16 ? mfma : (T * Hq >= 64 * 1024 ? 32 : 16);
    const dim3 grid((unsigned)(T / qrows + S), (unsigned)Hq);
#define K8SLLM_WP(DK, DV, QT)                                                                                          \
  hipLaunchKernelGGL((window_prefill_mfma_kernel<DK, DV, QT>), grid, dim3(64), 0, s, (bf16_t*)out, (const bf16_t*)qkv,  \
                     q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, cu, ctx, block_tables, bt_stride, S, Hq, \
                     G, scale, window, sink, sinks)
#define K8SLLM_WPQ(DK, DV)                                       \
  if (qrows == 64) K8SLLM_WP(DK, DV, 4);                         \
  else if (qrows == 32) K8SLLM_WP(DK, DV, 2);                    \
  else K8SLLM_WP(DK, DV, 1)
    if (mfma >= 16 && mfma != 16 && mfma != 32 && mfma != 64) return -1;
    if (dk == 64 && dv == 64) { K8SLLM_WPQ(64, 64); }
    else if (dk == 64) { K8SLLM_WPQ(64, 128); }
    else if (dv == 64) { K8SLLM_WPQ(128, 64); }
    else { K8SLLM_WPQ(128, 128); }
#undef K8SLLM_WPQ
#undef K8SLLM_WP
    return (int)hipGetLastError();
  }
  if (f32)
    hipLaunchKernelGGL(window_prefill_kernel<float>, dim3(T, Hq), dim3(64), 0, s, (float*)out, (const float*)qkv,
                       q_stride, (const float*)k_cache, (const float*)v_cache, cu, ctx, block_tables, bt_stride, S, Hq,
                       G, dk, dv, bs, scale, window, sink, sinks);
  else
    hipLaunchKernelGGL(window_prefill_kernel<bf16_t>, dim3(T, Hq), dim3(64), 0, s, (bf16_t*)out, (const bf16_t*)qkv,
                       q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, cu, ctx, block_tables, bt_stride, S,
                       Hq, G, dk, dv, bs, scale, window, sink, sinks);
  return (int)hipGetLastError();
}

int k8sllm_hy_window_decode(void* out, const void* qkv, long q_stride, const void* k_cache, const void* v_cache,
                            const int* block_tables, int bt_stride, const int* seq_lens, int B, int Hq, int G, int dk,
                            int dv, int bs, float scale, int window, int sink, const float* sinks, int f32, int vec,
                            hipStream_t s) {
  if (B <= 0) return 0;
  if (dk > kGenDK || dv > 64 * kGenVC || G < 1 || Hq % G) return -1;
  const int R = Hq / G;
  if (!f32 && vec && bs == 16 && dk % 8 == 0 && q_stride % 8 == 0 && dk <= kMaxDK && dv <= 64 * kMaxVC &&
      (R == 1 || R == 2 || R == 4 || R == 8)) {
#define K8SLLM_WD(RR)                                                                                                  \
  hipLaunchKernelGGL((window_decode_vec_kernel<RR, (RR == 8 ? 4 : 8)>), dim3(B, G), dim3(RR == 8 ? 256 : 512), 0, s,     \
                     (bf16_t*)out, (const bf16_t*)qkv,                                                                  \
                     q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, bt_stride, seq_lens, Hq, G, \
                     dk, dv, scale, window, sink, sinks)
    if (R == 1) K8SLLM_WD(1);
    else if (R == 2) K8SLLM_WD(2);
    else if (R == 4) K8SLLM_WD(4);
    else K8SLLM_WD(8);
#undef K8SLLM_WD
    return (int)hipGetLastError();
  }
  if (f32)
    hipLaunchKernelGGL(window_decode_kernel<float>, dim3(B, Hq), dim3(64), 0, s, (float*)out, (const float*)qkv,
                       q_stride, (const float*)k_cache, (const float*)v_cache, block_tables, bt_stride, seq_lens, Hq, G,
                       dk, dv, bs, scale, window, sink, sinks);
  else
    hipLaunchKernelGGL(window_decode_kernel<bf16_t>, dim3(B, Hq), dim3(64), 0, s, (bf16_t*)out, (const bf16_t*)qkv,
                       q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, bt_stride, seq_lens, Hq,
                       G, dk, dv, bs, scale, window, sink, sinks);
  return (int)hipGetLastError();
}
}
