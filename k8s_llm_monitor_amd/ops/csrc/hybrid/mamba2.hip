// Mamba-2 mixer kernels (any sizes; state and recurrence fp32).
//   conv_silu        causal per-channel convolution + SiLU over a column range of the in-projection,
//                    one thread per (row, channel); the taps-1 inputs before a segment come from the
//                    sequence's conv state slot (zeros for a sequence that starts in this step)
//   conv_state_step  advances each segment's conv state slot to the segment's end
//   ssm_scan         S <- exp(-exp(A_log) dt) S + dt B x^T;  y = S^T C + D x, token by token per
//                    segment; the state slot [nh][N][P] is read at the start, written at the end
// A segment is one sequence's rows of this step: cu[s] .. cu[s+1], ctx[s] tokens already in its
// state (0: starts from zero), slot[s] its state slot (< 0: skipped).
#include "hy_common.h"

namespace k8sllm {

constexpr int kMaxTaps = 16;

template <typename T>
__global__ __launch_bounds__(256) void conv_silu_kernel(T* __restrict__ out, const T* __restrict__ proj, long stride,
                                                        int col0, int C, const float* __restrict__ cw,
                                                        const float* __restrict__ cb, int taps,
                                                        const T* __restrict__ state, const int* __restrict__ cu,
                                                        const int* __restrict__ ctx, const int* __restrict__ slot,
                                                        int S) {
  const int row = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int s = find_segment(cu, S, row);
  const int sl = slot[s];
  if (sl < 0) {  // padding row: defined output, no state
    stf(out + (long)row * C + c, 0.f);
    return;
  }
  const int r = row - cu[s];
  const bool carried = ctx[s] > 0;
  float acc = cb[c];
  for (int j = 0; j < taps; ++j) {
    const int i = r - (taps - 1) + j;  // offset within the segment of the input under tap j
    float x = 0.f;
    if (i >= 0)
      x = ldf(proj + (long)(row - (taps - 1) + j) * stride + col0 + c);
    else if (carried)
      x = ldf(state + ((long)sl * (taps - 1) + (taps - 1 + i)) * C + c);
    acc += cw[(long)c * taps + j] * x;
  }
  stf(out + (long)row * C + c, silu_f(acc));
}

template <typename T>
__global__ __launch_bounds__(256) void conv_state_step_kernel(T* __restrict__ state, const T* __restrict__ proj,
                                                              long stride, int col0, int C, int taps,
                                                              const int* __restrict__ cu, const int* __restrict__ ctx,
                                                              const int* __restrict__ slot) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  const int sl = slot[s];
  const int n = cu[s + 1] - cu[s];
  if (c >= C || sl < 0 || n <= 0) return;
  const int H = taps - 1;
  const bool carried = ctx[s] > 0;
  T* st = state + (long)sl * H * C + c;
  T keep[kMaxTaps];
  for (int i = 0; i < H; ++i) {  // entry i of the new history = element n + i of [old history ; segment]
    const int k = n + i;
    if (k >= H)
      keep[i] = proj[(long)(cu[s] + k - H) * stride + col0 + c];
    else if (carried)
      keep[i] = st[(long)k * C];
    else
      stf(&keep[i], 0.f);
  }
  for (int i = 0; i < H; ++i) st[(long)i * C] = keep[i];
}

// Workgroup = 4 waves = 64 values of p for one (segment, head); in a wave lanes are (p % 16,
// chunk = lane / 16): chunk k holds states n in [k * NPT, (k + 1) * NPT) of its p in registers, and
// the 4 partial sums of y meet through two xor-shuffles.
template <typename T, int NPT>
__global__ __launch_bounds__(256) void ssm_scan_kernel(float* __restrict__ y, const T* __restrict__ xbc,
                                                       const T* __restrict__ proj, long p_stride, int dt_col,
                                                       const float* __restrict__ dt_bias,
                                                       const float* __restrict__ a_log,
                                                       const float* __restrict__ d_skip, float* __restrict__ state,
                                                       const int* __restrict__ cu, const int* __restrict__ ctx,
                                                       const int* __restrict__ slot, int nh, int P, int N, int G) {
  const int s = blockIdx.x, h = blockIdx.y;
  const int sl = slot[s];
  const int t0 = cu[s], t1 = cu[s + 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int p = blockIdx.z * 64 + wave * 16 + (lane & 15);
  if (sl < 0) {  // padding rows: defined output, no state
    if (p < P && lane < 16)
      for (int t = t0; t < t1; ++t) y[(long)t * nh * P + (long)h * P + p] = 0.f;
    return;
  }
  if (t1 <= t0) return;
  const int n0 = (lane >> 4) * NPT;
  const bool live = p < P;
  const int g = h / (nh / G);
  const int inner = nh * P, C = inner + 2 * G * N;
  float S[NPT];
  float* sp = state + (((long)sl * nh + h) * N) * P + p;
  const bool carried = ctx[s] > 0;
#pragma unroll
  for (int i = 0; i < NPT; ++i) S[i] = (carried && live && n0 + i < N) ? sp[(long)(n0 + i) * P] : 0.f;
  const float A = expf(a_log[h]), Dh = d_skip[h], bias = dt_bias[h];
  for (int t = t0; t < t1; ++t) {
    const T* row = xbc + (long)t * C;
    const float raw = ldf(proj + (long)t * p_stride + dt_col + h) + bias;
    const float dt = raw > 20.f ? raw : log1pf(expf(raw));
    const float dA = expf(-A * dt);
    const float x = live ? ldf(row + (long)h * P + p) : 0.f;
    const T* Bp = row + inner + (long)g * N + n0;
    const T* Cp = Bp + (long)G * N;
    const float dtx = dt * x;
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
      if (n0 + i < N) {
        S[i] = dA * S[i] + dtx * ldf(Bp + i);
        acc += S[i] * ldf(Cp + i);
      }
    }
    acc += __shfl_xor(acc, 16, 64);
    acc += __shfl_xor(acc, 32, 64);
    if (live && lane < 16) y[(long)t * inner + (long)h * P + p] = acc + Dh * x;
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < NPT; ++i)
      if (n0 + i < N) sp[(long)(n0 + i) * P] = S[i];
  }
}

}  // namespace k8sllm

using namespace k8sllm;

template <typename T>
static int launch_scan(float* y, const void* xbc, const void* proj, long p_stride, int dt_col, const float* dt_bias,
                       const float* a_log, const float* d_skip, float* state, const int* cu, const int* ctx,
                       const int* slot, int S, int nh, int P, int N, int G, hipStream_t s) {
  const dim3 grid((unsigned)S, (unsigned)nh, (unsigned)((P + 63) / 64));
#define K8SLLM_SCAN(NPT)                                                                                              \
  hipLaunchKernelGGL((ssm_scan_kernel<T, NPT>), grid, dim3(256), 0, s, y, (const T*)xbc, (const T*)proj, p_stride,    \
                     dt_col, dt_bias, a_log, d_skip, state, cu, ctx, slot, nh, P, N, G)
  if (N <= 16) K8SLLM_SCAN(4);
  else if (N <= 32) K8SLLM_SCAN(8);
  else if (N <= 64) K8SLLM_SCAN(16);
  else if (N <= 128) K8SLLM_SCAN(32);
  else if (N <= 256) K8SLLM_SCAN(64);
  else return -1;
#undef K8SLLM_SCAN
  return (int)hipGetLastError();
}

extern "C" {

int k8sllm_hy_conv_silu(void* out, const void* proj, long stride, int col0, int C, const float* cw, const float* cb,
                        int taps, void* state, const int* cu, const int* ctx, const int* slot, int S, long T, int f32,
                        hipStream_t s) {
  if (T <= 0 || S <= 0) return 0;
  if (taps < 1 || taps > kMaxTaps) return -1;
  const dim3 g1((unsigned)T, (unsigned)((C + 255) / 256)), g2((unsigned)S, (unsigned)((C + 255) / 256));
  if (f32) {
    hipLaunchKernelGGL(conv_silu_kernel<float>, g1, dim3(256), 0, s, (float*)out, (const float*)proj, stride, col0, C,
                       cw, cb, taps, (const float*)state, cu, ctx, slot, S);
    if (taps > 1)
      hipLaunchKernelGGL(conv_state_step_kernel<float>, g2, dim3(256), 0, s, (float*)state, (const float*)proj, stride,
                         col0, C, taps, cu, ctx, slot);
  } else {
    hipLaunchKernelGGL(conv_silu_kernel<bf16_t>, g1, dim3(256), 0, s, (bf16_t*)out, (const bf16_t*)proj, stride, col0,
                       C, cw, cb, taps, (const bf16_t*)state, cu, ctx, slot, S);
    if (taps > 1)
      hipLaunchKernelGGL(conv_state_step_kernel<bf16_t>, g2, dim3(256), 0, s, (bf16_t*)state, (const bf16_t*)proj,
                         stride, col0, C, taps, cu, ctx, slot);
  }
  return (int)hipGetLastError();
}

int k8sllm_hy_ssm_scan(float* y, const void* xbc, const void* proj, long p_stride, int dt_col, const float* dt_bias,
                       const float* a_log, const float* d_skip, float* state, const int* cu, const int* ctx,
                       const int* slot, int S, int nh, int P, int N, int G, int f32, hipStream_t s) {
  if (S <= 0) return 0;
  if (G < 1 || nh % G) return -1;
  return f32 ? launch_scan<float>(y, xbc, proj, p_stride, dt_col, dt_bias, a_log, d_skip, state, cu, ctx, slot, S, nh,
                                  P, N, G, s)
             : launch_scan<bf16_t>(y, xbc, proj, p_stride, dt_col, dt_bias, a_log, d_skip, state, cu, ctx, slot, S,
                                   nh, P, N, G, s);
}
}
