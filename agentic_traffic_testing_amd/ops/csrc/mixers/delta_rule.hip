// Gated delta rule over ragged batches of portions, state carried per sequence in fp32.
//
// Per head, with S [dim, vdim] the state, per token:
//     S = diag(g) S            (g: one decay per head, or one per key channel)
//     u = beta (v - S^T k)
//     S = S + k u^T
//     o = S^T q
// with k = k_raw / sqrt(|k_raw|^2 + 1e-6), q likewise times dim^-1/2, beta = sigmoid(b) and
// g = exp(-exp(a_log) * softplus(a + dt_bias)); all of it in fp32.
//
// The columns of S evolve independently, so one lane owns one column: its dim entries stay in
// registers for the whole portion and both dot products are private to the lane - no
// cross-lane traffic in the recurrence.  A workgroup is one wave = 64 columns of one
// (sequence, head); k, q, g and beta of TB tokens at a time are prepared cooperatively (lane i
// normalises channel i) and broadcast through LDS.  State I/O is coalesced along vdim.
// DP is the key width padded to a multiple of 32 (padding rows stay zero).
#include "mix_common.h"
#include "mixers.h"

namespace mixk {

constexpr int kTB = 8;  // tokens staged per round

template <typename T, int DP, bool CH>
__global__ void __launch_bounds__(64)
gated_delta_rule_kernel(float* __restrict__ out, const T* __restrict__ qkv,
                        const T* __restrict__ beta, int64_t beta_stride,
                        const T* __restrict__ decay, int64_t decay_stride,
                        const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                        float* __restrict__ state, const int* __restrict__ positions,
                        const int* __restrict__ seq_qstart, const int* __restrict__ seq_slot,
                        int H, int G, int dim, int vdim) {
  __shared__ __attribute__((aligned(16))) float sk[kTB][DP];
  __shared__ __attribute__((aligned(16))) float sq[kTB][DP];
  __shared__ __attribute__((aligned(16))) float sg[kTB][CH ? DP : 4];
  __shared__ float sbeta[kTB];
  const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int slot = seq_slot[s];
  const int first = seq_qstart[s], n = seq_qstart[s + 1] - first;
  if (slot < 0 || n <= 0) return;
  const int col = blockIdx.z * kWave + lane;
  const bool active = col < vdim;
  const int kvh = h / (H / G);
  const int C = 2 * G * dim + H * vdim;          // row width of qkv
  const int q_off = kvh * dim, k_off = G * dim + kvh * dim, v_off = 2 * G * dim + h * vdim;
  float* st = state + (static_cast<int64_t>(slot) * H + h) * dim * vdim;
  float S[DP];
  const bool fresh = positions[first] == 0;
#pragma unroll
  for (int i = 0; i < DP; ++i)
    S[i] = (!fresh && active && i < dim) ? st[static_cast<int64_t>(i) * vdim + col] : 0.f;
  const float rate = expf(a_log[h]);
  const float qscale = 1.0f / sqrtf(static_cast<float>(dim));
  for (int t0 = 0; t0 < n; t0 += kTB) {
    const int nt = min(kTB, n - t0);
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const int64_t row = first + t0 + tt;
      const T* xr = qkv + row * C;
      float kv[DP / kWave + 1], qv[DP / kWave + 1];
      float kss = 0.f, qss = 0.f;
#pragma unroll
      for (int j = 0; j < DP / kWave + 1; ++j) {
        const int i = lane + j * kWave;
        kv[j] = qv[j] = 0.f;
        if (i < dim) {
          kv[j] = ldf(xr + k_off + i);
          qv[j] = ldf(xr + q_off + i);
        }
        kss += kv[j] * kv[j];
        qss += qv[j] * qv[j];
      }
      kss = wave_sum(kss);
      qss = wave_sum(qss);
      const float kinv = 1.0f / sqrtf(kss + 1e-6f);
      const float qinv = qscale / sqrtf(qss + 1e-6f);
#pragma unroll
      for (int j = 0; j < DP / kWave + 1; ++j) {
        const int i = lane + j * kWave;
        if (i < DP) {
          sk[tt][i] = kv[j] * kinv;
          sq[tt][i] = qv[j] * qinv;
          if (CH) {
            float gv = 1.f;
            if (i < dim)
              gv = expf(-rate * softplusf_(ldf(decay + row * decay_stride + h * dim + i) +
                                           dt_bias[h * dim + i]));
            sg[tt][i] = gv;
          }
        }
      }
      if (lane == 0) {
        sbeta[tt] = sigmoidf_(ldf(beta + row * beta_stride + h));
        if (!CH) sg[tt][0] = expf(-rate * softplusf_(ldf(decay + row * decay_stride + h) +
                                                     dt_bias[h]));
      }
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const int64_t row = first + t0 + tt;
      const float v = active ? ldf(qkv + row * C + v_off + col) : 0.f;
      const float b = sbeta[tt];
      float dot = 0.f;
      if (CH) {
#pragma unroll
        for (int i = 0; i < DP; ++i) {
          S[i] *= sg[tt][i];
          dot += S[i] * sk[tt][i];
        }
      } else {
        const float g = sg[tt][0];
#pragma unroll
        for (int i = 0; i < DP; ++i) {
          S[i] *= g;
          dot += S[i] * sk[tt][i];
        }
      }
      const float u = b * (v - dot);
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < DP; ++i) {
        S[i] += sk[tt][i] * u;
        o += S[i] * sq[tt][i];
      }
      if (active) out[(row * H + h) * vdim + col] = o;
    }
  }
  if (active) {
#pragma unroll
    for (int i = 0; i < DP; ++i)
      if (i < dim) st[static_cast<int64_t>(i) * vdim + col] = S[i];
  }
}

template <typename T, int DP>
int launch_dp(float* out, const void* qkv, const void* beta, int64_t beta_stride,
              const void* decay, int64_t decay_stride, int per_channel, const float* a_log,
              const float* dt_bias, float* state, const int* positions, const int* seq_qstart,
              const int* seq_slot, int S, int H, int G, int dim, int vdim, hipStream_t st) {
  const dim3 grid(S, H, (vdim + kWave - 1) / kWave);
  if (per_channel)
    hipLaunchKernelGGL((gated_delta_rule_kernel<T, DP, true>), grid, dim3(kWave), 0, st, out,
                       static_cast<const T*>(qkv), static_cast<const T*>(beta), beta_stride,
                       static_cast<const T*>(decay), decay_stride, a_log, dt_bias, state,
                       positions, seq_qstart, seq_slot, H, G, dim, vdim);
  else
    hipLaunchKernelGGL((gated_delta_rule_kernel<T, DP, false>), grid, dim3(kWave), 0, st, out,
                       static_cast<const T*>(qkv), static_cast<const T*>(beta), beta_stride,
                       static_cast<const T*>(decay), decay_stride, a_log, dt_bias, state,
                       positions, seq_qstart, seq_slot, H, G, dim, vdim);
  return static_cast<int>(hipGetLastError());
}

template <typename T>
int launch_t(float* out, const void* qkv, const void* beta, int64_t beta_stride,
             const void* decay, int64_t decay_stride, int per_channel, const float* a_log,
             const float* dt_bias, float* state, const int* positions, const int* seq_qstart,
             const int* seq_slot, int S, int H, int G, int dim, int vdim, hipStream_t st) {
#define MIXK_DP(N)                                                                              \
  if (dim <= N)                                                                                 \
    return launch_dp<T, N>(out, qkv, beta, beta_stride, decay, decay_stride, per_channel, a_log, \
                           dt_bias, state, positions, seq_qstart, seq_slot, S, H, G, dim, vdim, st)
  MIXK_DP(32);
  MIXK_DP(64);
  MIXK_DP(96);
  MIXK_DP(128);
  MIXK_DP(192);
  MIXK_DP(256);
#undef MIXK_DP
  return -1;
}

}  // namespace mixk

using namespace mixk;

extern "C" int mixk_gated_delta_rule(float* out, const void* qkv, const void* beta,
                                     int64_t beta_stride, const void* decay, int64_t decay_stride,
                                     int per_channel, const float* a_log, const float* dt_bias,
                                     float* state, const int* positions, const int* seq_qstart,
                                     const int* seq_slot, int S, int H, int G, int dim, int vdim,
                                     int dtype, hipStream_t st) {
  if (S <= 0) return 0;
  if (H % G != 0) return -1;
  int rc = 0;
  MIXK_DISPATCH(dtype, rc = launch_t<T>(out, qkv, beta, beta_stride, decay, decay_stride,
                                        per_channel, a_log, dt_bias, state, positions, seq_qstart,
                                        seq_slot, S, H, G, dim, vdim, st));
  return rc;
}
