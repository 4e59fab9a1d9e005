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
// The columns of S evolve independently, and so do the rows once S^T k and S^T q are reduced
// over them: a column is owned by a group of 8 or 16 adjacent lanes, lane r of the group holding
// rows LPC j + r in registers for the whole portion, so each dot product is a private loop over
// DP / LPC rows plus a DPP exchange inside the group (no LDS on the serial chain).  A workgroup
// is LPC waves = 64 columns of one (sequence, head), so every SIMD holds several waves of the
// chain; k, q, g and beta of kTB tokens at a time are prepared by the waves (wave w takes tokens
// w, w + LPC, ...; lane i normalises channel i) and broadcast through LDS in a
// [group lane][row] layout that each lane reads with 16-byte loads.  The raw inputs of the
// next round are fetched into registers while the current round runs, so the serial chain over
// tokens never waits on memory.  State I/O is coalesced along vdim.
// DP is the key width padded to a multiple of 32 (padding rows stay zero).
#include "mix_common.h"
#include "mixers.h"

namespace mixk {

constexpr int kTB = 16;           // tokens staged per round
// lanes per column of S = waves per workgroup (64 columns x lanes): 16 where the padded key
// width splits into 16-byte groups per lane, else 8
constexpr int lanes_per_column(int dp) { return dp % 64 == 0 ? 16 : 8; }

typedef __attribute__((ext_vector_type(4))) float f32x4_t;

template <typename T, int DP, bool CH>
__global__ void __launch_bounds__(64 * lanes_per_column(DP))
gated_delta_rule_kernel(float* __restrict__ out, const T* __restrict__ qkv,
                        const T* __restrict__ beta, int64_t beta_stride,
                        const T* __restrict__ decay, int64_t decay_stride,
                        const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                        float* __restrict__ state, const int* __restrict__ positions,
                        const int* __restrict__ seq_qstart, const int* __restrict__ seq_slot,
                        int H, int G, int dim, int vdim) {
  constexpr int kLPC = lanes_per_column(DP), kWaves = kLPC;
  constexpr int kTPW = kTB / kWaves;   // tokens each wave prepares per round
  constexpr int R = DP / kLPC;     // rows per lane
  constexpr int RS = R + 4;        // LDS stride between the group lanes' row lists (bank spread)
  constexpr int NJ = (DP + kWave - 1) / kWave;   // channels per lane when staging
  __shared__ __attribute__((aligned(16))) float sk[kTB][kLPC * RS];
  __shared__ __attribute__((aligned(16))) float sq[kTB][kLPC * RS];
  __shared__ __attribute__((aligned(16))) float sg[kTB][CH ? kLPC * RS : 4];
  __shared__ float sbeta[kTB];
  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int slot = seq_slot[s];
  const int first = seq_qstart[s], n = seq_qstart[s + 1] - first;
  if (slot < 0 || n <= 0) return;
  const int lane = tid & 63, w = tid >> 6, r4 = tid & (kLPC - 1);
  const int col = blockIdx.z * 64 + (tid / kLPC);
  const bool active = col < vdim;
  const int kvh = h / (H / G);
  const int C = 2 * G * dim + H * vdim;          // row width of qkv
  const int q_off = kvh * dim, k_off = G * dim + kvh * dim, v_off = 2 * G * dim + h * vdim;
  float* st = state + (static_cast<int64_t>(slot) * H + h) * dim * vdim;
  float S[R];
  const bool fresh = positions[first] == 0;
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const int i = kLPC * j + r4;
    S[j] = (!fresh && active && i < dim) ? st[static_cast<int64_t>(i) * vdim + col] : 0.f;
  }
  const float rate = expf(a_log[h]);
  const float qscale = 1.0f / sqrtf(static_cast<float>(dim));
  float rk[kTPW][NJ], rq[kTPW][NJ], rd[kTPW][CH ? NJ : 1], rb[kTPW], rv[kTB];
  auto load_round = [&](int t0) {
#pragma unroll
    for (int u = 0; u < kTPW; ++u) {
      const int tt = w + kWaves * u;
      const bool ok = t0 + tt < n;
      const int64_t row = first + t0 + (ok ? tt : 0);
      const T* xr = qkv + row * C;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int i = lane + j * kWave;
        const bool in = ok && i < dim;
        rk[u][j] = in ? ldf(xr + k_off + i) : 0.f;
        rq[u][j] = in ? ldf(xr + q_off + i) : 0.f;
        if (CH) rd[u][j] = in ? ldf(decay + row * decay_stride + h * dim + i) : 0.f;
      }
      if (!CH) rd[u][0] = ok ? ldf(decay + row * decay_stride + h) : 0.f;
      rb[u] = ok ? ldf(beta + row * beta_stride + h) : 0.f;
    }
#pragma unroll
    for (int tt = 0; tt < kTB; ++tt) {
      const bool ok = t0 + tt < n && active;
      rv[tt] = ok ? ldf(qkv + (first + t0 + tt) * static_cast<int64_t>(C) + v_off + col) : 0.f;
    }
  };
  float bias[CH ? NJ : 1];
  if (CH) {
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int i = lane + j * kWave;
      bias[j] = i < dim ? dt_bias[h * dim + i] : 0.f;
    }
  } else {
    bias[0] = dt_bias[h];
  }
  load_round(0);
  for (int t0 = 0; t0 < n; t0 += kTB) {
    const int nt = min(kTB, n - t0);
    float v[kTB];
    __syncthreads();   // the previous round's LDS reads are done
#pragma unroll
    for (int u = 0; u < kTPW; ++u) {
      const int tt = w + kWaves * u;
      float kss = 0.f, qss = 0.f;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        kss += rk[u][j] * rk[u][j];
        qss += rq[u][j] * rq[u][j];
      }
      kss = wave_sum(kss);
      qss = wave_sum(qss);
      const float kinv = 1.0f / sqrtf(kss + 1e-6f);
      const float qinv = qscale / sqrtf(qss + 1e-6f);
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int i = lane + j * kWave;
        if (i < DP) {
          const int at = (i % kLPC) * RS + i / kLPC;   // channel i lives with group lane i % kLPC
          sk[tt][at] = rk[u][j] * kinv;
          sq[tt][at] = rq[u][j] * qinv;
          if (CH) sg[tt][at] = i < dim ? expf(-rate * softplusf_(rd[u][j] + bias[j])) : 1.f;
        }
      }
      if (lane == 0) {
        sbeta[tt] = sigmoidf_(rb[u]);
        if (!CH) sg[tt][0] = expf(-rate * softplusf_(rd[u][0] + bias[0]));
      }
    }
#pragma unroll
    for (int tt = 0; tt < kTB; ++tt) v[tt] = rv[tt];
    __syncthreads();
    if (t0 + kTB < n) load_round(t0 + kTB);   // in flight during the recurrence below
#pragma unroll
    for (int tt = 0; tt < kTB; ++tt) {
      if (tt >= nt) break;
      const int64_t row = first + t0 + tt;
      const float b = sbeta[tt];
      const f32x4_t* kp = reinterpret_cast<const f32x4_t*>(&sk[tt][r4 * RS]);
      const f32x4_t* qp = reinterpret_cast<const f32x4_t*>(&sq[tt][r4 * RS]);
      float dot = 0.f;
      f32x4_t kreg[R / 4];
      if (CH) {
        const f32x4_t* gp = reinterpret_cast<const f32x4_t*>(&sg[tt][r4 * RS]);
#pragma unroll
        for (int j4 = 0; j4 < R / 4; ++j4) {
          const f32x4_t g = gp[j4];
          kreg[j4] = kp[j4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            S[4 * j4 + e] *= g[e];
            dot += S[4 * j4 + e] * kreg[j4][e];
          }
        }
      } else {
        const float g = sg[tt][0];
#pragma unroll
        for (int j4 = 0; j4 < R / 4; ++j4) {
          kreg[j4] = kp[j4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            S[4 * j4 + e] *= g;
            dot += S[4 * j4 + e] * kreg[j4][e];
          }
        }
      }
      dot = group_sum<kLPC>(dot);
      const float u = b * (v[tt] - dot);
      float o = 0.f;
#pragma unroll
      for (int j4 = 0; j4 < R / 4; ++j4) {
        const f32x4_t qv = qp[j4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          S[4 * j4 + e] += kreg[j4][e] * u;
          o += S[4 * j4 + e] * qv[e];
        }
      }
      o = group_sum<kLPC>(o);
      if (active && r4 == 0) out[(row * H + h) * vdim + col] = o;
    }
  }
  if (active) {
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int i = kLPC * j + r4;
      if (i < dim) st[static_cast<int64_t>(i) * vdim + col] = S[j];
    }
  }
}

template <typename T, int DP>
int launch_dp(float* out, const void* qkv, const void* beta, int64_t beta_stride,
              const void* decay, int64_t decay_stride, int per_channel, const float* a_log,
              const float* dt_bias, float* state, const int* positions, const int* seq_qstart,
              const int* seq_slot, int S, int H, int G, int dim, int vdim, hipStream_t st) {
  const dim3 grid(S, H, (vdim + 63) / 64);
  if (per_channel)
    hipLaunchKernelGGL((gated_delta_rule_kernel<T, DP, true>), grid, dim3(64 * lanes_per_column(DP)), 0, st, out,
                       static_cast<const T*>(qkv), static_cast<const T*>(beta), beta_stride,
                       static_cast<const T*>(decay), decay_stride, a_log, dt_bias, state,
                       positions, seq_qstart, seq_slot, H, G, dim, vdim);
  else
    hipLaunchKernelGGL((gated_delta_rule_kernel<T, DP, false>), grid, dim3(64 * lanes_per_column(DP)), 0, st, out,
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
