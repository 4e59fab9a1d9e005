// Gated linear recurrence over ragged batches of portions, state carried per sequence in fp32.
//
// Per head, with S [dk, dv] the state, per token:
//     S[i, :] = a[i] S[i, :] + k[i] v[:]        o[:] = sum_i q[i] S[i, :]  (+ skip * v[:])
// Two front ends produce (a, k, q) of a token from the raw projections, all in fp32:
//   * forget-gate form (HGRN2):  a = l + (1 - l) sigmoid(f + f_bias), k = 1 - a, q = silu(q_raw);
//     one gate per head and key channel, `l` a per-channel lower bound.
//   * state-space form (Mamba-2): dt = softplus(dt_raw + dt_bias), a = exp(-exp(A_log) dt) for the
//     whole head, k = dt B, q = C, skip = D; B and C are shared by the heads of a group.
//
// The columns of S evolve independently: a column is owned by 8 adjacent lanes, lane r holding
// rows r R ... r R + R - 1 in registers for the whole portion, so a token costs R multiply-adds
// per lane for the update, R for the read-out and one DPP sum over the 8 lanes.  A workgroup is
// 4 waves = 32 columns of one (sequence, head); (a, k, q) of kTB tokens at a time are prepared
// by all threads and broadcast through LDS in a [group lane][row] layout read with 16-byte loads.
// A portion whose first position is 0 starts from the zero state whatever its slot holds.
#include "mix_common.h"
#include "mixers.h"

namespace mixk {

constexpr int kScanLPC = 8;     // lanes per column
constexpr int kScanCols = 32;   // columns per workgroup
constexpr int kScanThreads = kScanLPC * kScanCols;

struct ScanArgs {
  float* out;             // [T, H, dv]
  float* state;           // [slots, H, dk, dv]
  const void* q;          // forget-gate: q_raw [T, H dk]; state-space: C [T, G dk]
  const void* k;          // forget-gate: f [T, H dk];     state-space: B [T, G dk]
  const void* v;          // [T, H dv]
  const void* dt;         // state-space: dt_raw [T, H]
  const float* p0;        // forget-gate: f_bias [H dk];   state-space: dt_bias [H]
  const float* p1;        // forget-gate: lower [H dk];    state-space: A_log [H]
  const float* p2;        // state-space: D [H]
  const int* positions;
  const int* seq_qstart;
  const int* seq_slot;
  int64_t q_stride, k_stride, v_stride, dt_stride;
  int H, G, dk, dv;
};

// MODE 0: forget-gate form, MODE 1: state-space form.  R: rows per lane (dk <= 8 R).
template <typename T, int R, int MODE>
__global__ void __launch_bounds__(kScanThreads)
gated_linear_scan_kernel(ScanArgs a) {
  constexpr int kTB = R >= 24 ? 8 : 16;            // tokens staged per round
  constexpr int RS = (R + 3) / 4 * 4 + 4;          // LDS stride between the group lanes' rows
  constexpr int DKP = kScanLPC * R;
  __shared__ __attribute__((aligned(16))) float sk[kTB][kScanLPC * RS];
  __shared__ __attribute__((aligned(16))) float sq[kTB][kScanLPC * RS];
  __shared__ __attribute__((aligned(16))) float sa[MODE == 0 ? kTB : 1][MODE == 0 ? kScanLPC * RS : 4];
  __shared__ float sdec[kTB];
  __shared__ float sv[kTB][kScanCols];
  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int slot = a.seq_slot[s];
  const int first = a.seq_qstart[s], n = a.seq_qstart[s + 1] - first;
  if (slot < 0 || n <= 0) return;
  const int H = a.H, dk = a.dk, dv = a.dv;
  const int r = tid & (kScanLPC - 1), cl = tid >> 3;
  const int col = blockIdx.z * kScanCols + cl;
  const bool active = col < dv;
  const int g = MODE == 0 ? h : h / (H / a.G);
  const T* qp = static_cast<const T*>(a.q);
  const T* kp = static_cast<const T*>(a.k);
  const T* vp = static_cast<const T*>(a.v);
  const T* dtp = static_cast<const T*>(a.dt);
  float* st = a.state + (static_cast<int64_t>(slot) * H + h) * dk * dv;
  float S[R];
  const bool fresh = a.positions[first] == 0;
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const int i = r * R + j;
    S[j] = (!fresh && active && i < dk) ? st[static_cast<int64_t>(i) * dv + col] : 0.f;
  }
  // padding rows (dk < 8 R) stay zero in every staged array
  for (int i = tid; i < kTB * kScanLPC * RS; i += kScanThreads) {
    (&sk[0][0])[i] = 0.f;
    (&sq[0][0])[i] = 0.f;
    if (MODE == 0) (&sa[0][0])[i] = 0.f;
  }
  float rate = 0.f, dtb = 0.f, skip = 0.f;
  if (MODE == 1) {
    rate = expf(a.p1[h]);
    dtb = a.p0[h];
    skip = a.p2[h];
  }
  for (int t0 = 0; t0 < n; t0 += kTB) {
    const int nt = min(kTB, n - t0);
    __syncthreads();   // the previous round's LDS reads (and the zero fill) are done
    for (int e = tid; e < nt * dk; e += kScanThreads) {
      const int tt = e / dk, i = e - tt * dk;
      const int64_t row = first + t0 + tt;
      const int at = (i / R) * RS + i % R;
      if (MODE == 0) {
        const int ch = h * dk + i;
        const float lo = a.p1[ch];
        const float f = lo + (1.0f - lo) * sigmoidf_(ldf(kp + row * a.k_stride + ch) + a.p0[ch]);
        sa[tt][at] = f;
        sk[tt][at] = 1.0f - f;
        sq[tt][at] = siluf_(ldf(qp + row * a.q_stride + ch));
      } else {
        const float dt = softplusf_(ldf(dtp + row * a.dt_stride + h) + dtb);
        sk[tt][at] = dt * ldf(kp + row * a.k_stride + g * dk + i);
        sq[tt][at] = ldf(qp + row * a.q_stride + g * dk + i);
      }
    }
    if (MODE == 1 && tid < nt) {
      const float dt = softplusf_(ldf(dtp + (first + t0 + tid) * a.dt_stride + h) + dtb);
      sdec[tid] = expf(-rate * dt);
    }
    for (int e = tid; e < nt * kScanCols; e += kScanThreads) {
      const int tt = e / kScanCols, c = e - tt * kScanCols;
      const int cc = blockIdx.z * kScanCols + c;
      sv[tt][c] = cc < dv ? ldf(vp + (first + t0 + tt) * a.v_stride + h * dv + cc) : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float vv = sv[tt][cl];
      const float* pk = &sk[tt][r * RS];
      const float* pq = &sq[tt][r * RS];
      float o = 0.f;
      if (MODE == 0) {
        const float* pa = &sa[tt][r * RS];
#pragma unroll
        for (int j = 0; j < R; ++j) {
          S[j] = pa[j] * S[j] + pk[j] * vv;
          o += pq[j] * S[j];
        }
      } else {
        const float dec = sdec[tt];
#pragma unroll
        for (int j = 0; j < R; ++j) {
          S[j] = dec * S[j] + pk[j] * vv;
          o += pq[j] * S[j];
        }
      }
      o = group_sum<kScanLPC>(o);
      if (active && r == 0)
        a.out[(static_cast<int64_t>(first + t0 + tt) * H + h) * dv + col] = o + skip * vv;
    }
  }
  if (active) {
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int i = r * R + j;
      if (i < dk) st[static_cast<int64_t>(i) * dv + col] = S[j];
    }
  }
  (void)DKP;
}

template <typename T, int MODE>
int launch_scan(const ScanArgs& a, int S, hipStream_t st) {
  const dim3 grid(S, a.H, (a.dv + kScanCols - 1) / kScanCols);
#define MIXK_SCAN_R(N)                                                                      \
  if (a.dk <= kScanLPC * N) {                                                               \
    hipLaunchKernelGGL((gated_linear_scan_kernel<T, N, MODE>), grid, dim3(kScanThreads), 0, \
                       st, a);                                                              \
    return static_cast<int>(hipGetLastError());                                             \
  }
  MIXK_SCAN_R(2)
  MIXK_SCAN_R(4)
  MIXK_SCAN_R(6)
  MIXK_SCAN_R(8)
  MIXK_SCAN_R(12)
  MIXK_SCAN_R(16)
  MIXK_SCAN_R(24)
  MIXK_SCAN_R(32)
#undef MIXK_SCAN_R
  return -1;
}

}  // namespace mixk

using namespace mixk;

// mode 0: forget-gate form (q = q_raw, k = f, p0 = f_bias, p1 = lower; G ignored);
// mode 1: state-space form (q = C, k = B, dt, p0 = dt_bias, p1 = A_log, p2 = D; H % G == 0).
extern "C" int mixk_gated_linear_scan(float* out, float* state, const void* q, int64_t q_stride,
                                      const void* k, int64_t k_stride, const void* v,
                                      int64_t v_stride, const void* dt, int64_t dt_stride,
                                      const float* p0, const float* p1, const float* p2,
                                      const int* positions, const int* seq_qstart,
                                      const int* seq_slot, int S, int H, int G, int dk, int dv,
                                      int mode, int dtype, hipStream_t st) {
  if (S <= 0) return 0;
  if (dk <= 0 || dv <= 0 || H <= 0) return -1;
  if (mode == 1 && (G <= 0 || H % G != 0)) return -1;
  ScanArgs a{out, state, q, k, v, dt, p0, p1, p2, positions, seq_qstart, seq_slot,
             q_stride, k_stride, v_stride, dt_stride, H, mode == 1 ? G : H, dk, dv};
  int rc = 0;
  if (mode == 0)
    MIXK_DISPATCH(dtype, rc = (launch_scan<T, 0>(a, S, st)));
  else
    MIXK_DISPATCH(dtype, rc = (launch_scan<T, 1>(a, S, st)));
  return rc;
}
