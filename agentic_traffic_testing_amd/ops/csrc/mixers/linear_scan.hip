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
// by all threads and broadcast through LDS in a [group lane][row] layout read with 16-byte loads;
// the raw inputs of the next round are fetched into registers while the current round runs, so
// the serial chain over tokens does not wait on memory.
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

// MODE 0: forget-gate form, MODE 1: state-space form.  R: rows per lane (dk <= 8 R).  CPL: columns
// per lane (a workgroup covers 32 CPL columns).  Only CPL = 1 is instantiated: two columns per
// lane halve the LDS reads per multiply-add, but the loop is bound by VALU issue (three fp32
// operations per state element and token), so they measured no faster (1.74 vs 1.69 ms for 4 x
// 2048 tokens of 32 heads of 128 x 128).
template <typename T, int R, int MODE, int CPL>
__global__ void __launch_bounds__(kScanThreads)
gated_linear_scan_kernel(ScanArgs a) {
  constexpr int kTB = R >= 24 ? 8 : 16;            // tokens staged per round
  constexpr int RS = (R + 3) / 4 * 4 + 4;          // LDS stride between the group lanes' rows
  constexpr int DKP = kScanLPC * R;                // padded key width
  constexpr int NE = kTB * DKP / kScanThreads;     // (token, channel) entries per thread and round
  constexpr int BC = kScanCols * CPL;              // columns per workgroup
  constexpr int NV = kTB * BC / kScanThreads;
  static_assert(NE * kScanThreads == kTB * DKP && NV * kScanThreads == kTB * BC, "staging");
  __shared__ __attribute__((aligned(16))) float sk[kTB][kScanLPC * RS];
  __shared__ __attribute__((aligned(16))) float sq[kTB][kScanLPC * RS];
  __shared__ __attribute__((aligned(16))) float sa[MODE == 0 ? kTB : 1][MODE == 0 ? kScanLPC * RS : 4];
  __shared__ float sp0[MODE == 0 ? DKP : 1], sp1[MODE == 0 ? DKP : 1];
  __shared__ float sdec[kTB], sdt[kTB];
  __shared__ float sv[kTB][BC];
  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int slot = a.seq_slot[s];
  const int first = a.seq_qstart[s], n = a.seq_qstart[s + 1] - first;
  if (slot < 0 || n <= 0) return;
  const int H = a.H, dk = a.dk, dv = a.dv;
  const int r = tid & (kScanLPC - 1), cl = tid >> 3;
  const int col0 = blockIdx.z * BC + cl;           // this lane's columns: col0 + 32 c

  const int g = MODE == 0 ? h : h / (H / a.G);
  const T* qp = static_cast<const T*>(a.q) + static_cast<int64_t>(g) * dk;
  const T* kp = static_cast<const T*>(a.k) + static_cast<int64_t>(g) * dk;
  const T* vp = static_cast<const T*>(a.v) + static_cast<int64_t>(h) * dv + blockIdx.z * BC;
  const T* dtp = static_cast<const T*>(a.dt);
  float* st = a.state + (static_cast<int64_t>(slot) * H + h) * dk * dv;
  float S[CPL][R];
  const bool fresh = a.positions[first] == 0;
#pragma unroll
  for (int c = 0; c < CPL; ++c)
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int i = r * R + j, col = col0 + kScanCols * c;
      S[c][j] = (!fresh && col < dv && i < dk) ? st[static_cast<int64_t>(i) * dv + col] : 0.f;
    }
  // padding rows (dk < 8 R) stay zero in every staged array
  for (int i = tid; i < kTB * kScanLPC * RS; i += kScanThreads) {
    (&sk[0][0])[i] = 0.f;
    (&sq[0][0])[i] = 0.f;
    if (MODE == 0) (&sa[0][0])[i] = 0.f;
  }
  float rate = 0.f, dtb = 0.f, skip = 0.f;
  if (MODE == 0) {
    for (int i = tid; i < dk; i += kScanThreads) {
      sp0[i] = a.p0[h * dk + i];
      sp1[i] = a.p1[h * dk + i];
    }
  } else {
    rate = expf(a.p1[h]);
    dtb = a.p0[h];
    skip = a.p2[h];
  }
  // raw inputs of a round, fetched into registers one round ahead of their use
  float rq[NE], rk[NE], rv[NV], rdt = 0.f;
  auto load_round = [&](int t0) {
#pragma unroll
    for (int m = 0; m < NE; ++m) {
      const int e = tid + m * kScanThreads;
      const int tt = e / DKP, i = e % DKP;
      const bool ok = t0 + tt < n && i < dk;
      const int64_t row = first + t0 + (ok ? tt : 0);
      rq[m] = ok ? ldf(qp + row * a.q_stride + i) : 0.f;
      rk[m] = ok ? ldf(kp + row * a.k_stride + i) : 0.f;
    }
#pragma unroll
    for (int m = 0; m < NV; ++m) {
      const int e = tid + m * kScanThreads;
      const int tt = e / BC, c = e % BC;
      const bool ok = t0 + tt < n && blockIdx.z * BC + c < dv;
      rv[m] = ok ? ldf(vp + (first + t0 + tt) * a.v_stride + c) : 0.f;
    }
    if (MODE == 1 && tid < kTB && t0 + tid < n)
      rdt = ldf(dtp + (first + t0 + tid) * a.dt_stride + h);
  };
  load_round(0);
  for (int t0 = 0; t0 < n; t0 += kTB) {
    const int nt = min(kTB, n - t0);
    __syncthreads();   // the previous round's LDS reads (and the fills above) are done
    if (MODE == 1) {
      if (tid < nt) {
        const float dt = softplusf_(rdt + dtb);
        sdt[tid] = dt;
        sdec[tid] = expf(-rate * dt);
      }
      __syncthreads();
    }
#pragma unroll
    for (int m = 0; m < NE; ++m) {
      const int e = tid + m * kScanThreads;
      const int tt = e / DKP, i = e % DKP;
      if (tt < nt && i < dk) {
        const int at = (i / R) * RS + i % R;
        if (MODE == 0) {
          const float lo = sp1[i];
          const float f = lo + (1.0f - lo) * sigmoidf_(rk[m] + sp0[i]);
          sa[tt][at] = f;
          sk[tt][at] = 1.0f - f;
          sq[tt][at] = siluf_(rq[m]);
        } else {
          sk[tt][at] = sdt[tt] * rk[m];
          sq[tt][at] = rq[m];
        }
      }
    }
#pragma unroll
    for (int m = 0; m < NV; ++m) {
      const int e = tid + m * kScanThreads;
      sv[e / BC][e % BC] = rv[m];
    }
    __syncthreads();
    if (t0 + kTB < n) load_round(t0 + kTB);   // in flight during the recurrence below
#pragma unroll 4
    for (int tt = 0; tt < kTB; ++tt) {
      if (tt >= nt) break;
      float vv[CPL], o[CPL];
#pragma unroll
      for (int c = 0; c < CPL; ++c) {
        vv[c] = sv[tt][cl + kScanCols * c];
        o[c] = 0.f;
      }
      const float* pk = &sk[tt][r * RS];
      const float* pq = &sq[tt][r * RS];
      const float* pa = &sa[MODE == 0 ? tt : 0][MODE == 0 ? r * RS : 0];
      const float dec = MODE == 1 ? sdec[tt] : 0.f;
#pragma unroll
      for (int j = 0; j < R; ++j) {
        const float aj = MODE == 0 ? pa[j] : dec, kj = pk[j], qj = pq[j];
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
          S[c][j] = aj * S[c][j] + kj * vv[c];
          o[c] += qj * S[c][j];
        }
      }
#pragma unroll
      for (int c = 0; c < CPL; ++c) {
        const float oc = group_sum<kScanLPC>(o[c]);
        const int col = col0 + kScanCols * c;
        if (col < dv && r == 0)
          a.out[(static_cast<int64_t>(first + t0 + tt) * H + h) * dv + col] = oc + skip * vv[c];
      }
    }
  }
#pragma unroll
  for (int c = 0; c < CPL; ++c) {
    const int col = col0 + kScanCols * c;
    if (col < dv) {
#pragma unroll
      for (int j = 0; j < R; ++j) {
        const int i = r * R + j;
        if (i < dk) st[static_cast<int64_t>(i) * dv + col] = S[c][j];
      }
    }
  }
}

template <typename T, int MODE>
int launch_scan(const ScanArgs& a, int S, hipStream_t st) {
  const dim3 grid(S, a.H, (a.dv + kScanCols - 1) / kScanCols);
#define MIXK_SCAN_R(N)                                                                         \
  if (a.dk <= kScanLPC * N) {                                                                  \
    hipLaunchKernelGGL((gated_linear_scan_kernel<T, N, MODE, 1>), grid, dim3(kScanThreads), 0, \
                       st, a);                                                                 \
    return static_cast<int>(hipGetLastError());                                                \
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
