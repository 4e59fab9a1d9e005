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
// The columns of S evolve independently: a column is owned by 8 or 16 adjacent lanes, lane r
// holding rows r R ... r R + R - 1 in registers for the whole portion, so a token costs R
// multiply-adds per lane for the update, R for the read-out and one DPP sum over the lanes.  A
// workgroup is 32 columns of one (sequence, head); (a, k, q) of kTB tokens at a time are prepared
// by all threads and broadcast through LDS in a [group lane][row] layout read with 16-byte loads;
// the raw inputs of the next round are fetched into registers while the current round runs, so
// the serial chain over tokens does not wait on memory.
// A portion whose first position is 0 starts from the zero state whatever its slot holds.
#include "mix_common.h"
#include "mixers.h"

namespace mixk {

constexpr int kScanCols = 32;   // columns per workgroup (threads = 32 x lanes per column)

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

// MODE 0: forget-gate form, MODE 1: state-space form.  LPC: lanes per column (8 or 16), R: rows
// per lane (dk <= LPC R).  Sixteen lanes per column double the waves of a launch: the loop is
// bound by VALU issue once a SIMD holds four waves, and by latency below that, so launches with
// few (sequence, head, column) workgroups take the 16-lane form.
template <typename T, int R, int MODE, int LPC>
__global__ void __launch_bounds__(kScanCols * LPC, R <= 16 ? 4 : 2)   // four waves per SIMD
gated_linear_scan_kernel(ScanArgs a) {
  constexpr int kThreads = kScanCols * LPC;
  constexpr int kUnroll = R <= 8 ? 4 : (R <= 16 && LPC == 16 ? 2 : 1);
  constexpr int kTB = LPC * R >= 192 ? 8 : 16;     // tokens staged per round
  constexpr int RS = (R + 3) / 4 * 4 + 4;          // LDS stride between the group lanes' rows
  constexpr int DKP = LPC * R;                     // padded key width
  constexpr int NE = kTB * DKP / kThreads;         // (token, channel) entries per thread and round
  constexpr int NV = (kTB * kScanCols + kThreads - 1) / kThreads;
  static_assert(NE * kThreads == kTB * DKP, "staging");
  __shared__ __attribute__((aligned(16))) float sk[kTB][LPC * RS];
  __shared__ __attribute__((aligned(16))) float sq[kTB][LPC * RS];
  __shared__ __attribute__((aligned(16))) float sa[MODE == 0 ? kTB : 1][MODE == 0 ? LPC * RS : 4];
  __shared__ float sp0[MODE == 0 ? DKP : 1], sp1[MODE == 0 ? DKP : 1];
  __shared__ float sdec[kTB], sdt[kTB];
  __shared__ float sv[kTB][kScanCols];
  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int slot = a.seq_slot[s];
  const int first = a.seq_qstart[s], n = a.seq_qstart[s + 1] - first;
  if (slot < 0 || n <= 0) return;
  const int H = a.H, dk = a.dk, dv = a.dv;
  const int r = tid & (LPC - 1), cl = tid / LPC;
  const int col = blockIdx.z * kScanCols + cl;
  const bool active = col < dv;
  const int g = MODE == 0 ? h : h / (H / a.G);
  const T* qp = static_cast<const T*>(a.q) + static_cast<int64_t>(g) * dk;
  const T* kp = static_cast<const T*>(a.k) + static_cast<int64_t>(g) * dk;
  const T* vp = static_cast<const T*>(a.v) + static_cast<int64_t>(h) * dv + blockIdx.z * kScanCols;
  const T* dtp = static_cast<const T*>(a.dt);
  float* st = a.state + (static_cast<int64_t>(slot) * H + h) * dk * dv;
  float S[R];
  const bool fresh = a.positions[first] == 0;
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const int i = r * R + j;
    S[j] = (!fresh && active && i < dk) ? st[static_cast<int64_t>(i) * dv + col] : 0.f;
  }
  // padding rows (dk < LPC R) stay zero in every staged array
  for (int i = tid; i < kTB * LPC * RS; i += kThreads) {
    (&sk[0][0])[i] = 0.f;
    (&sq[0][0])[i] = 0.f;
    if (MODE == 0) (&sa[0][0])[i] = 0.f;
  }
  float rate = 0.f, dtb = 0.f, skip = 0.f;
  if (MODE == 0) {
    for (int i = tid; i < dk; i += kThreads) {
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
      const int e = tid + m * kThreads;
      const int tt = e / DKP, i = e % DKP;
      const bool ok = t0 + tt < n && i < dk;
      const int64_t row = first + t0 + (ok ? tt : 0);
      rq[m] = ok ? ldf(qp + row * a.q_stride + i) : 0.f;
      rk[m] = ok ? ldf(kp + row * a.k_stride + i) : 0.f;
    }
#pragma unroll
    for (int m = 0; m < NV; ++m) {
      const int e = tid + m * kThreads;
      const int tt = e / kScanCols, c = e % kScanCols;
      const bool ok = tt < kTB && t0 + tt < n && blockIdx.z * kScanCols + c < dv;
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
      const int e = tid + m * kThreads;
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
      const int e = tid + m * kThreads;
      if (e < kTB * kScanCols) sv[e / kScanCols][e % kScanCols] = rv[m];
    }
    __syncthreads();
    if (t0 + kTB < n) load_round(t0 + kTB);   // in flight during the recurrence below
    auto token = [&](int tt) {
      const float vv = sv[tt][cl];
      const float* pk = &sk[tt][r * RS];
      const float* pq = &sq[tt][r * RS];
      const float* pa = &sa[MODE == 0 ? tt : 0][MODE == 0 ? r * RS : 0];
      const float dec = MODE == 1 ? sdec[tt] : 0.f;
      float o = 0.f;
#pragma unroll
      for (int j = 0; j < R; ++j) {
        S[j] = (MODE == 0 ? pa[j] : dec) * S[j] + pk[j] * vv;
        o += pq[j] * S[j];
      }
      o = group_sum<LPC>(o);
      if (active && r == 0)
        a.out[(static_cast<int64_t>(first + t0 + tt) * H + h) * dv + col] = o + skip * vv;
    };
    if (kUnroll > 1 && nt == kTB) {
      // full round, constant trip count: unrolled where the registers allow four waves per
      // SIMD with it, so the next token's LDS reads overlap this token's multiply-adds
#pragma unroll kUnroll
      for (int tt = 0; tt < kTB; ++tt) token(tt);
    } else {
#pragma unroll 1
      for (int tt = 0; tt < nt; ++tt) token(tt);
    }
  }
  if (active) {
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const int i = r * R + j;
      if (i < dk) st[static_cast<int64_t>(i) * dv + col] = S[j];
    }
  }
}

template <typename T, int MODE>
int launch_scan(const ScanArgs& a, int S, hipStream_t st) {
  const dim3 grid(S, a.H, (a.dv + kScanCols - 1) / kScanCols);
#define MIXK_SCAN(LPC, N)                                                                        \
  if (a.dk <= LPC * N) {                                                                         \
    hipLaunchKernelGGL((gated_linear_scan_kernel<T, N, MODE, LPC>), grid, dim3(kScanCols * LPC), \
                       0, st, a);                                                                \
    return static_cast<int>(hipGetLastError());                                                  \
  }
  // fewer than ~3 four-wave workgroups per SIMD-quad of the chip: 16 lanes per column
  const int64_t groups = static_cast<int64_t>(grid.x) * grid.y * grid.z;
  if (groups < 768 && a.dk > 32) {
    MIXK_SCAN(16, 4)
    MIXK_SCAN(16, 8)
    MIXK_SCAN(16, 16)
  }
  MIXK_SCAN(8, 2)
  MIXK_SCAN(8, 4)
  MIXK_SCAN(8, 6)
  MIXK_SCAN(8, 8)
  MIXK_SCAN(8, 12)
  MIXK_SCAN(8, 16)
  MIXK_SCAN(8, 24)
  MIXK_SCAN(8, 32)
#undef MIXK_SCAN
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
