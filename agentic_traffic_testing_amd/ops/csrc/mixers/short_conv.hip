// Short causal convolution over time, per channel, followed by SiLU, on ragged batches of
// portions with the last taps - 1 inputs of every sequence carried in its state slot.
//
//   y[t, c] = silu(b[c] + sum_j w[c, j] * x[t - (taps - 1) + j, c]),  x = 0 before position 0
// (the bias b is optional).
//
// conv kernel: grid (rows, channel blocks); inputs before the portion's first row come from
// conv_state[slot, taps - 1, C] - but only where their position is >= 0, so a slot's stale
// contents never reach a sequence that starts at position 0.  A second kernel (launched after
// it on the same stream) advances the tails: it reads old tail and portion, then writes.
#include "mix_common.h"
#include "mixers.h"

namespace mixk {

constexpr int kMaxTaps = 8;

template <typename T>
__global__ void short_conv_silu_kernel(T* __restrict__ out, const T* __restrict__ x,
                                       int64_t x_stride, const T* __restrict__ w,
                                       const T* __restrict__ bias,
                                       const T* __restrict__ conv_state,
                                       const int* __restrict__ positions,
                                       const int* __restrict__ seq_qstart,
                                       const int* __restrict__ seq_slot, int S, int C, int taps) {
  __shared__ int sh[2];
  const int r = blockIdx.x;
  if (threadIdx.x == 0) {
    const int s = seq_of_row(seq_qstart, S, r);
    sh[0] = s < 0 ? -1 : seq_slot[s];
    sh[1] = s < 0 ? 0 : seq_qstart[s];
  }
  __syncthreads();
  const int slot = sh[0], first = sh[1];
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  T* o = out + static_cast<int64_t>(r) * C + c;
  if (slot < 0) {
    stf(o, 0.f);
    return;
  }
  const int pos = positions[r];
  const int j = r - first;  // row index inside the portion
  float acc = bias != nullptr ? ldf(bias + c) : 0.f;
  for (int t = 0; t < taps; ++t) {
    const int back = taps - 1 - t;        // how many tokens before this row
    if (pos - back < 0) continue;
    float xv;
    if (j - back >= 0) {
      xv = ldf(x + (r - back) * x_stride + c);
    } else {
      // tail entry u holds the input (taps - 1 - u) tokens before the portion's first row
      const int u = (taps - 1) + (j - back);
      xv = ldf(conv_state + (static_cast<int64_t>(slot) * (taps - 1) + u) * C + c);
    }
    acc += ldf(w + static_cast<int64_t>(c) * taps + t) * xv;
  }
  stf(o, siluf_(acc));
}

// Eight channels per thread (16-byte loads) for C % 8 == 0 with aligned rows; a thread keeps the
// taps of its eight channels in registers and walks `rows_per_block` rows (8 for prefill-sized
// steps, 1 for decode-sized ones, where the rows are the only parallelism).
constexpr int kConvRows = 8;

template <typename T>
__global__ void __launch_bounds__(128)
short_conv_silu_vec_kernel(T* __restrict__ out, const T* __restrict__ x, int64_t x_stride,
                           const T* __restrict__ w, const T* __restrict__ bias,
                           const T* __restrict__ conv_state,
                           const int* __restrict__ positions, const int* __restrict__ seq_qstart,
                           const int* __restrict__ seq_slot, int T_, int S, int C, int taps,
                           int rows_per_block) {
  __shared__ int sh_slot[kConvRows], sh_first[kConvRows];
  const int r0 = blockIdx.x * rows_per_block;
  if (threadIdx.x < rows_per_block) {
    const int r = r0 + threadIdx.x;
    const int s = r < T_ ? seq_of_row(seq_qstart, S, r) : -1;
    sh_slot[threadIdx.x] = s < 0 ? -1 : seq_slot[s];
    sh_first[threadIdx.x] = s < 0 ? 0 : seq_qstart[s];
  }
  __syncthreads();
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (c >= C) return;
  float wv[kMaxTaps][8];   // [tap][channel], statically indexed below
  {
    const T* wp = w + static_cast<int64_t>(c) * taps;
#pragma unroll
    for (int t = 0; t < kMaxTaps; ++t)
#pragma unroll
      for (int e = 0; e < 8; ++e) wv[t][e] = t < taps ? ldf(wp + e * taps + t) : 0.f;
  }
  float bv[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) bv[e] = bias != nullptr ? ldf(bias + c + e) : 0.f;
#pragma unroll 1
  for (int rr = 0; rr < rows_per_block; ++rr) {
    const int r = r0 + rr;
    if (r >= T_) break;
    const int slot = sh_slot[rr], first = sh_first[rr];
    T* o = out + static_cast<int64_t>(r) * C + c;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    if (slot < 0) {
      st8(o, acc);
      continue;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = bv[e];
    const int pos = positions[r];
    const int j = r - first;
#pragma unroll
    for (int t = 0; t < kMaxTaps; ++t) {
      if (t >= taps) break;
      const int back = taps - 1 - t;
      if (pos - back < 0) continue;
      float xv[8];
      if (j - back >= 0) {
        ld8(x + (r - back) * x_stride + c, xv);
      } else {
        const int u = (taps - 1) + (j - back);
        ld8(conv_state + (static_cast<int64_t>(slot) * (taps - 1) + u) * C + c, xv);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += wv[t][e] * xv[e];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = siluf_(acc[e]);
    st8(o, acc);
  }
}

template <typename T>
__global__ void conv_state_update_kernel(const T* __restrict__ x, int64_t x_stride,
                                         T* __restrict__ conv_state,
                                         const int* __restrict__ positions,
                                         const int* __restrict__ seq_qstart,
                                         const int* __restrict__ seq_slot, int C, int taps) {
  const int s = blockIdx.x;
  const int slot = seq_slot[s];
  const int first = seq_qstart[s], n = seq_qstart[s + 1] - first;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (slot < 0 || n <= 0 || c >= C) return;
  const int start = positions[first];
  const int keep = taps - 1;
  T* tail = conv_state + static_cast<int64_t>(slot) * keep * C + c;
  float nv[kMaxTaps];
  for (int u = 0; u < keep; ++u) {
    // new tail entry u = element n + u of [old tail (keep entries), portion (n rows)]
    const int i = n + u;
    if (i >= keep) {
      nv[u] = ldf(x + (first + i - keep) * x_stride + c);
    } else {
      // old tail entry i is the input at position start - keep + i
      nv[u] = start - keep + i >= 0 ? ldf(tail + static_cast<int64_t>(i) * C) : 0.f;
    }
  }
  for (int u = 0; u < keep; ++u) stf(tail + static_cast<int64_t>(u) * C, nv[u]);
}

}  // namespace mixk

using namespace mixk;

extern "C" int mixk_short_conv_silu(void* out, const void* x, int64_t x_stride, const void* w,
                                    const void* bias, void* conv_state, const int* positions, const int* seq_qstart,
                                    const int* seq_slot, int T_, int S, int C, int taps, int dtype,
                                    hipStream_t st) {
  if (T_ <= 0 || S <= 0) return 0;
  if (taps < 1 || taps > kMaxTaps) return -1;
  const int cb = (C + 255) / 256;
  const bool vec = C % 8 == 0 && x_stride % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0;
  const int rpb = T_ >= 1024 ? kConvRows : 1;
  MIXK_DISPATCH(dtype, {
    if (vec)
      hipLaunchKernelGGL(short_conv_silu_vec_kernel<T>,
                         dim3((T_ + rpb - 1) / rpb, (C / 8 + 127) / 128), dim3(128), 0, st,
                         static_cast<T*>(out), static_cast<const T*>(x), x_stride,
                         static_cast<const T*>(w), static_cast<const T*>(bias),
                         static_cast<const T*>(conv_state), positions, seq_qstart, seq_slot, T_, S,
                         C, taps, rpb);
    else
      hipLaunchKernelGGL(short_conv_silu_kernel<T>, dim3(T_, cb), dim3(256), 0, st,
                         static_cast<T*>(out), static_cast<const T*>(x), x_stride,
                         static_cast<const T*>(w), static_cast<const T*>(bias),
                         static_cast<const T*>(conv_state), positions, seq_qstart, seq_slot, S, C,
                         taps);
    if (taps > 1)
      hipLaunchKernelGGL(conv_state_update_kernel<T>, dim3(S, cb), dim3(256), 0, st,
                         static_cast<const T*>(x), x_stride, static_cast<T*>(conv_state),
                         positions, seq_qstart, seq_slot, C, taps);
  });
  return static_cast<int>(hipGetLastError());
}
