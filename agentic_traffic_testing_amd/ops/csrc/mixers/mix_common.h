// Shared helpers of the sequence-mixer kernels (gfx950, wave = 64 lanes).
//
// Activations are bf16 or fp32 (template parameter T); everything between a load and the final
// store is fp32.  Batch metadata is int32: positions[T], seq_qstart[S + 1], seq_slot[S]
// (-1: padding sequence, skipped), slot_mapping[T] (-1: row not cached).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mixk {

constexpr int kWave = 64;

template <typename T>
__device__ __forceinline__ float ldf(const T* p) {
  return static_cast<float>(*p);
}
template <typename T>
__device__ __forceinline__ void stf(T* p, float v) {
  *p = static_cast<T>(v);
}

// 8 consecutive activations as fp32 (16-byte loads; p must be 16-byte aligned for bf16,
// 32-byte aligned pairs of 16-byte loads for fp32) and back.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4v;
__device__ __forceinline__ void ld8(const __bf16* p, float* o) {
  const bf16x8_t v = *reinterpret_cast<const bf16x8_t*>(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = static_cast<float>(v[i]);
}
__device__ __forceinline__ void ld8(const float* p, float* o) {
  const f32x4v a = *reinterpret_cast<const f32x4v*>(p), b = *reinterpret_cast<const f32x4v*>(p + 4);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    o[i] = a[i];
    o[4 + i] = b[i];
  }
}
__device__ __forceinline__ void st8(__bf16* p, const float* o) {
  bf16x8_t v;
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = static_cast<__bf16>(o[i]);
  *reinterpret_cast<bf16x8_t*>(p) = v;
}
__device__ __forceinline__ void st8(float* p, const float* o) {
  *reinterpret_cast<f32x4v*>(p) = f32x4v{o[0], o[1], o[2], o[3]};
  *reinterpret_cast<f32x4v*>(p + 4) = f32x4v{o[4], o[5], o[6], o[7]};
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

// Sum over the block (blockDim.x a multiple of 64, <= 1024); scratch: blockDim.x / 64 floats.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  v = wave_sum(v);
  if (lane == 0) scratch[wid] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += scratch[i];
  __syncthreads();
  return t;
}

// Sum over the four lanes of a quad, result in all of them: two DPP quad permutes on the VALU
// (lane ^ 1, lane ^ 2) - no trip through the LDS crossbar on the recurrence's critical path.
__device__ __forceinline__ float quad_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1,
                                                             0xF, 0xF, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E,
                                                             0xF, 0xF, true));
  return v;
}
// ... and over the 8 or 16 lanes of an aligned group: the mirrored half-row brings the other
// quad, the mirrored row the other half.
template <int LPC>
__device__ __forceinline__ float group_sum(float v) {
  v = quad_sum(v);
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141,
                                                             0xF, 0xF, true));
  if (LPC == 16)
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v),
                                                               0x140, 0xF, 0xF, true));
  return v;
}

// Index of the sequence whose portion holds `row` (seq_qstart ascending, S >= 1), or -1 for a
// row past the last portion.
__device__ __forceinline__ int seq_of_row(const int* __restrict__ seq_qstart, int S, int row) {
  if (row >= seq_qstart[S] || row < seq_qstart[0]) return -1;
  int lo = 0, hi = S - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (seq_qstart[mid] <= row) lo = mid; else hi = mid - 1;
  }
  return lo;
}

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float siluf_(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplusf_(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

}  // namespace mixk

// dtype codes of the launchers: 0 = bf16, 2 = fp32
#define MIXK_DISPATCH(code, ...)                      \
  do {                                                \
    if ((code) == 2) {                                \
      using T = float;                                \
      __VA_ARGS__;                                    \
    } else {                                          \
      using T = __bf16;                               \
      __VA_ARGS__;                                    \
    }                                                 \
  } while (0)
