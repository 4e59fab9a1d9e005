// Per-head q / k RMS norm (plain weight), interleaved-pair rotary positions on the first
// 2 * n_freq channels, and the paged K / V write of the softmax mixer.
//
// Grid (rows, (H + 2 G) / 4), four waves per workgroup, one wave per (row, head): heads [0, H)
// are query heads (written to
// q_out [T, H, dim]), [H, H + G) key heads (normed, rotated, written to k_cache
// [nb, G, BS, dim] at the row's slot), [H + G, H + 2 G) value heads (copied to the
// channel-major pages v_cache [nb, G, vdim, BS]).  Angles are fp32: position * inv_freq[i].
#include "mix_common.h"
#include "mixers.h"

namespace mixk {

constexpr int kMaxPairs = 4;  // pairs per lane: head width <= 2 * 64 * kMaxPairs = 512

template <typename T>
__global__ void qk_norm_rope_cache_kernel(T* __restrict__ q_out, const T* __restrict__ qx,
                                          int64_t q_stride, const T* __restrict__ kx,
                                          int64_t k_stride, const T* __restrict__ vx,
                                          int64_t v_stride, const T* __restrict__ q_norm,
                                          const T* __restrict__ k_norm, float eps,
                                          const int* __restrict__ positions,
                                          const int* __restrict__ slot_mapping,
                                          const float* __restrict__ inv_freq, int n_freq,
                                          T* __restrict__ k_cache, T* __restrict__ v_cache, int H,
                                          int G, int dim, int vdim, int block_size) {
  const int t = blockIdx.x, head = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (head >= H + 2 * G) return;
  const int slot = slot_mapping[t];
  if (head >= H + G) {  // value head: copy into the channel-major page
    if (slot < 0) return;
    const int g = head - H - G;
    const T* src = vx + t * v_stride + g * vdim;
    T* dst = v_cache + (static_cast<int64_t>(slot / block_size) * G + g) * vdim * block_size +
             slot % block_size;
    for (int i = lane; i < vdim; i += kWave) dst[static_cast<int64_t>(i) * block_size] = src[i];
    return;
  }
  const bool is_q = head < H;
  if (!is_q && slot < 0) return;
  const T* src = is_q ? qx + t * q_stride + head * dim : kx + t * k_stride + (head - H) * dim;
  const T* w = is_q ? q_norm : k_norm;
  T* dst = is_q ? q_out + (static_cast<int64_t>(t) * H + head) * dim
                : k_cache + ((static_cast<int64_t>(slot / block_size) * G + (head - H)) *
                                 block_size + slot % block_size) * dim;
  const int pairs = dim >> 1;
  float u[kMaxPairs], v[kMaxPairs];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < kMaxPairs; ++j) {
    const int i = lane + j * kWave;
    u[j] = v[j] = 0.f;
    if (i < pairs) {
      u[j] = ldf(src + 2 * i);
      v[j] = ldf(src + 2 * i + 1);
      ss += u[j] * u[j] + v[j] * v[j];
    }
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(dim) + eps);
  const float pos = static_cast<float>(positions[t]);
#pragma unroll
  for (int j = 0; j < kMaxPairs; ++j) {
    const int i = lane + j * kWave;
    if (i >= pairs) continue;
    float a = u[j] * inv * ldf(w + 2 * i);
    float b = v[j] * inv * ldf(w + 2 * i + 1);
    if (i < n_freq) {
      float sn, cs;
      sincosf(pos * inv_freq[i], &sn, &cs);
      const float ra = a * cs - b * sn;
      const float rb = b * cs + a * sn;
      a = ra;
      b = rb;
    }
    stf(dst + 2 * i, a);
    stf(dst + 2 * i + 1, b);
  }
}

}  // namespace mixk

using namespace mixk;

extern "C" int mixk_qk_norm_rope_cache(void* q_out, const void* qx, int64_t q_stride,
                                       const void* kx, int64_t k_stride, const void* vx,
                                       int64_t v_stride, const void* q_norm, const void* k_norm,
                                       float eps, const int* positions, const int* slot_mapping,
                                       const float* inv_freq, int n_freq, void* k_cache,
                                       void* v_cache, int T_, int H, int G, int dim, int vdim,
                                       int block_size, int dtype, hipStream_t st) {
  if (T_ <= 0) return 0;
  if (dim > 2 * kWave * kMaxPairs || (dim & 1)) return -1;
  MIXK_DISPATCH(dtype,
                hipLaunchKernelGGL(qk_norm_rope_cache_kernel<T>, dim3(T_, (H + 2 * G + 3) / 4), dim3(256),
                                   0, st, static_cast<T*>(q_out), static_cast<const T*>(qx),
                                   q_stride, static_cast<const T*>(kx), k_stride,
                                   static_cast<const T*>(vx), v_stride,
                                   static_cast<const T*>(q_norm), static_cast<const T*>(k_norm),
                                   eps, positions, slot_mapping, inv_freq, n_freq,
                                   static_cast<T*>(k_cache), static_cast<T*>(v_cache), H, G, dim,
                                   vdim, block_size));
  return static_cast<int>(hipGetLastError());
}
