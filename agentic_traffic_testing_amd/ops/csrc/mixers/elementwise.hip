// Embedding (token + hashed token-pair rows), fp32-residual RMS norm, squared ReLU, the
// residual sum of a layer's branches, and the gated per-head output norm of the delta rule.
#include "mix_common.h"
#include "mixers.h"

namespace mixk {

// One block per row.  The token before a portion's first row is the sequence's state
// (prev_token[slot]); the block of that first row reads it and then replaces it with the
// portion's last token, so no other block touches the slot's entry in this launch.
template <typename T>
__global__ void embed_pair_kernel(float* __restrict__ out, const T* __restrict__ table,
                                  const T* __restrict__ pair, const int* __restrict__ ids,
                                  const int* __restrict__ positions,
                                  const int* __restrict__ seq_qstart,
                                  const int* __restrict__ seq_slot, int* __restrict__ prev_token,
                                  int S, int W, int64_t mul_prev, int64_t mul_cur,
                                  int64_t buckets) {
  __shared__ int64_t sh_row;
  __shared__ int sh_ok;
  const int r = blockIdx.x;
  if (threadIdx.x == 0) {
    const int s = seq_of_row(seq_qstart, S, r);
    const int slot = s < 0 ? -1 : seq_slot[s];
    sh_ok = slot >= 0;
    if (slot >= 0) {
      const int first = seq_qstart[s];
      const int64_t id = ids[r];
      int64_t row = buckets;
      if (positions[r] != 0) {
        const int64_t prev = r == first ? prev_token[slot] : ids[r - 1];
        row = (prev * mul_prev + id * mul_cur) % buckets;
      }
      sh_row = row;
      if (r == first) prev_token[slot] = ids[seq_qstart[s + 1] - 1];
    }
  }
  __syncthreads();
  float* o = out + static_cast<int64_t>(r) * W;
  if (!sh_ok) {
    for (int i = threadIdx.x; i < W; i += blockDim.x) o[i] = 0.f;
    return;
  }
  const T* e = table + static_cast<int64_t>(ids[r]) * W;
  const T* p = pair + sh_row * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) o[i] = ldf(e + i) + ldf(p + i);
}

template <typename T>
__global__ void rms_norm_f32_kernel(T* __restrict__ out, const float* __restrict__ x,
                                    const T* __restrict__ w, int W, float eps, float plus) {
  __shared__ float scratch[16];
  const float* xr = x + static_cast<int64_t>(blockIdx.x) * W;
  T* o = out + static_cast<int64_t>(blockIdx.x) * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) ss += xr[i] * xr[i];
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(W) + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) stf(o + i, xr[i] * inv * (ldf(w + i) + plus));
}

template <typename T>
__global__ void relu_sq_kernel(T* __restrict__ out, const T* __restrict__ x, int N,
                               int64_t x_stride) {
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= N) return;
  const float v = fmaxf(ldf(x + blockIdx.x * x_stride + i), 0.f);
  stf(out + static_cast<int64_t>(blockIdx.x) * N + i, v * v);
}

template <typename T>
__global__ void residual_add_kernel(float* __restrict__ x, const T* __restrict__ a, float sa,
                                    const T* __restrict__ b, float sb, const T* __restrict__ c,
                                    int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float y = ldf(a + i) * sa;
  if (b != nullptr) y += ldf(b + i) * sb;
  if (c != nullptr) y += ldf(c + i);
  x[i] += y;
}

// One wave per (row, head): o / sqrt(mean(o^2) + eps) * w * act(gate).
template <typename T>
__global__ void gated_rms_norm_kernel(T* __restrict__ out, const float* __restrict__ o,
                                      const T* __restrict__ gate, int64_t gate_stride,
                                      const T* __restrict__ w, int H, int dv, float eps, int act) {
  const int t = blockIdx.x / H, h = blockIdx.x % H;
  const float* orow = o + (static_cast<int64_t>(t) * H + h) * dv;
  const T* g = gate + t * gate_stride + h * dv;
  T* y = out + (static_cast<int64_t>(t) * H + h) * dv;
  float ss = 0.f;
  for (int i = threadIdx.x; i < dv; i += kWave) ss += orow[i] * orow[i];
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(dv) + eps);
  for (int i = threadIdx.x; i < dv; i += kWave) {
    const float gv = ldf(g + i);
    const float ga = act == 1 ? sigmoidf_(gv) : siluf_(gv);
    stf(y + i, orow[i] * inv * ldf(w + i) * ga);
  }
}

}  // namespace mixk

using namespace mixk;

extern "C" int mixk_embed_pair(float* out, const void* table, const void* pair_table,
                               const int* ids, const int* positions, const int* seq_qstart,
                               const int* seq_slot, int* prev_token, int T_, int S, int W,
                               int64_t mul_prev, int64_t mul_cur, int64_t buckets, int dtype,
                               hipStream_t st) {
  if (T_ <= 0) return 0;
  MIXK_DISPATCH(dtype, hipLaunchKernelGGL(embed_pair_kernel<T>, dim3(T_), dim3(256), 0, st, out,
                                          static_cast<const T*>(table),
                                          static_cast<const T*>(pair_table), ids, positions,
                                          seq_qstart, seq_slot, prev_token, S, W, mul_prev,
                                          mul_cur, buckets));
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_rms_norm_f32(void* out, const float* x, const void* w, int T_, int W,
                                 float eps, int one_plus, int dtype, hipStream_t st) {
  if (T_ <= 0) return 0;
  MIXK_DISPATCH(dtype, hipLaunchKernelGGL(rms_norm_f32_kernel<T>, dim3(T_), dim3(256), 0, st,
                                          static_cast<T*>(out), x, static_cast<const T*>(w), W,
                                          eps, one_plus ? 1.0f : 0.0f));
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_relu_sq(void* out, const void* x, int T_, int N, int64_t x_stride, int dtype,
                            hipStream_t st) {
  if (T_ <= 0 || N <= 0) return 0;
  MIXK_DISPATCH(dtype, hipLaunchKernelGGL(relu_sq_kernel<T>, dim3(T_, (N + 255) / 256), dim3(256),
                                          0, st, static_cast<T*>(out), static_cast<const T*>(x), N,
                                          x_stride));
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_residual_add(float* x, const void* a, float sa, const void* b, float sb,
                                 const void* c, int64_t n, int dtype, hipStream_t st) {
  if (n <= 0) return 0;
  MIXK_DISPATCH(dtype, hipLaunchKernelGGL(residual_add_kernel<T>,
                                          dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256),
                                          0, st, x, static_cast<const T*>(a), sa,
                                          static_cast<const T*>(b), sb, static_cast<const T*>(c),
                                          n));
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_gated_rms_norm(void* out, const float* o, const void* gate,
                                   int64_t gate_stride, const void* w, int T_, int H, int dv,
                                   float eps, int act, int dtype, hipStream_t st) {
  if (T_ <= 0) return 0;
  MIXK_DISPATCH(dtype, hipLaunchKernelGGL(gated_rms_norm_kernel<T>, dim3(T_ * H), dim3(kWave), 0,
                                          st, static_cast<T*>(out), o,
                                          static_cast<const T*>(gate), gate_stride,
                                          static_cast<const T*>(w), H, dv, eps, act));
  return static_cast<int>(hipGetLastError());
}
