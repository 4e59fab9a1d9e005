// Causal paged softmax attention for any head widths, with an optional sink (one extra key of
// score 0 and no value in every denominator); fp32 scores, weights and accumulation for bf16
// and fp32 activations alike.
//
// One workgroup of 256 threads per (tile of 16 query rows of one portion, query head).  Keys
// are streamed in tiles of KT tokens through LDS (K and V converted to fp32 once per tile);
// thread (r, c) = (tid / 16, tid % 16) scores row r against keys c, c + 16, ... of the tile,
// the 16 threads of a row share max / sum by lane shuffles (online softmax), and the same
// thread accumulates value channels c, c + 16, ... of row r.  The sink enters as the initial
// state of the online softmax: running max 0, running sum 1, zero accumulator.
#include "mix_common.h"
#include "mixers.h"

namespace mixk {

constexpr int kRows = 16;       // query rows per workgroup
constexpr int kMaxVPer = 16;    // value channels per thread: vdim <= 256
constexpr float kNegBig = -1.0e30f;

template <typename T>
__global__ void __launch_bounds__(256)
sink_attention_kernel(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k_cache,
                      const T* __restrict__ v_cache, const int* __restrict__ block_tables,
                      int bt_width, const int* __restrict__ seq_kvlen,
                      const int* __restrict__ seq_qstart, const int* __restrict__ tile_seq,
                      const int* __restrict__ tile_qoff, int H, int G, int dim, int vdim,
                      int block_size, float scale, int sink, int KT) {
  extern __shared__ float smem[];
  const int tile = blockIdx.x, h = blockIdx.y, g = h / (H / G);
  const int s = tile_seq[tile], qo = tile_qoff[tile];
  const int row0 = seq_qstart[s];
  const int n = seq_qstart[s + 1] - row0;
  const int kvlen = seq_kvlen[s];
  if (n <= 0 || kvlen <= 0 || qo >= n) return;
  const int nrows = min(kRows, n - qo);
  const int tid = threadIdx.x, r = tid >> 4, c = tid & 15;
  const int kstride = dim + 1;
  float* Qs = smem;                        // [kRows][dim]
  float* Ks = Qs + kRows * dim;            // [KT][dim + 1]
  float* Vs = Ks + KT * kstride;           // [KT][vdim]
  float* Ps = Vs + KT * vdim;              // [kRows][KT]
  for (int i = tid; i < kRows * dim; i += 256) {
    const int rr = i / dim, d = i - rr * dim;
    Qs[i] = rr < nrows ? ldf(q + (static_cast<int64_t>(row0 + qo + rr) * H + h) * dim + d) : 0.f;
  }
  const int qpos = kvlen - n + qo + r;          // position of this thread's row
  const bool row_ok = r < nrows;
  const int kend = min(kvlen, kvlen - n + qo + nrows);   // keys any row of the tile may see
  float m = sink ? 0.f : kNegBig, l = sink ? 1.f : 0.f;
  float acc[kMaxVPer];
#pragma unroll
  for (int j = 0; j < kMaxVPer; ++j) acc[j] = 0.f;
  const int* bt = block_tables + static_cast<int64_t>(s) * bt_width;
  const int kper = KT >> 4;
  for (int k0 = 0; k0 < kend; k0 += KT) {
    __syncthreads();  // previous tile fully consumed (and Qs written, first time round)
    for (int i = tid; i < KT * dim; i += 256) {
      const int kk = i / dim, d = i - kk * dim;
      const int tok = k0 + kk;
      float val = 0.f;
      if (tok < kend) {
        const int64_t page = bt[tok / block_size];
        val = ldf(k_cache + ((page * G + g) * block_size + tok % block_size) * dim + d);
      }
      Ks[kk * kstride + d] = val;
    }
    for (int i = tid; i < KT * vdim; i += 256) {
      const int kk = i / vdim, d = i - kk * vdim;
      const int tok = k0 + kk;
      float val = 0.f;
      if (tok < kend) {
        const int64_t page = bt[tok / block_size];
        val = ldf(v_cache + ((page * G + g) * block_size + tok % block_size) * vdim + d);
      }
      Vs[i] = val;
    }
    __syncthreads();
    float sc[4];
    float tmax = kNegBig;
    for (int j = 0; j < kper; ++j) {
      const int kk = c + 16 * j;
      const float* kr = Ks + kk * kstride;
      const float* qr = Qs + r * dim;
      float dot = 0.f;
      for (int d = 0; d < dim; ++d) dot += qr[d] * kr[d];
      const int tok = k0 + kk;
      sc[j] = (row_ok && tok <= qpos && tok < kvlen) ? dot * scale : kNegBig;
      tmax = fmaxf(tmax, sc[j]);
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, o, kWave));
    const float m_new = fmaxf(m, tmax);
    const float alpha = expf(m - m_new);
    float psum = 0.f;
    for (int j = 0; j < kper; ++j) {
      const float p = sc[j] <= kNegBig ? 0.f : expf(sc[j] - m_new);
      Ps[r * KT + c + 16 * j] = p;
      psum += p;
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) psum += __shfl_xor(psum, o, kWave);
    l = l * alpha + psum;
    m = m_new;
    __syncthreads();
    const float* pr = Ps + r * KT;
#pragma unroll
    for (int j = 0; j < kMaxVPer; ++j) {
      const int d = c + 16 * j;
      if (d < vdim) {
        float a = acc[j] * alpha;
        for (int kk = 0; kk < KT; ++kk) a += pr[kk] * Vs[kk * vdim + d];
        acc[j] = a;
      }
    }
  }
  if (!row_ok) return;
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  T* o = out + (static_cast<int64_t>(row0 + qo + r) * H + h) * vdim;
#pragma unroll
  for (int j = 0; j < kMaxVPer; ++j) {
    const int d = c + 16 * j;
    if (d < vdim) stf(o + d, acc[j] * inv);
  }
}

template <typename T>
int launch_sink_attention(void* out, const void* q, const void* k_cache, const void* v_cache,
                          const int* block_tables, int bt_width, const int* seq_kvlen,
                          const int* seq_qstart, const int* tile_seq, const int* tile_qoff,
                          int num_tiles, int H, int G, int dim, int vdim, int block_size,
                          float scale, int sink, hipStream_t st) {
  int KT = 64;
  auto bytes = [&](int kt) {
    return sizeof(float) * (static_cast<size_t>(kRows) * dim + static_cast<size_t>(kt) * (dim + 1) +
                            static_cast<size_t>(kt) * vdim + static_cast<size_t>(kRows) * kt);
  };
  while (KT > 16 && bytes(KT) > 96 * 1024) KT >>= 1;
  const size_t smem = bytes(KT);
  if (smem > 150 * 1024) return -1;
  static size_t opted = 0;
  if (smem > 48 * 1024 && smem > opted) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(sink_attention_kernel<T>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                       static_cast<int>(smem));
    if (e != hipSuccess) return static_cast<int>(e);
    opted = smem;
  }
  hipLaunchKernelGGL(sink_attention_kernel<T>, dim3(num_tiles, H), dim3(256), smem, st,
                     static_cast<T*>(out), static_cast<const T*>(q),
                     static_cast<const T*>(k_cache), static_cast<const T*>(v_cache), block_tables,
                     bt_width, seq_kvlen, seq_qstart, tile_seq, tile_qoff, H, G, dim, vdim,
                     block_size, scale, sink, KT);
  return static_cast<int>(hipGetLastError());
}

}  // namespace mixk

using namespace mixk;

extern "C" int mixk_sink_attention(void* out, const void* q, const void* k_cache,
                                   const void* v_cache, const int* block_tables, int bt_width,
                                   const int* seq_kvlen, const int* seq_qstart,
                                   const int* tile_seq, const int* tile_qoff, int num_tiles, int H,
                                   int G, int dim, int vdim, int block_size, float scale, int sink,
                                   int dtype, hipStream_t st) {
  if (num_tiles <= 0) return 0;
  if (vdim > 16 * kMaxVPer || H % G != 0) return -1;
  int rc = 0;
  MIXK_DISPATCH(dtype, rc = launch_sink_attention<T>(out, q, k_cache, v_cache, block_tables,
                                                     bt_width, seq_kvlen, seq_qstart, tile_seq,
                                                     tile_qoff, num_tiles, H, G, dim, vdim,
                                                     block_size, scale, sink, st));
  return rc;
}
