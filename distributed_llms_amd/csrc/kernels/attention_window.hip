// Sliding-window attention over a paged K/V cache whose key and value head sizes differ
// (ops/seqmix.py window_attention): caches k [NB, G, BS, D], v [NB, G, BS, Dv] (one row per key),
// query head h reads K/V head h / (H / G), a query at position p sees the keys j of its sequence with
// 0 <= p - j < window.  Scores, softmax weights and the weighted sum are float32; T is the storage
// type (bf16 or float).  Head sizes, window and block size are runtime values.
//
//   window_attn_row_kernel   one workgroup per (query token, head): keys in tiles of 256, one key per
//                            thread for q.k, an online softmax across tiles, then P.V with the
//                            threads laid out (value channel, key subgroup).  Decode rows, and prompt
//                            chunks too short to fill a query tile.
#include <math.h>

#include "common.h"
#include "launchers.h"

namespace dllm {

template <typename T> __device__ __forceinline__ float wld(const T* p) { return (float)*p; }

constexpr int kWinTile = 256;     // keys per tile = threads per workgroup
constexpr int kWinMaxAcc = 2;     // value channels per thread: Dv <= 256 * kWinMaxAcc

template <typename T>
__device__ __forceinline__ float dot_row(const float* __restrict__ qs, const T* __restrict__ k, int D) {
  float s = 0.f;
  for (int d = 0; d < D; ++d) s = fmaf(qs[d], wld(k + d), s);
  return s;
}

// 16-byte loads when rows are 16-byte aligned (D % 8 == 0)
template <>
__device__ __forceinline__ float dot_row<bf16>(const float* __restrict__ qs, const bf16* __restrict__ k, int D) {
  float s = 0.f;
  if ((D & 7) == 0) {
    const bf16x8* kv = reinterpret_cast<const bf16x8*>(k);
    for (int d = 0; d < D; d += 8) {
      const bf16x8 v = kv[d >> 3];
#pragma unroll
      for (int j = 0; j < 8; ++j) s = fmaf(qs[d + j], bf2f(v[j]), s);
    }
    return s;
  }
  for (int d = 0; d < D; ++d) s = fmaf(qs[d], bf2f(k[d]), s);
  return s;
}

template <>
__device__ __forceinline__ float dot_row<float>(const float* __restrict__ qs, const float* __restrict__ k, int D) {
  float s = 0.f;
  if ((D & 3) == 0) {
    const f32x4* kv = reinterpret_cast<const f32x4*>(k);
    for (int d = 0; d < D; d += 4) {
      const f32x4 v = kv[d >> 2];
      s = fmaf(qs[d], v[0], s);
      s = fmaf(qs[d + 1], v[1], s);
      s = fmaf(qs[d + 2], v[2], s);
      s = fmaf(qs[d + 3], v[3], s);
    }
    return s;
  }
  for (int d = 0; d < D; ++d) s = fmaf(qs[d], k[d], s);
  return s;
}

template <typename T>
__global__ void __launch_bounds__(kWinTile) window_attn_row_kernel(
    void* __restrict__ out_, const void* __restrict__ q_, const void* __restrict__ k_cache_,
    const void* __restrict__ v_cache_, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ tok_seq, int t0, int H, int G, int D, int Dv,
    int bs, int window, float scale) {
  extern __shared__ float lds[];
  float* qs = lds;                       // [D]
  float* p = qs + D;                     // [kWinTile]
  int* rows = reinterpret_cast<int*>(p + kWinTile);   // [kWinTile] cache row of each key of the tile
  float* red = reinterpret_cast<float*>(rows + kWinTile);   // [16]
  float* part = red + 16;                // [nsub][Dv] at the end
  const int t = t0 + blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int g = h / (H / G);
  const int pos = positions[t], b = tok_seq[t];
  const int lo = max(0, pos - window + 1);
  const T* q = (const T*)q_ + ((size_t)t * H + h) * D;
  const T* kc = (const T*)k_cache_;
  const T* vc = (const T*)v_cache_;
  const int32_t* bt = block_tables + (size_t)b * max_blocks;
  for (int d = tid; d < D; d += kWinTile) qs[d] = wld(q + d);
  // P.V layout: thread = (channel e of ew, key subgroup sub of nsub); channels beyond ew loop
  const int ew = min(kWinTile, ((Dv + 63) / 64) * 64);
  const int nsub = kWinTile / ew;
  const int e0 = tid % ew, sub = tid / ew;
  float acc[kWinMaxAcc];
#pragma unroll
  for (int i = 0; i < kWinMaxAcc; ++i) acc[i] = 0.f;
  float m = -INFINITY, l = 0.f;
  __syncthreads();
  for (int k0 = lo; k0 <= pos; k0 += kWinTile) {
    const int j = k0 + tid;
    float s = -INFINITY;
    if (j <= pos) {
      const int blk = bt[j / bs];
      const int row = (blk * G + g) * bs + (j % bs);
      rows[tid] = row;
      s = dot_row<T>(qs, kc + (size_t)row * D, D) * scale;
    }
    const float m_new = fmaxf(m, block_max(s, red));
    const float pj = j <= pos ? expf(s - m_new) : 0.f;
    p[tid] = pj;
    const float psum = block_sum(pj, red);      // ends with a barrier: p and rows are visible
    const float corr = expf(m - m_new);         // 0 at the first tile (m = -inf)
    l = l * corr + psum;
    m = m_new;
    const int nk = min(kWinTile, pos + 1 - k0);
#pragma unroll
    for (int i = 0; i < kWinMaxAcc; ++i) {
      const int e = e0 + i * ew;
      if (sub < nsub && e < Dv) {
        float a = acc[i] * corr;
        for (int k = sub; k < nk; k += nsub) a = fmaf(p[k], wld(vc + (size_t)rows[k] * Dv + e), a);
        acc[i] = a;
      }
    }
    __syncthreads();                            // before the next tile overwrites p and rows
  }
  // sum the key subgroups
  T* out = (T*)out_ + ((size_t)t * H + h) * Dv;
#pragma unroll
  for (int i = 0; i < kWinMaxAcc; ++i) {
    const int e = e0 + i * ew;
    if (sub < nsub && e < Dv) part[sub * Dv + e] = acc[i];
    __syncthreads();
    if (sub == 0 && e < Dv) {
      float a = 0.f;
      for (int s2 = 0; s2 < nsub; ++s2) a += part[s2 * Dv + e];
      out[e] = (T)(a / l);
    }
    __syncthreads();
  }
}

static size_t win_row_lds(int D, int Dv) {
  const int ew = std::min(kWinTile, ((Dv + 63) / 64) * 64);
  return sizeof(float) * ((size_t)D + kWinTile + kWinTile + 16 + (size_t)(kWinTile / ew) * Dv);
}

static void launch_rows(uintptr_t out, uintptr_t q, uintptr_t k_cache, uintptr_t v_cache, uintptr_t block_tables,
                        int max_blocks, uintptr_t positions, uintptr_t tok_seq, int t0, int rows, int H, int G, int D,
                        int Dv, int bs, int window, float scale, int f32, uintptr_t stream) {
  DLLM_HOST_CHECK(H > 0 && G > 0 && H % G == 0 && D > 0 && Dv > 0 && Dv <= kWinTile * kWinMaxAcc, "window attention heads");
  DLLM_HOST_CHECK(bs > 0 && window >= 1 && max_blocks > 0 && H <= 65535, "window attention sizes");
  const size_t lds = win_row_lds(D, Dv);
  DLLM_HOST_CHECK(lds <= 64 * 1024, "window attention head size");
  if (f32)
    hipLaunchKernelGGL(HIP_KERNEL_NAME(window_attn_row_kernel<float>), dim3(rows, H), dim3(kWinTile), lds,
                       (hipStream_t)stream, (void*)out, (const void*)q, (const void*)k_cache, (const void*)v_cache,
                       (const int32_t*)block_tables, max_blocks, (const int32_t*)positions, (const int32_t*)tok_seq, t0,
                       H, G, D, Dv, bs, window, scale);
  else
    hipLaunchKernelGGL(HIP_KERNEL_NAME(window_attn_row_kernel<bf16>), dim3(rows, H), dim3(kWinTile), lds,
                       (hipStream_t)stream, (void*)out, (const void*)q, (const void*)k_cache, (const void*)v_cache,
                       (const int32_t*)block_tables, max_blocks, (const int32_t*)positions, (const int32_t*)tok_seq, t0,
                       H, G, D, Dv, bs, window, scale);
  DLLM_HIP_CHECK(hipGetLastError());
}

// Decode rows: tokens [0, rows) are one-token sequences.
void sm_window_attn_decode(uintptr_t out, uintptr_t q, uintptr_t k_cache, uintptr_t v_cache, uintptr_t block_tables,
                           int max_blocks, uintptr_t positions, uintptr_t tok_seq, int rows, int H, int G, int D,
                           int Dv, int bs, int window, float scale, int f32, uintptr_t stream) {
  if (rows <= 0) return;
  launch_rows(out, q, k_cache, v_cache, block_tables, max_blocks, positions, tok_seq, 0, rows, H, G, D, Dv, bs, window,
              scale, f32, stream);
}

// Prompt chunks: tokens [t0 .. tokens) of sequences [seq0, seqs).
void sm_window_attn_prefill(uintptr_t out, uintptr_t q, uintptr_t k_cache, uintptr_t v_cache, uintptr_t block_tables,
                            int max_blocks, uintptr_t cu, uintptr_t positions, uintptr_t tok_seq, int seq0, int seqs,
                            int tokens, int max_q_len, int H, int G, int D, int Dv, int bs, int window, float scale,
                            int f32, uintptr_t stream) {
  // tokens of the decode rows come first: one per sequence before seq0
  const int t0 = seq0;
  if (tokens <= t0) return;
  launch_rows(out, q, k_cache, v_cache, block_tables, max_blocks, positions, tok_seq, t0, tokens - t0, H, G, D, Dv, bs,
              window, scale, f32, stream);
}

}  // namespace dllm
