// Kernels of layer-list models with per-sequence state (ops/seqmix.py): a float32 residual stream
// with RMS norms before and after every sublayer, short causal convolutions whose tail lives in a
// state slot, the real-gated linear recurrent unit (gates, then a chunked linear scan), the
// attention input stage (convolution + per-head norm + interleaved rotation + paged append), a
// clipped GLU and the logit soft cap.
//
// Every kernel is a template over the activation type T (bf16 or float): the float32 build is the
// exact path (true 32-bit everywhere), the bf16 build keeps in float32 what feeds a norm, a
// rotation, a gate of the recurrence or the state.  Sizes are runtime values with bounds checks,
// no divisibility assumed: widths, head sizes, taps and block counts come from the model's config.
#include <math.h>

#include "common.h"
#include "launchers.h"

namespace dllm {

template <typename T> __device__ __forceinline__ float ldf(const T* p) { return (float)*p; }
template <typename T> __device__ __forceinline__ void stf(T* p, float v) { *p = (T)v; }

#define SM_DISPATCH(f32, KERNEL, grid, block, lds, stream, ...)                                        \
  do {                                                                                                 \
    if (f32)                                                                                           \
      hipLaunchKernelGGL(HIP_KERNEL_NAME(KERNEL<float>), grid, block, lds, (hipStream_t)(stream), __VA_ARGS__); \
    else                                                                                               \
      hipLaunchKernelGGL(HIP_KERNEL_NAME(KERNEL<bf16>), grid, block, lds, (hipStream_t)(stream), __VA_ARGS__);  \
    DLLM_HIP_CHECK(hipGetLastError());                                                                 \
  } while (0)

// --------------------------------------------------------------------------- embedding -> f32
template <typename T>
__global__ void __launch_bounds__(256) sm_embed_kernel(float* __restrict__ out, const int32_t* __restrict__ ids,
                                                       const void* __restrict__ table_, int width, int vocab) {
  const T* table = (const T*)table_;
  int id = ids[blockIdx.x];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* src = table + (size_t)id * width;
  float* dst = out + (size_t)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += 256) dst[i] = ldf(src + i);
}

void sm_embed_f32(uintptr_t out, uintptr_t ids, uintptr_t table, int tokens, int width, int vocab, int f32,
                  uintptr_t stream) {
  if (tokens <= 0) return;
  DLLM_HOST_CHECK(width > 0 && vocab > 0, "embed sizes");
  SM_DISPATCH(f32, sm_embed_kernel, dim3(tokens), dim3(256), 0, stream, (float*)out, (const int32_t*)ids,
              (const void*)table, width, vocab);
}

// --------------------------------------------------------------------------- RMS norm of an f32 row
// y = x * rsqrt(mean(x^2) + eps) * (offset + w); one workgroup per row.
template <typename T>
__global__ void __launch_bounds__(256) sm_rms_norm_kernel(void* __restrict__ y_, const float* __restrict__ x,
                                                          const void* __restrict__ w_, int width, float eps,
                                                          float offset) {
  __shared__ float red[16];
  T* y = (T*)y_ + (size_t)blockIdx.x * width;
  const T* w = (const T*)w_;
  const float* xr = x + (size_t)blockIdx.x * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += 256) {
    const float v = xr[i];
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += 256) stf(y + i, xr[i] * inv * (offset + ldf(w + i)));
}

void sm_rms_norm(uintptr_t y, uintptr_t x, uintptr_t w, int rows, int width, float eps, float offset, int f32,
                 uintptr_t stream) {
  if (rows <= 0) return;
  DLLM_HOST_CHECK(width > 0, "norm width");
  SM_DISPATCH(f32, sm_rms_norm_kernel, dim3(rows), dim3(256), 0, stream, (void*)y, (const float*)x, (const void*)w,
              width, eps, offset);
}

// --------------------------------------------------------------------------- close of a sublayer
// x += mult * rms_norm(o + bias) * (1 + w_post);  h = rms_norm(x) * (1 + w_next) when w_next.
template <typename T>
__global__ void __launch_bounds__(256) sm_post_norm_add_kernel(float* __restrict__ x, const void* __restrict__ o_,
                                                               const void* __restrict__ bias_,
                                                               const void* __restrict__ wp_,
                                                               const void* __restrict__ wn_, void* __restrict__ h_,
                                                               int width, float eps, float mult) {
  __shared__ float red[16];
  const T* o = (const T*)o_ + (size_t)blockIdx.x * width;
  const T* bias = (const T*)bias_;
  const T* wp = (const T*)wp_;
  const T* wn = (const T*)wn_;
  float* xr = x + (size_t)blockIdx.x * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += 256) {
    const float v = ldf(o + i) + (bias ? ldf(bias + i) : 0.f);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  float s2 = 0.f;
  for (int i = threadIdx.x; i < width; i += 256) {
    const float v = ldf(o + i) + (bias ? ldf(bias + i) : 0.f);
    const float nx = xr[i] + mult * (v * inv * (1.0f + ldf(wp + i)));
    xr[i] = nx;
    s2 += nx * nx;
  }
  if (!wn) return;
  s2 = block_sum(s2, red);
  const float inv2 = 1.0f / sqrtf(s2 / (float)width + eps);
  T* h = (T*)h_ + (size_t)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += 256) stf(h + i, xr[i] * inv2 * (1.0f + ldf(wn + i)));
}

void sm_post_norm_add(uintptr_t x, uintptr_t o, uintptr_t bias, uintptr_t w_post, uintptr_t w_next, uintptr_t h,
                      int rows, int width, float eps, float mult, int f32, uintptr_t stream) {
  if (rows <= 0) return;
  DLLM_HOST_CHECK(width > 0 && (!w_next || h), "post_norm_add arguments");
  SM_DISPATCH(f32, sm_post_norm_add_kernel, dim3(rows), dim3(256), 0, stream, (float*)x, (const void*)o,
              (const void*)bias, (const void*)w_post, (const void*)w_next, (void*)h, width, eps, mult);
}

// --------------------------------------------------------------------------- causal convolution with state
// Input d rows before token (t, channel c) of a chunk that starts at position `start` with the token
// at local index tl: the batch row t - d while tl - d >= 0, else the state tail row
// tl - d + (taps - 1) while the position start + tl - d >= 0, else zero (before the sequence).
template <typename T>
__device__ __forceinline__ float conv_input(const T* __restrict__ u, long stride, const T* __restrict__ st, int t,
                                            int tl, int pos, int d, int taps, int c, int C, float in_bias) {
  if (d > pos) return 0.f;
  if (d <= tl) return ldf(u + (size_t)(t - d) * stride + c) + in_bias;
  return ldf(st + (size_t)(tl - d + taps - 1) * C + c) + in_bias;
}

template <typename T, typename OT>
__global__ void __launch_bounds__(256) sm_causal_conv_kernel(void* __restrict__ y_, const void* __restrict__ u_,
                                                             long stride, const void* __restrict__ w_,
                                                             const void* __restrict__ bias_,
                                                             const void* __restrict__ in_bias_,
                                                             const void* __restrict__ state_,
                                                             const int32_t* __restrict__ cu,
                                                             const int32_t* __restrict__ positions,
                                                             const int32_t* __restrict__ tok_seq,
                                                             const int32_t* __restrict__ slots, int C, int taps) {
  const int t = blockIdx.x;
  const int b = tok_seq[t];
  const int tl = t - cu[b], pos = positions[t];
  const T* u = (const T*)u_;
  const T* w = (const T*)w_;
  const T* st = (const T*)state_ + (size_t)slots[b] * (taps - 1) * C;
  const T* bias = (const T*)bias_;
  const T* in_bias = (const T*)in_bias_;
  OT* y = (OT*)y_ + (size_t)t * C;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < C; c += gridDim.y * 256) {
    const float ib = in_bias ? ldf(in_bias + c) : 0.f;
    float acc = bias ? ldf(bias + c) : 0.f;
    for (int j = 0; j < taps; ++j)
      acc += ldf(w + (size_t)c * taps + j) * conv_input(u, stride, st, t, tl, pos, taps - 1 - j, taps, c, C, ib);
    stf(y + c, acc);
  }
}

// New tail of every sequence: row j of the state becomes the input at position end - (taps - 1) + j
// (end = the chunk's last position + 1).  One thread per (sequence, channel) walks j upwards: row j
// of the old tail is read (as row j + n, n the chunk's length) only before it is overwritten.
template <typename T>
__global__ void __launch_bounds__(256) sm_conv_state_kernel(void* __restrict__ state_, const void* __restrict__ u_,
                                                            long stride, const int32_t* __restrict__ cu,
                                                            const int32_t* __restrict__ positions,
                                                            const int32_t* __restrict__ slots, int C, int taps) {
  const int b = blockIdx.x;
  const int lo = cu[b], n = cu[b + 1] - lo;
  if (n <= 0) return;
  const int start = positions[lo];
  T* st = (T*)state_ + (size_t)slots[b] * (taps - 1) * C;
  const T* u = (const T*)u_;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < C; c += gridDim.y * 256) {
    for (int j = 0; j < taps - 1; ++j) {
      const int tl = n - (taps - 1) + j;              // local index of the row that lands in tail row j
      float v;
      if (tl >= 0) v = ldf(u + (size_t)(lo + tl) * stride + c);
      else if (start + tl >= 0) v = ldf(st + (size_t)(j + n) * C + c);
      else v = 0.f;
      stf(st + (size_t)j * C + c, v);
    }
  }
}

void sm_causal_conv(uintptr_t y, uintptr_t u, long stride, uintptr_t w, uintptr_t bias, uintptr_t in_bias,
                    uintptr_t state, uintptr_t cu, uintptr_t positions, uintptr_t tok_seq, uintptr_t slots,
                    int tokens, int seqs, int C, int taps, int f32, int out_f32, uintptr_t stream) {
  if (tokens <= 0 || seqs <= 0) return;
  DLLM_HOST_CHECK(C > 0 && taps >= 1 && stride >= C, "conv sizes");
  const dim3 grid(tokens, std::min(8, (C + 255) / 256));
  hipStream_t s = (hipStream_t)stream;
#define SM_CONV(T, OT)                                                                                       \
  hipLaunchKernelGGL(HIP_KERNEL_NAME(sm_causal_conv_kernel<T, OT>), grid, dim3(256), 0, s, (void*)y, (const void*)u, \
                     stride, (const void*)w, (const void*)bias, (const void*)in_bias, (const void*)state,     \
                     (const int32_t*)cu, (const int32_t*)positions, (const int32_t*)tok_seq, (const int32_t*)slots, C, taps)
  if (f32) SM_CONV(float, float);
  else if (out_f32) SM_CONV(bf16, float);
  else SM_CONV(bf16, bf16);
#undef SM_CONV
  DLLM_HIP_CHECK(hipGetLastError());
  if (taps > 1)
    SM_DISPATCH(f32, sm_conv_state_kernel, dim3(seqs, std::min(8, (C + 255) / 256)), dim3(256), 0, stream,
                (void*)state, (const void*)u, stride, (const int32_t*)cu, (const int32_t*)positions,
                (const int32_t*)slots, C, taps);
}

// --------------------------------------------------------------------------- RG-LRU gates
// a = exp(-scale * sigmoid(Ra_b u_b + ra_b) * softplus(lam)),  g = sqrt(1 - a^2) * sigmoid(Ri_b u_b + ri_b) * u
// for GT tokens x one block of bw channels per workgroup; the token tile's u_b sits in LDS, the
// transposed gate matrices [nb, in, out] are read with consecutive lanes on consecutive outputs.
constexpr int GT = 8;

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplus_f(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

template <typename T>
__global__ void __launch_bounds__(256) sm_rglru_gates_kernel(float* __restrict__ a_out, float* __restrict__ g_out,
                                                             const float* __restrict__ u,
                                                             const void* __restrict__ ra_t_,
                                                             const void* __restrict__ ra_b_,
                                                             const void* __restrict__ ri_t_,
                                                             const void* __restrict__ ri_b_,
                                                             const void* __restrict__ lam_, int tokens, int nb, int bw,
                                                             float scale) {
  extern __shared__ float ub[];                       // [GT][bw]
  const int t0 = blockIdx.x * GT, b = blockIdx.y, C = nb * bw;
  const int nt = min(GT, tokens - t0);
  for (int i = threadIdx.x; i < GT * bw; i += 256) {
    const int k = i / bw, c = i - k * bw;
    ub[i] = k < nt ? u[(size_t)(t0 + k) * C + b * bw + c] : 0.f;
  }
  __syncthreads();
  const T* ra = (const T*)ra_t_ + (size_t)b * bw * bw;
  const T* ri = (const T*)ri_t_ + (size_t)b * bw * bw;
  for (int o = threadIdx.x; o < bw; o += 256) {
    float ar[GT], ai[GT];
    const float br = ldf((const T*)ra_b_ + b * bw + o), bi = ldf((const T*)ri_b_ + b * bw + o);
#pragma unroll
    for (int k = 0; k < GT; ++k) ar[k] = br, ai[k] = bi;
    for (int i = 0; i < bw; ++i) {
      const float wr = ldf(ra + (size_t)i * bw + o), wi = ldf(ri + (size_t)i * bw + o);
#pragma unroll
      for (int k = 0; k < GT; ++k) {
        const float x = ub[k * bw + i];
        ar[k] = fmaf(wr, x, ar[k]);
        ai[k] = fmaf(wi, x, ai[k]);
      }
    }
    const float sp = softplus_f(ldf((const T*)lam_ + b * bw + o));
#pragma unroll
    for (int k = 0; k < GT; ++k) {
      if (k < nt) {
        const float av = expf(-scale * sigmoid_f(ar[k]) * sp);
        const size_t idx = (size_t)(t0 + k) * C + b * bw + o;
        a_out[idx] = av;
        g_out[idx] = sqrtf(1.0f - av * av) * sigmoid_f(ai[k]) * ub[k * bw + o];
      }
    }
  }
}

void sm_rglru_gates(uintptr_t a, uintptr_t g, uintptr_t u, uintptr_t ra_t, uintptr_t ra_b, uintptr_t ri_t,
                    uintptr_t ri_b, uintptr_t lam, int tokens, int nb, int bw, float scale, int f32,
                    uintptr_t stream) {
  if (tokens <= 0) return;
  DLLM_HOST_CHECK(nb > 0 && bw > 0 && (size_t)GT * bw * 4 <= 160 * 1024 && nb <= 65535, "rglru gate sizes");
  const size_t lds = (size_t)GT * bw * sizeof(float);
  if (lds > 48 * 1024) {
    if (f32) DLLM_HIP_CHECK(hipFuncSetAttribute((const void*)sm_rglru_gates_kernel<float>,
                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    else DLLM_HIP_CHECK(hipFuncSetAttribute((const void*)sm_rglru_gates_kernel<bf16>,
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  }
  SM_DISPATCH(f32, sm_rglru_gates_kernel, dim3((tokens + GT - 1) / GT, nb), dim3(256), lds, stream, (float*)a,
              (float*)g, (const float*)u, (const void*)ra_t, (const void*)ra_b, (const void*)ri_t, (const void*)ri_b,
              (const void*)lam, tokens, nb, bw, scale);
}

// --------------------------------------------------------------------------- RG-LRU scan
// S_t = a_t S_(t-1) + g_t per (sequence, channel), from the slot's state (zero at position 0);
// out_t = S_t * gelu_tanh(y_raw_t + y_bias).  One thread per channel walks its sequence's chunk.
__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename T>
__global__ void __launch_bounds__(64) sm_rglru_scan_kernel(void* __restrict__ out_, const float* __restrict__ a,
                                                           const float* __restrict__ g,
                                                           const void* __restrict__ y_raw_, long y_stride,
                                                           const void* __restrict__ y_bias_,
                                                           float* __restrict__ state, const int32_t* __restrict__ cu,
                                                           const int32_t* __restrict__ positions,
                                                           const int32_t* __restrict__ slots, int C) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * 64 + threadIdx.x;
  const int lo = cu[b], hi = cu[b + 1];
  if (c >= C || hi <= lo) return;
  const T* y_raw = (const T*)y_raw_;
  T* out = (T*)out_;
  float* sp = state + (size_t)slots[b] * C + c;
  float s = positions[lo] > 0 ? *sp : 0.f;
  const float yb = ldf((const T*)y_bias_ + c);
  for (int t = lo; t < hi; ++t) {
    const size_t i = (size_t)t * C + c;
    s = fmaf(a[i], s, g[i]);
    stf(out + i, s * gelu_tanh_f(ldf(y_raw + (size_t)t * y_stride + c) + yb));
  }
  *sp = s;
}

void sm_rglru_scan(uintptr_t out, uintptr_t a, uintptr_t g, uintptr_t y_raw, long y_stride, uintptr_t y_bias,
                   uintptr_t state, uintptr_t cu, uintptr_t positions, uintptr_t slots, int seqs, int C, int max_q_len,
                   int f32, uintptr_t stream) {
  if (seqs <= 0) return;
  DLLM_HOST_CHECK(C > 0 && y_stride >= C && seqs <= 65535, "rglru scan sizes");
  SM_DISPATCH(f32, sm_rglru_scan_kernel, dim3((C + 63) / 64, seqs), dim3(64), 0, stream, (void*)out, (const float*)a,
              (const float*)g, (const void*)y_raw, y_stride, (const void*)y_bias, (float*)state, (const int32_t*)cu,
              (const int32_t*)positions, (const int32_t*)slots, C);
}

// --------------------------------------------------------------------------- clipped GLU
template <typename T>
__global__ void __launch_bounds__(256) sm_clipped_glu_kernel(void* __restrict__ out_, const void* __restrict__ gu_,
                                                             const void* __restrict__ bias_, long n, int F,
                                                             float limit, float alpha) {
  const T* gu = (const T*)gu_;
  const T* bias = (const T*)bias_;
  T* out = (T*)out_;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
    const long t = i / F;
    const int c = (int)(i - t * F);
    float gv = ldf(gu + t * 2 * F + c), uv = ldf(gu + t * 2 * F + F + c);
    if (bias) gv += ldf(bias + c), uv += ldf(bias + F + c);
    gv = fminf(gv, limit);
    uv = fminf(fmaxf(uv, -limit), limit);
    stf(out + i, gv * (1.0f / (1.0f + expf(-alpha * gv))) * (uv + 1.0f));
  }
}

void sm_clipped_glu(uintptr_t out, uintptr_t gu, uintptr_t bias, int tokens, int F, float limit, float alpha, int f32,
                    uintptr_t stream) {
  const long n = (long)tokens * F;
  if (n <= 0) return;
  const int grid = (int)std::min<long>((n + 255) / 256, 65535);
  SM_DISPATCH(f32, sm_clipped_glu_kernel, dim3(grid), dim3(256), 0, stream, (void*)out, (const void*)gu,
              (const void*)bias, n, F, limit, alpha);
}

// --------------------------------------------------------------------------- logit soft cap
template <typename T>
__global__ void __launch_bounds__(256) sm_softcap_kernel(float* __restrict__ out, const void* __restrict__ x_, long n,
                                                         float cap) {
  const T* x = (const T*)x_;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
    const float v = ldf(x + i);
    out[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
  }
}

void sm_softcap(uintptr_t out, uintptr_t x, long n, float cap, int f32, uintptr_t stream) {
  if (n <= 0) return;
  const int grid = (int)std::min<long>((n + 255) / 256, 65535);
  SM_DISPATCH(f32, sm_softcap_kernel, dim3(grid), dim3(256), 0, stream, (float*)out, (const void*)x, n, cap);
}

// --------------------------------------------------------------------------- attention input stage
// One wave per (token, head) of the fused projection [q heads | k heads | v heads]: the causal
// convolution of the head's channels, then for q / k the RMS norm over the head (plain weight) and
// the rotation of pairs (2i, 2i + 1), i < nrot, by pos * freqs[i] (cos and sin scaled by mag);
// q goes to q_out [T, H, D], k / v to the paged caches [NB, G, BS, D] / [NB, G, Dv, BS] (V transposed
// inside a block).
template <typename T>
__global__ void __launch_bounds__(64) sm_attn_prep_kernel(
    void* __restrict__ q_out_, const void* __restrict__ qkv_, const void* __restrict__ conv_w_,
    const void* __restrict__ state_, const void* __restrict__ q_norm_, const void* __restrict__ k_norm_,
    const float* __restrict__ freqs, int nrot, float mag, float eps, void* __restrict__ k_cache_,
    void* __restrict__ v_cache_, const int32_t* __restrict__ slot_mapping, const int32_t* __restrict__ cu,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ slots,
    int H, int G, int D, int Dv, int taps, int bs) {
  extern __shared__ float hv[];                      // the head's values [max(D, Dv)]
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int C = H * D + G * (D + Dv);
  const int b = tok_seq[t];
  const int tl = t - cu[b], pos = positions[t];
  const T* qkv = (const T*)qkv_;
  const T* w = (const T*)conv_w_;
  const T* st = (const T*)state_ + (size_t)slots[b] * (taps - 1) * C;
  // channel range and kind of this head
  int c0, n, kind;                                   // kind 0 q, 1 k, 2 v
  if (head < H) c0 = head * D, n = D, kind = 0;
  else if (head < H + G) c0 = H * D + (head - H) * D, n = D, kind = 1;
  else c0 = H * D + G * D + (head - H - G) * Dv, n = Dv, kind = 2;
  float ss = 0.f;
  for (int e = lane; e < n; e += 64) {
    const int c = c0 + e;
    float acc = 0.f;
    for (int j = 0; j < taps; ++j)
      acc += ldf(w + (size_t)c * taps + j) * conv_input(qkv, (long)C, st, t, tl, pos, taps - 1 - j, taps, c, C, 0.f);
    hv[e] = acc;
    ss += acc * acc;
  }
  T* dst;
  if (kind == 0) dst = (T*)q_out_ + ((size_t)t * H + head) * D;
  else {
    const int slot = slot_mapping[t];
    const int blk = slot / bs, off = slot - blk * bs;
    if (kind == 1) dst = (T*)k_cache_ + (((size_t)blk * G + (head - H)) * bs + off) * D;
    else dst = (T*)v_cache_ + ((size_t)blk * G + (head - H - G)) * Dv * bs + off;
  }
  if (kind == 2) {
    for (int e = lane; e < n; e += 64) stf(dst + (size_t)e * bs, hv[e]);
    return;
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)n + eps);
  const T* nw = (const T*)(kind == 0 ? q_norm_ : k_norm_);
  __syncthreads();
  for (int e = lane; e < n; e += 64) hv[e] = hv[e] * inv * ldf(nw + e);
  __syncthreads();
  const float fpos = (float)pos;
  for (int i = lane; 2 * i < n; i += 64) {
    float x0 = hv[2 * i], x1 = 2 * i + 1 < n ? hv[2 * i + 1] : 0.f;
    if (i < nrot) {
      const float ang = fpos * freqs[i];
      const float cs = cosf(ang) * mag, sn = sinf(ang) * mag;
      const float r0 = x0 * cs - x1 * sn, r1 = x1 * cs + x0 * sn;
      x0 = r0, x1 = r1;
    }
    stf(dst + 2 * i, x0);
    if (2 * i + 1 < n) stf(dst + 2 * i + 1, x1);
  }
}

void sm_attn_prep(uintptr_t q_out, uintptr_t qkv, uintptr_t conv_w, uintptr_t state, uintptr_t q_norm,
                  uintptr_t k_norm, uintptr_t freqs, int nrot, float mag, float eps, uintptr_t k_cache,
                  uintptr_t v_cache, uintptr_t slot_mapping, uintptr_t cu, uintptr_t positions, uintptr_t tok_seq,
                  uintptr_t slots, int tokens, int seqs, int H, int G, int D, int Dv, int taps, int bs, int f32,
                  uintptr_t stream) {
  if (tokens <= 0 || seqs <= 0) return;
  DLLM_HOST_CHECK(H > 0 && G >= 0 && D > 0 && Dv > 0 && taps >= 1 && bs > 0 && 2 * nrot <= D, "attn_prep sizes");
  DLLM_HOST_CHECK(G == 0 || (k_cache && v_cache && k_norm), "attn_prep caches");
  DLLM_HOST_CHECK(H + 2 * G <= 65535, "attn_prep heads");
  const int C = H * D + G * (D + Dv);
  const size_t lds = (size_t)std::max(D, Dv) * sizeof(float);
  SM_DISPATCH(f32, sm_attn_prep_kernel, dim3(tokens, H + 2 * G), dim3(64), lds, stream, (void*)q_out, (const void*)qkv,
              (const void*)conv_w, (const void*)state, (const void*)q_norm, (const void*)k_norm, (const float*)freqs,
              nrot, mag, eps, (void*)k_cache, (void*)v_cache, (const int32_t*)slot_mapping, (const int32_t*)cu,
              (const int32_t*)positions, (const int32_t*)tok_seq, (const int32_t*)slots, H, G, D, Dv, taps, bs);
  // the projection's last taps - 1 rows of every sequence become its new tail
  if (taps > 1)
    SM_DISPATCH(f32, sm_conv_state_kernel, dim3(seqs, std::min(8, (C + 255) / 256)), dim3(256), 0, stream,
                (void*)state, (const void*)qkv, (long)C, (const int32_t*)cu, (const int32_t*)positions,
                (const int32_t*)slots, C, taps);
}

}  // namespace dllm
