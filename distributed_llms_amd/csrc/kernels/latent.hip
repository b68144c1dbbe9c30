// Kernels of latent attention and of parallel layers on a float32 residual stream (ops/latent.py).
//
// Latent attention caches one small vector per token: the RMS-normed latent c [rank] that every
// head's keys and values are up-projections of, and optionally one rotated key part [rot_dim] that all
// heads share.  With the key up-projection folded into the query (q~_h = Wuk_h^T q_h) a head's score
// is q~_h . c + q_rot_h . k_rot, and its output Wuv_h (sum_j p_j c_j): attention over ONE shared
// K/V head of width rank + rot_dim (keys) / rank (values), which the paged window-attention kernels
// run.  The cache holds the latent in the two layouts those kernels read: k [NB, 1, BS, rank + rot_dim]
// (row per key: latent | rotated part) and v [NB, 1, rank, BS] (transposed inside a block).
//
//   lat_prep       per token: RMS norm of the query latent -> cq; RMS norm of the key/value latent and
//                  the interleaved-pair rotation of the shared key part, appended to both caches
//   lat_q_pack     per token: [H, T, rank] folded queries + the rotated part of q -> q~ [T, H, rank + rot_dim]
//   lat_head_gate  [H, T, vdim] head outputs x sigmoid(gate[t, h]) -> [T, H * vdim]
//   par_add        x += a (+ b) on the float32 stream, optionally also the stream rounded to T
//   stream_cat     [x | x0] rounded to T (input of a projection of two streams); stream_set: x = (float)a
//   side_gate      gelu_tanh(z) * table[token, off : off + dim]
//   silu_glu       silu(gate) * up of a fused gate | up projection
//
// Every kernel is a template over the activation type T (bf16 or float); norms, angles and gates
// are float32 in both.  Sizes are runtime values.
#include <math.h>

#include "common.h"
#include "launchers.h"
#include "stream_common.h"

namespace dllm {

// --------------------------------------------------------------------------- latent input stage
template <typename T>
__global__ void __launch_bounds__(256) lat_prep_kernel(
    void* __restrict__ cq_, const void* __restrict__ down_, long ld, int q_off, int q_rank,
    const void* __restrict__ qn_w_, int c_off, int rank, const void* __restrict__ cn_w_, int r_off, int rot_dim,
    const float* __restrict__ freqs, int nfreq, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ slot_mapping, void* __restrict__ k_cache_, void* __restrict__ v_cache_, int bs,
    float eps) {
  __shared__ float red[16];
  const int t = blockIdx.x, tid = threadIdx.x;
  const T* row = (const T*)down_ + (size_t)t * ld;
  float sq = 0.f, sc = 0.f;
  for (int i = tid; i < q_rank; i += 256) {
    const float v = ldf(row + q_off + i);
    sq += v * v;
  }
  for (int i = tid; i < rank; i += 256) {
    const float v = ldf(row + c_off + i);
    sc += v * v;
  }
  sq = block_sum(sq, red);
  sc = block_sum(sc, red);
  if (q_rank > 0) {
    const float inv = 1.0f / sqrtf(sq / (float)q_rank + eps);
    T* cq = (T*)cq_ + (size_t)t * q_rank;
    const T* w = (const T*)qn_w_;
    for (int i = tid; i < q_rank; i += 256) stf(cq + i, ldf(row + q_off + i) * inv * ldf(w + i));
  }
  const int slot = slot_mapping[t];
  const int blk = slot / bs, off = slot - blk * bs;
  const int D = rank + rot_dim;
  T* krow = (T*)k_cache_ + ((size_t)blk * bs + off) * D;
  T* vblk = (T*)v_cache_ + (size_t)blk * rank * bs + off;
  const float inv = 1.0f / sqrtf(sc / (float)rank + eps);
  const T* w = (const T*)cn_w_;
  for (int i = tid; i < rank; i += 256) {
    T c;
    stf(&c, ldf(row + c_off + i) * inv * ldf(w + i));
    krow[i] = c;
    vblk[(size_t)i * bs] = c;
  }
  const float pos = (float)positions[t];
  for (int i = tid; i < rot_dim / 2; i += 256) {
    const float u = ldf(row + r_off + 2 * i), v = ldf(row + r_off + 2 * i + 1);
    float a = u, b = v;
    if (i < nfreq) {
      const float ang = pos * freqs[i];
      const float c = cosf(ang), s = sinf(ang);
      a = u * c - v * s;
      b = v * c + u * s;
    }
    stf(krow + rank + 2 * i, a);
    stf(krow + rank + 2 * i + 1, b);
  }
  if ((rot_dim & 1) && tid == 0) krow[D - 1] = row[r_off + rot_dim - 1];
}

void lat_prep(uintptr_t cq, uintptr_t down, long ld, int q_off, int q_rank, uintptr_t qn_w, int c_off, int rank,
              uintptr_t cn_w, int r_off, int rot_dim, uintptr_t freqs, int nfreq, uintptr_t positions,
              uintptr_t slot_mapping, uintptr_t k_cache, uintptr_t v_cache, int bs, float eps, int tokens, int f32,
              uintptr_t stream) {
  if (tokens <= 0) return;
  DLLM_HOST_CHECK(rank > 0 && q_rank >= 0 && rot_dim >= 0 && bs > 0 && 2 * nfreq <= rot_dim, "latent sizes");
  DLLM_HOST_CHECK(q_off >= 0 && q_off + q_rank <= ld && c_off >= 0 && c_off + rank <= ld && r_off >= 0 &&
                      r_off + rot_dim <= ld,
                  "latent row layout");
  DLLM_HOST_CHECK((q_rank == 0 || (cq && qn_w)) && cn_w && k_cache && v_cache && (nfreq == 0 || freqs),
                  "latent arguments");
  SM_DISPATCH(f32, lat_prep_kernel, dim3(tokens), dim3(256), 0, stream, (void*)cq, (const void*)down, ld, q_off,
              q_rank, (const void*)qn_w, c_off, rank, (const void*)cn_w, r_off, rot_dim, (const float*)freqs, nfreq,
              (const int32_t*)positions, (const int32_t*)slot_mapping, (void*)k_cache, (void*)v_cache, bs, eps);
}

// q~ [T, H, rank + rot_dim] from qa [H, T, rank] (queries with the key up-projection folded in) and
// the rotated part of q [T, H, dim + rot_dim].  One workgroup per token: first the folded parts of all
// heads, V elements per lane and step (V = 8 needs rank and rot_dim in multiples of 8), then the
// rotation pairs of all heads, a pair per lane.
template <typename T, int V>
__global__ void __launch_bounds__(256) lat_q_pack_kernel(void* __restrict__ out_, const void* __restrict__ qa_,
                                                         const void* __restrict__ q_, int tokens, int H, int rank,
                                                         int dim, int rot_dim, const float* __restrict__ freqs,
                                                         int nfreq, const int32_t* __restrict__ positions) {
  const int t = blockIdx.x;
  const int D = rank + rot_dim, dq = dim + rot_dim;
  T* out = (T*)out_ + (size_t)t * H * D;
  const T* qa = (const T*)qa_ + (size_t)t * rank;
  const T* q = (const T*)q_ + (size_t)t * H * dq + dim;
  const int cpr = rank / V;                                  // chunks per head
  for (int idx = threadIdx.x; idx < H * cpr; idx += 256) {
    const int h = idx / cpr, c = idx - h * cpr;
    float v[V];
    ldv<V>(qa + (size_t)h * tokens * rank + c * V, v);
    stv<V>(out + h * D + c * V, v);
  }
  const float pos = (float)positions[t];
  const int ppr = (rot_dim + 1) / 2;                         // pairs per head (a last single element counts as one)
  for (int idx = threadIdx.x; idx < H * ppr; idx += 256) {
    const int h = idx / ppr, i = idx - h * ppr;
    const T* qr = q + h * dq + 2 * i;
    T* o = out + h * D + rank + 2 * i;
    const float u = ldf(qr);
    if (2 * i + 1 >= rot_dim) {
      stf(o, u);
      continue;
    }
    const float w = ldf(qr + 1);
    float a = u, b2 = w;
    if (i < nfreq) {
      const float ang = pos * freqs[i];
      const float c = cosf(ang), s = sinf(ang);
      a = u * c - w * s;
      b2 = w * c + u * s;
    }
    stf(o, a);
    stf(o + 1, b2);
  }
}

void lat_q_pack(uintptr_t out, uintptr_t qa, uintptr_t q, int tokens, int H, int rank, int dim, int rot_dim,
                uintptr_t freqs, int nfreq, uintptr_t positions, int f32, uintptr_t stream) {
  if (tokens <= 0) return;
  DLLM_HOST_CHECK(H > 0 && rank > 0 && dim >= 0 && rot_dim >= 0 && 2 * nfreq <= rot_dim, "latent query sizes");
  DLLM_HOST_CHECK(out && qa && (rot_dim == 0 || q) && (nfreq == 0 || freqs), "latent query arguments");
  SM_DISPATCH_V(f32, rank % 8 == 0 && rot_dim % 8 == 0, lat_q_pack_kernel, dim3(tokens), dim3(256), 0, stream,
                (void*)out, (const void*)qa, (const void*)q, tokens, H, rank, dim, rot_dim, (const float*)freqs, nfreq,
                (const int32_t*)positions);
}

// Few tokens (decode steps): the per-head products themselves, one workgroup per (token, head), instead
// of a library batched product plus a pack / gate launch.
//   lat_q_fold    q~[t, h] = [ q[t, h, :dim] . Wuk[h] ([dim, rank])  |  rotated q[t, h, dim:] ]
//   lat_v_unfold  out[t, h] = (o_lat[t, h] . WuvT[h] ([rank, vdim])) * sigmoid(gate[t, h])
// Consecutive threads own consecutive output columns, so every weight row is read in whole lines; the
// token's vector sits in LDS as float; sums are float32.
template <typename T>
__global__ void __launch_bounds__(256) lat_q_fold_kernel(void* __restrict__ out_, const void* __restrict__ q_,
                                                         const void* __restrict__ wuk_, int H, int rank, int dim,
                                                         int rot_dim, const float* __restrict__ freqs, int nfreq,
                                                         const int32_t* __restrict__ positions) {
  extern __shared__ float qs[];                              // [dim]
  const int t = blockIdx.x, h = blockIdx.y;
  const int D = rank + rot_dim, dq = dim + rot_dim;
  T* out = (T*)out_ + ((size_t)t * H + h) * D;
  const T* q = (const T*)q_ + ((size_t)t * H + h) * dq;
  const T* w = (const T*)wuk_ + (size_t)h * dim * rank;
  for (int d = threadIdx.x; d < dim; d += 256) qs[d] = ldf(q + d);
  __syncthreads();
  for (int j = threadIdx.x; j < rank; j += 256) {
    float acc = 0.f;
    for (int d = 0; d < dim; ++d) acc = fmaf(qs[d], ldf(w + (size_t)d * rank + j), acc);
    stf(out + j, acc);
  }
  const float pos = (float)positions[t];
  for (int i = threadIdx.x; i < (rot_dim + 1) / 2; i += 256) {
    const T* qr = q + dim + 2 * i;
    T* o = out + rank + 2 * i;
    const float u = ldf(qr);
    if (2 * i + 1 >= rot_dim) {
      stf(o, u);
      continue;
    }
    const float v = ldf(qr + 1);
    float a = u, b = v;
    if (i < nfreq) {
      const float ang = pos * freqs[i];
      const float c = cosf(ang), s = sinf(ang);
      a = u * c - v * s;
      b = v * c + u * s;
    }
    stf(o, a);
    stf(o + 1, b);
  }
}

// bf16 with 8 | rank: a thread owns 8 consecutive outputs (16-byte weight loads) and every ng-th input
// row; the ng partial sums of an output meet in LDS.
__global__ void __launch_bounds__(256) lat_q_fold_vec_kernel(bf16* __restrict__ out_, const bf16* __restrict__ q_,
                                                             const bf16* __restrict__ wuk, int H, int rank, int dim,
                                                             int rot_dim, const float* __restrict__ freqs, int nfreq,
                                                             const int32_t* __restrict__ positions, int ng) {
  extern __shared__ float sm[];
  float* qs = sm;                                            // [dim]
  float* red = sm + dim;                                     // [ng][rank]
  const int t = blockIdx.x, h = blockIdx.y;
  const int D = rank + rot_dim, dq = dim + rot_dim;
  bf16* out = out_ + ((size_t)t * H + h) * D;
  const bf16* q = q_ + ((size_t)t * H + h) * dq;
  const bf16* w = wuk + (size_t)h * dim * rank;
  for (int d = threadIdx.x; d < dim; d += 256) qs[d] = bf2f(q[d]);
  __syncthreads();
  const int nc = rank >> 3, c = threadIdx.x % nc, g = threadIdx.x / nc;
  if (g < ng) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int d = g; d < dim; d += ng) {
      const bf16x8 w8 = *reinterpret_cast<const bf16x8*>(w + (size_t)d * rank + 8 * c);
      const float qv = qs[d];
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = fmaf(qv, bf2f(w8[i]), acc[i]);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) red[g * rank + 8 * c + i] = acc[i];
  }
  __syncthreads();
  for (int j = threadIdx.x; j < rank; j += 256) {
    float s = 0.f;
    for (int g2 = 0; g2 < ng; ++g2) s += red[g2 * rank + j];
    out[j] = f2bf(s);
  }
  const float pos = (float)positions[t];
  for (int i = threadIdx.x; i < (rot_dim + 1) / 2; i += 256) {
    const bf16* qr = q + dim + 2 * i;
    bf16* o = out + rank + 2 * i;
    const float u = bf2f(qr[0]);
    if (2 * i + 1 >= rot_dim) {
      o[0] = f2bf(u);
      continue;
    }
    const float v = bf2f(qr[1]);
    float a = u, b = v;
    if (i < nfreq) {
      const float ang = pos * freqs[i];
      const float cs = cosf(ang), sn = sinf(ang);
      a = u * cs - v * sn;
      b = v * cs + u * sn;
    }
    o[0] = f2bf(a);
    o[1] = f2bf(b);
  }
}

// groups of input rows for the vector forms: as many as 256 threads allow, at most one per input row
static int fold_groups(int out_width, int in_width) { return std::max(1, std::min(256 / (out_width / 8), in_width)); }

void lat_q_fold(uintptr_t out, uintptr_t q, uintptr_t wuk, int tokens, int H, int rank, int dim, int rot_dim,
                uintptr_t freqs, int nfreq, uintptr_t positions, int f32, uintptr_t stream) {
  if (tokens <= 0) return;
  DLLM_HOST_CHECK(H > 0 && H <= 65535 && rank > 0 && dim > 0 && dim <= 8192 && rot_dim >= 0 && 2 * nfreq <= rot_dim,
                  "latent query sizes");
  DLLM_HOST_CHECK(out && q && wuk && (nfreq == 0 || freqs), "latent query arguments");
  if (!f32 && rank % 8 == 0 && rank <= 2048) {
    const int ng = fold_groups(rank, dim);
    hipLaunchKernelGGL(lat_q_fold_vec_kernel, dim3(tokens, H), dim3(256), sizeof(float) * ((size_t)dim + (size_t)ng * rank),
                       (hipStream_t)stream, (bf16*)out, (const bf16*)q, (const bf16*)wuk, H, rank, dim, rot_dim,
                       (const float*)freqs, nfreq, (const int32_t*)positions, ng);
    DLLM_HIP_CHECK(hipGetLastError());
    return;
  }
  SM_DISPATCH(f32, lat_q_fold_kernel, dim3(tokens, H), dim3(256), sizeof(float) * dim, stream, (void*)out,
              (const void*)q, (const void*)wuk, H, rank, dim, rot_dim, (const float*)freqs, nfreq,
              (const int32_t*)positions);
}

template <typename T>
__global__ void __launch_bounds__(256) lat_v_unfold_kernel(void* __restrict__ out_, const void* __restrict__ o_,
                                                           const void* __restrict__ wuv_t_,
                                                           const void* __restrict__ gate_, long ld, int H, int rank,
                                                           int vdim) {
  extern __shared__ float os[];                              // [rank]
  const int t = blockIdx.x, h = blockIdx.y;
  T* out = (T*)out_ + ((size_t)t * H + h) * vdim;
  const T* o = (const T*)o_ + ((size_t)t * H + h) * rank;
  const T* w = (const T*)wuv_t_ + (size_t)h * rank * vdim;
  const T* gate = (const T*)gate_;
  for (int r = threadIdx.x; r < rank; r += 256) os[r] = ldf(o + r);
  __syncthreads();
  const float g = gate ? 1.0f / (1.0f + expf(-ldf(gate + (size_t)t * ld + h))) : 1.0f;
  for (int e = threadIdx.x; e < vdim; e += 256) {
    float acc = 0.f;
    for (int r = 0; r < rank; ++r) acc = fmaf(os[r], ldf(w + (size_t)r * vdim + e), acc);
    // the product is rounded to the activation type before the gate, like the batched product it stands for
    T y;
    stf(&y, acc);
    stf(out + e, ldf(&y) * g);
  }
}

__global__ void __launch_bounds__(256) lat_v_unfold_vec_kernel(bf16* __restrict__ out_, const bf16* __restrict__ o_,
                                                               const bf16* __restrict__ wuv_t,
                                                               const bf16* __restrict__ gate, long ld, int H, int rank,
                                                               int vdim, int ng) {
  extern __shared__ float sm[];
  float* os = sm;                                            // [rank]
  float* red = sm + rank;                                    // [ng][vdim]
  const int t = blockIdx.x, h = blockIdx.y;
  bf16* out = out_ + ((size_t)t * H + h) * vdim;
  const bf16* o = o_ + ((size_t)t * H + h) * rank;
  const bf16* w = wuv_t + (size_t)h * rank * vdim;
  for (int r = threadIdx.x; r < rank; r += 256) os[r] = bf2f(o[r]);
  __syncthreads();
  const int nc = vdim >> 3, c = threadIdx.x % nc, g = threadIdx.x / nc;
  if (g < ng) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int r = g; r < rank; r += ng) {
      const bf16x8 w8 = *reinterpret_cast<const bf16x8*>(w + (size_t)r * vdim + 8 * c);
      const float ov = os[r];
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = fmaf(ov, bf2f(w8[i]), acc[i]);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) red[g * vdim + 8 * c + i] = acc[i];
  }
  __syncthreads();
  const float gt = gate ? 1.0f / (1.0f + expf(-bf2f(gate[(size_t)t * ld + h]))) : 1.0f;
  for (int e = threadIdx.x; e < vdim; e += 256) {
    float s = 0.f;
    for (int g2 = 0; g2 < ng; ++g2) s += red[g2 * vdim + e];
    out[e] = f2bf(bf2f(f2bf(s)) * gt);           // rounded before the gate, like the batched product it stands for
  }
}

void lat_v_unfold(uintptr_t out, uintptr_t o, uintptr_t wuv_t, uintptr_t gate, long ld, int tokens, int H, int rank,
                  int vdim, int f32, uintptr_t stream) {
  if (tokens <= 0) return;
  DLLM_HOST_CHECK(H > 0 && H <= 65535 && rank > 0 && rank <= 8192 && vdim > 0 && out && o && wuv_t,
                  "latent value arguments");
  if (!f32 && vdim % 8 == 0 && vdim <= 2048) {
    const int ng = fold_groups(vdim, rank);
    hipLaunchKernelGGL(lat_v_unfold_vec_kernel, dim3(tokens, H), dim3(256),
                       sizeof(float) * ((size_t)rank + (size_t)ng * vdim), (hipStream_t)stream, (bf16*)out,
                       (const bf16*)o, (const bf16*)wuv_t, (const bf16*)gate, ld, H, rank, vdim, ng);
    DLLM_HIP_CHECK(hipGetLastError());
    return;
  }
  SM_DISPATCH(f32, lat_v_unfold_kernel, dim3(tokens, H), dim3(256), sizeof(float) * rank, stream, (void*)out,
              (const void*)o, (const void*)wuv_t, (const void*)gate, ld, H, rank, vdim);
}

// out [T, H * vdim] = o [H, T, vdim] * sigmoid(gate[t * ld + h]) (gate null: a plain transposing copy);
// one workgroup per (token, head)
template <typename T, int V>
__global__ void __launch_bounds__(64) lat_head_gate_kernel(void* __restrict__ out_, const void* __restrict__ o_,
                                                           const void* __restrict__ gate_, long ld, int tokens, int H,
                                                           int vdim) {
  const int t = blockIdx.x, h = blockIdx.y;
  T* out = (T*)out_ + ((size_t)t * H + h) * vdim;
  const T* o = (const T*)o_ + ((size_t)h * tokens + t) * vdim;
  const T* gate = (const T*)gate_;
  const float g = gate ? 1.0f / (1.0f + expf(-ldf(gate + (size_t)t * ld + h))) : 1.0f;
  for (int e = threadIdx.x * V; e < vdim; e += 64 * V) {
    float v[V];
    ldv<V>(o + e, v);
#pragma unroll
    for (int j = 0; j < V; ++j) v[j] *= g;
    stv<V>(out + e, v);
  }
}

void lat_head_gate(uintptr_t out, uintptr_t o, uintptr_t gate, long ld, int tokens, int H, int vdim, int f32,
                   uintptr_t stream) {
  if (tokens <= 0) return;
  DLLM_HOST_CHECK(H > 0 && H <= 65535 && vdim > 0 && out && o, "head gate arguments");
  SM_DISPATCH_V(f32, vdim % 8 == 0, lat_head_gate_kernel, dim3(tokens, H), dim3(64), 0, stream, (void*)out,
                (const void*)o, (const void*)gate, ld, tokens, H, vdim);
}

// --------------------------------------------------------------------------- parallel layer: x += a + b
template <typename T, int V>
__global__ void __launch_bounds__(256) par_add_kernel(float* __restrict__ x, const void* __restrict__ a_,
                                                      const void* __restrict__ b_, void* __restrict__ xr_, long n) {
  const T* a = (const T*)a_;
  const T* b = (const T*)b_;
  T* xr = (T*)xr_;
  for (long i = ((long)blockIdx.x * 256 + threadIdx.x) * V; i < n; i += (long)gridDim.x * 256 * V) {
    float xv[V], av[V];
    ldv<V>(x + i, xv);
    ldv<V>(a + i, av);
    if (b) {
      float bv[V];
      ldv<V>(b + i, bv);
#pragma unroll
      for (int j = 0; j < V; ++j) av[j] += bv[j];
    }
#pragma unroll
    for (int j = 0; j < V; ++j) xv[j] += av[j];
    stv<V>(x + i, xv);
    if (xr) stv<V>(xr + i, xv);
  }
}

static int flat_grid(long n, int per_thread) {
  const long blocks = (n + 256L * per_thread - 1) / (256L * per_thread);
  return (int)std::min<long>(std::max<long>(blocks, 1), 256L * 32);
}

void par_add(uintptr_t x, uintptr_t a, uintptr_t b, uintptr_t x_rounded, long n, int f32, uintptr_t stream) {
  if (n <= 0) return;
  DLLM_HOST_CHECK(x && a, "par_add arguments");
  const bool vec = n % 8 == 0;
  SM_DISPATCH_V(f32, vec, par_add_kernel, dim3(flat_grid(n, vec ? 8 : 1)), dim3(256), 0, stream, (float*)x,
                (const void*)a, (const void*)b, (void*)x_rounded, n);
}

// out [T, 2 W] = [x | x0] rounded to T
template <typename T>
__global__ void __launch_bounds__(256) stream_cat_kernel(void* __restrict__ out_, const float* __restrict__ x,
                                                         const float* __restrict__ x0, int width) {
  T* out = (T*)out_ + (size_t)blockIdx.x * 2 * width;
  const float* a = x + (size_t)blockIdx.x * width;
  const float* b = x0 + (size_t)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += 256) {
    stf(out + i, a[i]);
    stf(out + width + i, b[i]);
  }
}

void stream_cat(uintptr_t out, uintptr_t x, uintptr_t x0, int rows, int width, int f32, uintptr_t stream) {
  if (rows <= 0) return;
  DLLM_HOST_CHECK(width > 0 && out && x && x0, "stream_cat arguments");
  SM_DISPATCH(f32, stream_cat_kernel, dim3(rows), dim3(256), 0, stream, (void*)out, (const float*)x, (const float*)x0,
              width);
}

template <typename T>
__global__ void __launch_bounds__(256) stream_set_kernel(float* __restrict__ x, const void* __restrict__ a_, long n) {
  const T* a = (const T*)a_;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) x[i] = ldf(a + i);
}

void stream_set(uintptr_t x, uintptr_t a, long n, int f32, uintptr_t stream) {
  if (n <= 0) return;
  DLLM_HOST_CHECK(x && a, "stream_set arguments");
  SM_DISPATCH(f32, stream_set_kernel, dim3(flat_grid(n, 1)), dim3(256), 0, stream, (float*)x, (const void*)a, n);
}

// out [T, F] = silu(gu[:, :F]) * gu[:, F:]  (the unfused SwiGLU of shapes and types the GEMM epilogue does not take)
template <typename T>
__global__ void __launch_bounds__(256) silu_glu_kernel(void* __restrict__ out_, const void* __restrict__ gu_, int F,
                                                       long n) {
  T* out = (T*)out_;
  const T* gu = (const T*)gu_;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
    const long t = i / F;
    const int c = (int)(i - t * F);
    const float g = ldf(gu + t * 2 * F + c), u = ldf(gu + t * 2 * F + F + c);
    stf(out + i, g / (1.0f + expf(-g)) * u);
  }
}

void silu_glu(uintptr_t out, uintptr_t gu, int tokens, int F, int f32, uintptr_t stream) {
  if (tokens <= 0) return;
  DLLM_HOST_CHECK(F > 0 && out && gu, "silu_glu arguments");
  const long n = (long)tokens * F;
  SM_DISPATCH(f32, silu_glu_kernel, dim3(flat_grid(n, 1)), dim3(256), 0, stream, (void*)out, (const void*)gu, F, n);
}

// --------------------------------------------------------------------------- per-layer token input gate
// g [T, dim] = gelu_tanh(z [T, dim]) * table[ids[t], off : off + dim]   (table rows of `total` elements)
template <typename T>
__global__ void __launch_bounds__(256) side_gate_kernel(void* __restrict__ g_, const void* __restrict__ z_,
                                                        const void* __restrict__ table_,
                                                        const int32_t* __restrict__ ids, int vocab, int total, int off,
                                                        int dim, long n) {
  T* g = (T*)g_;
  const T* z = (const T*)z_;
  const T* table = (const T*)table_;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
    const long t = i / dim;
    const int j = (int)(i - t * dim);
    int id = ids[t];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const float v = ldf(z + i);
    const float act = 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    stf(g + i, act * ldf(table + (size_t)id * total + off + j));
  }
}

void side_gate(uintptr_t g, uintptr_t z, uintptr_t table, uintptr_t ids, int tokens, int vocab, int total, int off,
               int dim, int f32, uintptr_t stream) {
  if (tokens <= 0) return;
  DLLM_HOST_CHECK(dim > 0 && off >= 0 && off + dim <= total && vocab > 0 && g && z && table && ids, "side_gate arguments");
  const long n = (long)tokens * dim;
  SM_DISPATCH(f32, side_gate_kernel, dim3(flat_grid(n, 1)), dim3(256), 0, stream, (void*)g, (const void*)z,
              (const void*)table, (const int32_t*)ids, vocab, total, off, dim, n);
}

}  // namespace dllm
