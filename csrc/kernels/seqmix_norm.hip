// fp32 residual stream: scaled embedding + norm, sublayer sum + residual add + next norm,
// activations, partial rotary with multi-map heads + paged K / V^T write.
//
// The residual stream x is fp32 whatever the activation type T (bf16 bits or float); norms
// are x / sqrt(mean(x^2) + eps) * (w_offset + w) with fp32 weights, rounded once to T.
#include "seqmix_common.h"

namespace {

constexpr int NT = 256;

__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) red[w] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NT / 64; ++i) t += red[i];
  return t;
}

template <typename T>
__global__ __launch_bounds__(NT) void embed_scale_norm_kernel(const int* __restrict__ tokens, const T* __restrict__ table,
                                                              float scale, const float* __restrict__ w, float eps,
                                                              float w_offset, float* __restrict__ resid,
                                                              T* __restrict__ out, int W, int vocab) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x;
  int tok = tokens[t];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  const T* row = table + static_cast<size_t>(tok) * W;
  float* x = resid + static_cast<size_t>(t) * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += NT) {
    const float v = Elem<T>::ld(row[i]) * scale;
    x[i] = v;
    ss += v * v;
  }
  const float r = 1.0f / sqrtf(block_sum(ss, red) / W + eps);
  T* o = out + static_cast<size_t>(t) * W;
  for (int i = threadIdx.x; i < W; i += NT) o[i] = Elem<T>::st(x[i] * r * (w_offset + w[i]));
}

// x += (p0 + p1 + pf + sigmoid(gate) * pg); out = norm(x) (w == nullptr: no norm).
template <typename T>
__global__ __launch_bounds__(NT) void residual_norm_kernel(float* __restrict__ resid, const T* __restrict__ p0,
                                                           const T* __restrict__ p1, const float* __restrict__ pf,
                                                           const float* __restrict__ gate, const T* __restrict__ pg,
                                                           const float* __restrict__ w, float eps, float w_offset,
                                                           T* __restrict__ out, int W) {
  __shared__ float red[NT / 64];
  const size_t base = static_cast<size_t>(blockIdx.x) * W;
  float* x = resid + base;
  float g = 0.f;
  if (pg != nullptr) g = 1.0f / (1.0f + expf(-gate[blockIdx.x]));
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += NT) {
    float s = 0.f;
    if (p0 != nullptr) s = Elem<T>::ld(p0[base + i]);
    if (p1 != nullptr) s += Elem<T>::ld(p1[base + i]);
    if (pf != nullptr) s += pf[base + i];
    if (pg != nullptr) s += g * Elem<T>::ld(pg[base + i]);
    const float v = x[i] + s;
    x[i] = v;
    ss += v * v;
  }
  if (w == nullptr) return;
  const float r = 1.0f / sqrtf(block_sum(ss, red) / W + eps);
  T* o = out + base;
  for (int i = threadIdx.x; i < W; i += NT) o[i] = Elem<T>::st(x[i] * r * (w_offset + w[i]));
}

// kind 0: gelu (tanh form); 1: relu squared; 2: silu.  in rows have stride `in_stride`, out is dense.
template <typename T>
__global__ __launch_bounds__(NT) void act_kernel(const T* __restrict__ in, T* __restrict__ out, int64_t rows, int n,
                                                 int64_t in_stride, int kind) {
  const int64_t total = rows * n;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * NT + threadIdx.x; i < total; i += static_cast<int64_t>(gridDim.x) * NT) {
    const int64_t r = i / n;
    const int c = static_cast<int>(i - r * n);
    const float z = Elem<T>::ld(in[r * in_stride + c]);
    float y;
    if (kind == 0) {
      y = 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    } else if (kind == 2) {
      y = z / (1.0f + expf(-z));
    } else {
      const float p = fmaxf(z, 0.f);
      y = p * p;
    }
    out[i] = Elem<T>::st(y);
  }
}

// One block per token.  Row layout [q (n_q maps dim) | k (n_kv maps dim) | v (n_kv vdim) | ...].
// Feature i < 2 half of every map pairs with i +- half; angle = position * inv_freq[i % half] (fp32).
// K -> k_cache [NB, n_kv, BS, maps dim], V -> v_cache [NB, n_kv, vdim, BS] at `slots[t]` (slabs
// stored fragment-major when maps dim is a multiple of 4: see seqmix_attention.hip).
template <typename T>
__global__ __launch_bounds__(NT) void rope_multi_kv_kernel(const T* __restrict__ qkv, int64_t row_stride,
                                                           const int* __restrict__ positions,
                                                           const int* __restrict__ slots,
                                                           const float* __restrict__ inv_freq, int half,
                                                           T* __restrict__ q_out, T* __restrict__ k_cache,
                                                           T* __restrict__ v_cache, int n_q, int n_kv, int maps,
                                                           int dim, int vdim, int BS, int num_blocks) {
  const int t = blockIdx.x;
  const T* row = qkv + static_cast<size_t>(t) * row_stride;
  const float pos = static_cast<float>(positions[t]);
  const int slot = slots[t];
  const int blk = slot / BS, off = slot - blk * BS;
  const bool kv_ok = blk >= 0 && blk < num_blocks;
  const int qw = n_q * maps * dim, kw = n_kv * maps * dim, vw = n_kv * vdim;
  for (int idx = threadIdx.x; idx < qw + kw; idx += NT) {
    const int i = idx % dim;
    float val = Elem<T>::ld(row[idx]);
    if (i < 2 * half) {
      const bool lo = i < half;
      const float other = Elem<T>::ld(row[lo ? idx + half : idx - half]);
      float s, c;
      sincosf(pos * inv_freq[lo ? i : i - half], &s, &c);
      val = lo ? val * c - other * s : val * c + other * s;
    }
    if (idx < qw) {
      q_out[static_cast<size_t>(t) * qw + idx] = Elem<T>::st(val);
    } else if (kv_ok) {
      const int kk = idx - qw;
      const int KD = maps * dim;
      const int g = kk / KD, f = kk - g * KD;
      T* slab = k_cache + (static_cast<size_t>(blk) * n_kv + g) * BS * KD;
      // KD % 4 == 0: fragment-major slab [KD / 4][BS][4] (seqmix_attention.hip); else [BS][KD]
      if ((KD & 3) == 0) slab[(static_cast<size_t>(f >> 2) * BS + off) * 4 + (f & 3)] = Elem<T>::st(val);
      else slab[static_cast<size_t>(off) * KD + f] = Elem<T>::st(val);
    }
  }
  if (kv_ok) {
    for (int idx = threadIdx.x; idx < vw; idx += NT) {
      const int g = idx / vdim, e = idx - g * vdim;
      T* slab = v_cache + (static_cast<size_t>(blk) * n_kv + g) * vdim * BS;
      // fragment-major slab [BS / 4][vdim][4] with the K rule above; else [vdim][BS]
      if (((maps * dim) & 3) == 0) slab[(static_cast<size_t>(off >> 2) * vdim + e) * 4 + (off & 3)] = row[qw + kw + idx];
      else slab[static_cast<size_t>(e) * BS + off] = row[qw + kw + idx];
    }
  }
}

}  // namespace

BCG_API int bcg_embed_scale_rmsnorm(const void* tokens, const void* table, float scale, const void* w, float eps,
                                    float w_offset, void* resid, void* out, int T_, int W, int vocab, int is_f32,
                                    void* stream) {
  if (T_ <= 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (is_f32)
    embed_scale_norm_kernel<float><<<T_, NT, 0, s>>>(static_cast<const int*>(tokens), static_cast<const float*>(table), scale,
                                                    static_cast<const float*>(w), eps, w_offset,
                                                    static_cast<float*>(resid), static_cast<float*>(out), W, vocab);
  else
    embed_scale_norm_kernel<bf16_t><<<T_, NT, 0, s>>>(static_cast<const int*>(tokens), static_cast<const bf16_t*>(table), scale,
                                                     static_cast<const float*>(w), eps, w_offset,
                                                     static_cast<float*>(resid), static_cast<bf16_t*>(out), W, vocab);
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_residual_add_rmsnorm32(void* resid, const void* p0, const void* p1, const void* pf, const void* gate,
                                       const void* pg, const void* w, float eps, float w_offset, void* out, int T_,
                                       int W, int is_f32, void* stream) {
  if (T_ <= 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (is_f32)
    residual_norm_kernel<float><<<T_, NT, 0, s>>>(static_cast<float*>(resid), static_cast<const float*>(p0),
                                                 static_cast<const float*>(p1), static_cast<const float*>(pf),
                                                 static_cast<const float*>(gate), static_cast<const float*>(pg),
                                                 static_cast<const float*>(w), eps, w_offset, static_cast<float*>(out), W);
  else
    residual_norm_kernel<bf16_t><<<T_, NT, 0, s>>>(static_cast<float*>(resid), static_cast<const bf16_t*>(p0),
                                                  static_cast<const bf16_t*>(p1), static_cast<const float*>(pf),
                                                  static_cast<const float*>(gate), static_cast<const bf16_t*>(pg),
                                                  static_cast<const float*>(w), eps, w_offset, static_cast<bf16_t*>(out), W);
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_act_fn(const void* in, void* out, int64_t rows, int n, int64_t in_stride, int kind, int is_f32,
                       void* stream) {
  if (rows <= 0 || n <= 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t total = rows * n;
  const int grid = static_cast<int>(std::min<int64_t>((total + NT - 1) / NT, 65536));
  if (is_f32)
    act_kernel<float><<<grid, NT, 0, s>>>(static_cast<const float*>(in), static_cast<float*>(out), rows, n, in_stride, kind);
  else
    act_kernel<bf16_t><<<grid, NT, 0, s>>>(static_cast<const bf16_t*>(in), static_cast<bf16_t*>(out), rows, n, in_stride, kind);
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_rope_multi_kv_write(const void* qkv, int64_t row_stride, const void* positions, const void* slots,
                                    const void* inv_freq, int half, void* q_out, void* k_cache, void* v_cache, int T_,
                                    int n_q, int n_kv, int maps, int dim, int vdim, int BS, int num_blocks, int is_f32,
                                    void* stream) {
  if (T_ <= 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (is_f32)
    rope_multi_kv_kernel<float><<<T_, NT, 0, s>>>(static_cast<const float*>(qkv), row_stride, static_cast<const int*>(positions),
                                                 static_cast<const int*>(slots), static_cast<const float*>(inv_freq), half,
                                                 static_cast<float*>(q_out), static_cast<float*>(k_cache),
                                                 static_cast<float*>(v_cache), n_q, n_kv, maps, dim, vdim, BS, num_blocks);
  else
    rope_multi_kv_kernel<bf16_t><<<T_, NT, 0, s>>>(static_cast<const bf16_t*>(qkv), row_stride, static_cast<const int*>(positions),
                                                  static_cast<const int*>(slots), static_cast<const float*>(inv_freq), half,
                                                  static_cast<bf16_t*>(q_out), static_cast<bf16_t*>(k_cache),
                                                  static_cast<bf16_t*>(v_cache), n_q, n_kv, maps, dim, vdim, BS, num_blocks);
  return BCG_CHECK_LAUNCH();
}
