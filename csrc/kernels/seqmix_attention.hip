// Multi-map (differential) causal GQA attention over a paged KV cache, fp32 scores and softmax.
//
//   head h, map m:  a_m = softmax(scale q_m K_m^T) V      (every map over the SAME values)
//   o = a_0 - lam a_1   (maps = 2;  maps = 1: a_0),   o <- o / sqrt(mean(o^2) + eps) * out_scale
//
// Cache of one layer run: K [NB, G, BS, maps dim], V [NB, G, vdim, BS] (V transposed per
// block-head: 16 consecutive keys of one value feature are contiguous).  BS is a multiple of 16.
//
// prefill_kernel: a work tile is <= 64 query rows of one sequence (4 waves x 16 rows) for one
// query head.  Per 16 keys a wave computes S^T = K Q^T (keys x queries) with 16 x 16 MFMAs, so
// the C registers of S^T are already the B operand (keys x queries) of O^T = V^T P^T: no
// shuffle between the two products; softmax statistics are per query = per lane column
// (reduced over the 4 lane groups).  K / V^T fragments are read straight from the cache
// (a lane's share of an operand is 4 consecutive elements of one cache row).
//
// decode_kernel: one wave per (item, head, 256-key split); a lane scores one key per 64-key
// chunk (q in LDS, fp32), the probabilities go through LDS and every lane then owns value
// features e, e + 64, ... reading 16 contiguous keys of its V^T row per page.  The split
// size is fixed, so a row's result does not depend on what else is in the batch.
// decode_merge_kernel merges the splits and applies the map combination + head norm.
#include <algorithm>

#include "seqmix_common.h"

namespace {

constexpr int SPLIT_KEYS = 256;

struct AttnArgs {
  const void* q;            // [T, H, maps dim]
  const void* k_cache;
  const void* v_cache;
  const int* block_tables;  // [B, max_blocks]
  const int* q_start;       // [B + 1] (prefill)
  const int* seq_lens;      // [B]
  const int* work;          // prefill: tiles [n, 3] {seq, row0, row_end}; decode: items [n, 2] {row, seq} or null
  void* out;                // [T, H vdim]
  float* ws;                // decode partials
  int max_blocks, H, G, maps, dim, vdim, BS, num_blocks, n_splits;
  float scale, lam, head_eps, out_scale;
  int vec_k, vec_v;         // rows of K / V^T are aligned for 4-element vector loads
};

template <typename T, int KC, int VT>
__global__ __launch_bounds__(256) void prefill_kernel(AttnArgs a) {
  typedef typename Elem<T>::frag F;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int h = blockIdx.y, g = h / (a.H / a.G);
  const int seq = a.work[3 * blockIdx.x], row0 = a.work[3 * blockIdx.x + 1] + 16 * wave, row_end = a.work[3 * blockIdx.x + 2];
  if (row0 >= row_end) return;
  const int ctx = a.seq_lens[seq], q_end = a.q_start[seq + 1];
  const int n_rows = min(16, row_end - row0);
  const int row = row0 + min(col, n_rows - 1);             // columns past the tile repeat its last row (never stored)
  const int pos = ctx - (q_end - row);                     // position of this lane's query column
  const int pos_max = ctx - (q_end - (row0 + n_rows - 1));
  const int KD = a.maps * a.dim;
  const int kc = (a.dim + 15) >> 4, vt = (a.vdim + 15) >> 4;
  const T* qrow = static_cast<const T*>(a.q) + (static_cast<size_t>(row) * a.H + h) * KD;
  const bool vec_q = (KD & 3) == 0 && a.vec_k;

  F qf[2][KC];
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      const int f = 16 * c + 4 * grp;
      qf[m][c] = (m < a.maps && c < kc) ? load_frag<T>(qrow + m * a.dim + f, a.dim - f, vec_q && (a.dim & 3) == 0) : zero_frag<T>();
    }
  f32x4 acc[2][VT];
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int t = 0; t < VT; ++t) acc[m][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  float mx[2] = {-INFINITY, -INFINITY}, den[2] = {0.f, 0.f};
  const int* table = a.block_tables + static_cast<size_t>(seq) * a.max_blocks;
  const T* kc_base = static_cast<const T*>(a.k_cache);
  const T* vc_base = static_cast<const T*>(a.v_cache);

  for (int kb = 0; 16 * kb <= pos_max; ++kb) {
    const int key0 = 16 * kb;
    int page = table[key0 / a.BS];
    page = (page < 0 || page >= a.num_blocks) ? 0 : page;
    const int koff = key0 % a.BS;
    // ---- S^T = K Q^T: A = K rows (key col, features 4 grp + j) ----
    const T* krow = kc_base + ((static_cast<size_t>(page) * a.G + g) * a.BS + koff + col) * KD;
    f32x4 s[2];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      s[m] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (m < a.maps) {
#pragma unroll
        for (int c = 0; c < KC; ++c)
          if (c < kc) {
            const int f = 16 * c + 4 * grp;
            const F kf = load_frag<T>(krow + m * a.dim + f, a.dim - f, a.vec_k && (a.dim & 3) == 0);
            s[m] = mma16(kf, qf[m][c], s[m]);
          }
      }
    }
    // ---- online softmax per query column; lane holds keys key0 + 4 grp + i ----
    F pf[2];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      if (m >= a.maps) { pf[m] = zero_frag<T>(); continue; }
      float v[4], bm = -INFINITY;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[i] = (key0 + 4 * grp + i <= pos) ? s[m][i] * a.scale : -INFINITY;
        bm = fmaxf(bm, v[i]);
      }
      bm = fmaxf(bm, __shfl_xor(bm, 16, WAVE));
      bm = fmaxf(bm, __shfl_xor(bm, 32, WAVE));
      const float m_new = fmaxf(mx[m], bm);               // finite: key 0 is visible to every query
      const float alpha = expf(mx[m] - m_new);
      float ps = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[i] = expf(v[i] - m_new);
        ps += v[i];
      }
      ps += __shfl_xor(ps, 16, WAVE);
      ps += __shfl_xor(ps, 32, WAVE);
      den[m] = den[m] * alpha + ps;
      mx[m] = m_new;
#pragma unroll
      for (int t = 0; t < VT; ++t)
        if (t < vt) acc[m][t] *= alpha;
      pf[m] = Elem<T>::pack(v[0], v[1], v[2], v[3]);
    }
    // ---- O^T += V^T P^T: A = V^T rows (feature 16 t + col, keys 4 grp + j) ----
#pragma unroll
    for (int t = 0; t < VT; ++t)
      if (t < vt) {
        const int e = 16 * t + col;
        F vf = zero_frag<T>();
        if (e < a.vdim)
          vf = load_frag<T>(vc_base + ((static_cast<size_t>(page) * a.G + g) * a.vdim + e) * a.BS + koff + 4 * grp, 4, a.vec_v);
        acc[0][t] = mma16(vf, pf[0], acc[0][t]);
        if (a.maps > 1) acc[1][t] = mma16(vf, pf[1], acc[1][t]);
      }
  }
  // ---- combine the maps, unit norm over the head's value features, store ----
  const float i0 = 1.0f / den[0], i1 = a.maps > 1 ? a.lam / den[1] : 0.f;
  float ss = 0.f;
#pragma unroll
  for (int t = 0; t < VT; ++t)
    if (t < vt) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float o = acc[0][t][i] * i0;
        if (a.maps > 1) o -= acc[1][t][i] * i1;
        acc[0][t][i] = o;
        ss += o * o;   // rows >= vdim are zero (their V^T fragments were zero)
      }
    }
  ss += __shfl_xor(ss, 16, WAVE);
  ss += __shfl_xor(ss, 32, WAVE);
  const float r = (a.head_eps >= 0.f ? 1.0f / sqrtf(ss / a.vdim + a.head_eps) : 1.0f) * a.out_scale;
  if (col < n_rows) {
    T* orow = static_cast<T*>(a.out) + (static_cast<size_t>(row) * a.H + h) * a.vdim;
#pragma unroll
    for (int t = 0; t < VT; ++t)
      if (t < vt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int e = 16 * t + 4 * grp + i;
          if (e < a.vdim) orow[e] = Elem<T>::st(acc[0][t][i] * r);
        }
      }
  }
}

// ws layout per (item, head, split): [maps] max, [maps] denominator, [maps][vdim] numerators.
template <typename T, int VPL>
__global__ __launch_bounds__(64) void decode_kernel(AttnArgs a, int n_items) {
  extern __shared__ float smem[];
  const int lane = threadIdx.x;
  const int h = blockIdx.x, split = blockIdx.y, item = blockIdx.z;
  const int g = h / (a.H / a.G);
  const int row = a.work ? a.work[2 * item] : item, seq = a.work ? a.work[2 * item + 1] : item;
  const int ctx = a.seq_lens[seq];
  const int k_begin = split * SPLIT_KEYS, k_end = min(ctx, k_begin + SPLIT_KEYS);
  if (k_begin >= k_end) return;
  const int KD = a.maps * a.dim;
  float* qs = smem;                  // [KD] scaled query
  float* ps = smem + KD;             // [maps][64] probabilities of the chunk
  const T* qrow = static_cast<const T*>(a.q) + (static_cast<size_t>(row) * a.H + h) * KD;
  for (int i = lane; i < KD; i += 64) qs[i] = Elem<T>::ld(qrow[i]) * a.scale;
  __syncthreads();
  const int* table = a.block_tables + static_cast<size_t>(seq) * a.max_blocks;
  const T* kc_base = static_cast<const T*>(a.k_cache);
  const T* vc_base = static_cast<const T*>(a.v_cache);
  float mx[2] = {-INFINITY, -INFINITY}, den[2] = {0.f, 0.f};
  float acc[2][VPL];
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int j = 0; j < VPL; ++j) acc[m][j] = 0.f;

  for (int c0 = k_begin; c0 < k_end; c0 += 64) {
    const int key = c0 + lane;
    const bool ok = key < k_end;
    float s[2] = {-INFINITY, -INFINITY};
    if (ok) {
      int page = table[key / a.BS];
      page = (page < 0 || page >= a.num_blocks) ? 0 : page;
      const T* krow = kc_base + ((static_cast<size_t>(page) * a.G + g) * a.BS + key % a.BS) * KD;
      for (int m = 0; m < a.maps; ++m) {
        float d = 0.f;
        const T* kp = krow + m * a.dim;
        const float* qp = qs + m * a.dim;
        if (a.vec_k && (a.dim & 3) == 0) {
          for (int f = 0; f < a.dim; f += 4) {
            const typename Elem<T>::frag kv = *reinterpret_cast<const typename Elem<T>::frag*>(kp + f);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              float kvj;
              if constexpr (sizeof(T) == 2) kvj = bf2f(static_cast<bf16_t>(kv[j])); else kvj = kv[j];
              d += qp[f + j] * kvj;
            }
          }
        } else {
          for (int f = 0; f < a.dim; ++f) d += qp[f] * Elem<T>::ld(kp[f]);
        }
        s[m] = d;
      }
    }
    __syncthreads();  // the previous chunk's probabilities have been read
    float alpha[2] = {1.f, 1.f};
    for (int m = 0; m < a.maps; ++m) {
      const float m_new = fmaxf(mx[m], wave_max(s[m]));   // finite: the chunk holds >= 1 key
      alpha[m] = expf(mx[m] - m_new);
      const float p = ok ? expf(s[m] - m_new) : 0.f;
      den[m] = den[m] * alpha[m] + wave_sum(p);
      mx[m] = m_new;
      ps[m * 64 + lane] = p;
    }
    __syncthreads();
    // ---- values: this lane owns features lane + 64 j; 16 contiguous keys per page group ----
    const int n_grp = (min(64, k_end - c0) + 15) >> 4;
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      const int e = lane + 64 * j;
      if (e < a.vdim) {
        float a0 = 0.f, a1 = 0.f;
        for (int gi = 0; gi < n_grp; ++gi) {
          const int key0 = c0 + 16 * gi;
          int page = table[key0 / a.BS];
          page = (page < 0 || page >= a.num_blocks) ? 0 : page;
          const T* vp = vc_base + ((static_cast<size_t>(page) * a.G + g) * a.vdim + e) * a.BS + key0 % a.BS;
          const int n_ok = min(16, k_end - key0);
          for (int kk = 0; kk < n_ok; ++kk) {     // (keys past the end hold stale data: never read)
            const float v = Elem<T>::ld(vp[kk]);
            a0 += ps[16 * gi + kk] * v;
            if (a.maps > 1) a1 += ps[64 + 16 * gi + kk] * v;
          }
        }
        acc[0][j] = acc[0][j] * alpha[0] + a0;
        acc[1][j] = acc[1][j] * alpha[1] + a1;
      }
    }
  }
  float* w = a.ws + ((static_cast<size_t>(item) * a.H + h) * a.n_splits + split) * (2 * a.maps + a.maps * a.vdim);
  if (lane < a.maps) {
    w[lane] = mx[lane];
    w[a.maps + lane] = den[lane];
  }
  for (int m = 0; m < a.maps; ++m)
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      const int e = lane + 64 * j;
      if (e < a.vdim) w[2 * a.maps + m * a.vdim + e] = acc[m][j];
    }
}

template <typename T, int VPL>
__global__ __launch_bounds__(64) void decode_merge_kernel(AttnArgs a) {
  const int lane = threadIdx.x, h = blockIdx.x, item = blockIdx.y;
  const int row = a.work ? a.work[2 * item] : item, seq = a.work ? a.work[2 * item + 1] : item;
  const int ctx = a.seq_lens[seq];
  const int n = min(a.n_splits, (ctx + SPLIT_KEYS - 1) / SPLIT_KEYS);
  const int stride = 2 * a.maps + a.maps * a.vdim;
  const float* w = a.ws + (static_cast<size_t>(item) * a.H + h) * a.n_splits * stride;
  float o[VPL];
#pragma unroll
  for (int j = 0; j < VPL; ++j) o[j] = 0.f;
  for (int m = 0; m < a.maps; ++m) {
    float mx = -INFINITY;
    for (int s = 0; s < n; ++s) mx = fmaxf(mx, w[s * stride + m]);
    float den = 0.f, num[VPL];
#pragma unroll
    for (int j = 0; j < VPL; ++j) num[j] = 0.f;
    for (int s = 0; s < n; ++s) {
      const float f = expf(w[s * stride + m] - mx);
      den += w[s * stride + a.maps + m] * f;
#pragma unroll
      for (int j = 0; j < VPL; ++j) {
        const int e = lane + 64 * j;
        if (e < a.vdim) num[j] += w[s * stride + 2 * a.maps + m * a.vdim + e] * f;
      }
    }
    const float c = (m == 0 ? 1.0f : -a.lam) / den;
#pragma unroll
    for (int j = 0; j < VPL; ++j) o[j] += num[j] * c;
  }
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < VPL; ++j) ss += (lane + 64 * j < a.vdim) ? o[j] * o[j] : 0.f;
  ss = wave_sum(ss);
  const float r = (a.head_eps >= 0.f ? 1.0f / sqrtf(ss / a.vdim + a.head_eps) : 1.0f) * a.out_scale;
  T* orow = static_cast<T*>(a.out) + (static_cast<size_t>(row) * a.H + h) * a.vdim;
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const int e = lane + 64 * j;
    if (e < a.vdim) orow[e] = Elem<T>::st(o[j] * r);
  }
}

template <typename T>
int launch_prefill(const AttnArgs& a, int n_tiles, hipStream_t s) {
  dim3 grid(n_tiles, a.H);
  if (a.dim <= 64 && a.vdim <= 128) prefill_kernel<T, 4, 8><<<grid, 256, 0, s>>>(a);
  else prefill_kernel<T, 8, 16><<<grid, 256, 0, s>>>(a);
  return BCG_CHECK_LAUNCH();
}

template <typename T>
int launch_decode(const AttnArgs& a, int n_items, hipStream_t s) {
  dim3 grid(a.H, a.n_splits, n_items);
  const size_t lds = sizeof(float) * (a.maps * a.dim + 2 * 64);
  if (a.vdim <= 128) {
    decode_kernel<T, 2><<<grid, 64, lds, s>>>(a, n_items);
    decode_merge_kernel<T, 2><<<dim3(a.H, n_items), 64, 0, s>>>(a);
  } else {
    decode_kernel<T, 4><<<grid, 64, lds, s>>>(a, n_items);
    decode_merge_kernel<T, 4><<<dim3(a.H, n_items), 64, 0, s>>>(a);
  }
  return BCG_CHECK_LAUNCH();
}

}  // namespace

BCG_API int bcg_multimap_split_keys() { return SPLIT_KEYS; }

// mode 0: prefill tiles (work = tiles [n_work, 3]); mode 1: single-token items (work = [n_work, 2]
// {row, sequence}, or null: item i is row i of sequence i).
BCG_API int bcg_multimap_attention(int mode, const void* q, const void* k_cache, const void* v_cache,
                                   const void* block_tables, int max_blocks, const void* q_start, const void* seq_lens,
                                   const void* work, int n_work, void* out, void* ws, int n_splits, int H, int G, int maps,
                                   int dim, int vdim, int BS, int num_blocks, float scale, float lam, float head_eps,
                                   float out_scale, int is_f32, void* stream) {
  if (n_work <= 0) return 0;
  if (maps < 1 || maps > 2 || dim > 128 || vdim > 256 || BS % 16 || H % G || n_work > 65535 * 16) return -2;
  AttnArgs a;
  a.q = q; a.k_cache = k_cache; a.v_cache = v_cache;
  a.block_tables = static_cast<const int*>(block_tables); a.q_start = static_cast<const int*>(q_start);
  a.seq_lens = static_cast<const int*>(seq_lens); a.work = static_cast<const int*>(work);
  a.out = out; a.ws = static_cast<float*>(ws);
  a.max_blocks = max_blocks; a.H = H; a.G = G; a.maps = maps; a.dim = dim; a.vdim = vdim; a.BS = BS;
  a.num_blocks = num_blocks; a.n_splits = n_splits;
  a.scale = scale; a.lam = lam; a.head_eps = head_eps; a.out_scale = out_scale;
  a.vec_k = ((maps * dim) % 4 == 0) ? 1 : 0;
  a.vec_v = 1;  // BS % 16 == 0: every 4-key group of a V^T row is aligned
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (mode == 0) return is_f32 ? launch_prefill<float>(a, n_work, s) : launch_prefill<bf16_t>(a, n_work, s);
  if (n_splits < 1 || H > 65535 || n_splits > 65535 || n_work > 65535) return -2;
  return is_f32 ? launch_decode<float>(a, n_work, s) : launch_decode<bf16_t>(a, n_work, s);
}
