// Helpers of the fp32-stream mixer kernels (seqmix_*.hip): element traits for the two activation
// types (bf16 bits / float) and a 16 x 16 MFMA step that is the same code for both.
#pragma once

#include "common.h"

typedef short s16x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Elem;
template <> struct Elem<bf16_t> {
  typedef s16x4 frag;  // 4 consecutive elements: one lane's share of a 16-deep MFMA operand
  static __device__ __forceinline__ float ld(bf16_t v) { return bf2f(v); }
  static __device__ __forceinline__ bf16_t st(float f) { return f2bf(f); }
  // finite inputs (softmax weights): the hardware's round-to-nearest-even conversion
  static __device__ __forceinline__ frag pack(float a, float b, float c, float d) {
    typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
    bf16x4 r;
    r[0] = static_cast<__bf16>(a); r[1] = static_cast<__bf16>(b);
    r[2] = static_cast<__bf16>(c); r[3] = static_cast<__bf16>(d);
    return __builtin_bit_cast(frag, r);
  }
};
template <> struct Elem<float> {
  typedef f32x4 frag;
  static __device__ __forceinline__ float ld(float v) { return v; }
  static __device__ __forceinline__ float st(float f) { return f; }
  static __device__ __forceinline__ frag pack(float a, float b, float c, float d) {
    frag r;
    r[0] = a; r[1] = b; r[2] = c; r[3] = d;
    return r;
  }
};

// C[16 x 16] += A[16 x 16] B[16 x 16].  Lane l holds A[m = l % 16][k = 4 (l / 16) + j],
// B[k = 4 (l / 16) + j][n = l % 16] (j = 0..3) and C[m = 4 (l / 16) + i][n = l % 16].
// bf16: one v_mfma_f32_16x16x16_bf16.  fp32: four v_mfma_f32_16x16x4_f32 (true fp32), step j
// taking element j of every lane -- both operands use the same k order, so the sum is the same.
__device__ __forceinline__ f32x4 mma16(s16x4 a, s16x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mma16(f32x4 a, f32x4 b, f32x4 c) {
#pragma unroll
  for (int j = 0; j < 4; ++j) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j], b[j], c, 0, 0, 0);
  return c;
}

// 4 consecutive elements at p[0..3]; elements at index >= n_valid read as zero.  `vec`: p is
// aligned for a vector load (the caller checked the strides); otherwise element loads.
template <typename T>
__device__ __forceinline__ typename Elem<T>::frag load_frag(const T* p, int n_valid, bool vec) {
  typedef typename Elem<T>::frag F;
  if (n_valid >= 4 && vec) return *reinterpret_cast<const F*>(p);
  F r;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    T v = j < n_valid ? p[j] : T(0);
    if constexpr (sizeof(T) == 2) r[j] = static_cast<short>(v); else r[j] = v;
  }
  return r;
}

// FULL: the caller guarantees four valid, vector-aligned elements (no branch around the load,
// so a run of fragment loads is issued back to back).
template <typename T, bool FULL>
__device__ __forceinline__ typename Elem<T>::frag load_frag_t(const T* p, int n_valid, bool vec) {
  if constexpr (FULL) return *reinterpret_cast<const typename Elem<T>::frag*>(p);
  else return load_frag<T>(p, n_valid, vec);
}

template <typename T>
__device__ __forceinline__ typename Elem<T>::frag zero_frag() {
  typename Elem<T>::frag r;
#pragma unroll
  for (int j = 0; j < 4; ++j) r[j] = 0;
  return r;
}
