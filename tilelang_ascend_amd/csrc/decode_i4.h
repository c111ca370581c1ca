// Fast decoders for interleaved 4-bit weights on gfx950 (device functions, header only).
//
// Counterparts of the CUDA lop3 decoders of tilelang/quantize/lop3.py:5-421 and :998-1046, with the
// same names and argument order, so that a kernel written against those can call these:
//   decode_i4{u,s}_to_f16(src, dst)                              8 nibbles (one 32-bit word) -> 8 fp16
//   decode_i4{u,s}_to_f16_scale(src, dst, scale)                 ... * s
//   decode_i4u_to_f16_scale_zeros_original(src, dst, scale, z)   (u - z) * s      two roundings
//   decode_i4u_to_f16_scale_zeros_rescale(src, dst, scale, z)    fma(u, s, -z)    one rounding
//   decode_i4u_to_f16_scale_zeros_quantized(src, dst, scale, qz) (u - qz) * s     qz an integer 0..15
//   decode_i4{u,s}_to_i8s(src, dst)                              16 nibbles (two words) -> 16 int8
//   ..._offset(src, dst, scale[, zeros], offset)                 the forms for fragments whose two halves belong to
//       different groups (lop3.py:82-131, :177-230, :272-322, :364-421): outputs 0..3 use scale[0] / zeros[0],
//       outputs 4..7 use scale[offset] / zeros[offset]
// The source words hold the nibbles in the order tilelang/quantize/utils.py:73-126
// (interleave_weight) produces, so that one shift + one AND-OR yields two neighbouring weights:
// word >> 4i has logical elements (2i, 2i+1) at bits 0..3 and 16..19 (fp16 target) and logical
// elements (i, ...) in byte lanes (int8 target).
//
// gfx950 mapping: the three-input logic op is v_and_or_b32 (mask and magic-number OR in one
// instruction), the paired fp16 arithmetic is v_pk_add_f16 / v_pk_mul_f16 / v_pk_fma_f16.  OR-ing
// 0x6400 into a 16-bit lane holding u in its low bits gives the fp16 number 1024 + u exactly.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tlq_decode {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ h2 as_h2(uint32_t x) {
  h2 r;
  __builtin_memcpy(&r, &x, 4);
  return r;
}
__device__ __forceinline__ uint32_t as_u32(h2 x) {
  uint32_t r;
  __builtin_memcpy(&r, &x, 4);
  return r;
}
__device__ __forceinline__ h2 splat(_Float16 v) { return h2{v, v}; }
__device__ __forceinline__ h2 neg_abs(h2 v) { return as_h2(as_u32(v) | 0x80008000u); }
// (1024 + u_lo, 1024 + u_hi) from the two nibbles at bits 4i and 16 + 4i
__device__ __forceinline__ h2 biased_pair(uint32_t word, int i) {
  return as_h2(((word >> (4 * i)) & 0x000f000fu) | 0x64006400u);
}

template <typename T1, typename T2, bool isSigned>
__device__ __forceinline__ void decode_i4b_to_f16(T1* src, T2* dst, const int N = 8) {
  const uint32_t w = *reinterpret_cast<const uint32_t*>(src);
  uint32_t* h = reinterpret_cast<uint32_t*>(dst);
  const h2 median = splat((_Float16)(isSigned ? 1032.0f : 1024.0f));
#pragma unroll
  for (int i = 0; i < N / 2; ++i) h[i] = as_u32(biased_pair(w, i) - median);
}
template <typename T1, typename T2>
__device__ __forceinline__ void decode_i4u_to_f16(T1* src, T2* dst, const int N = 8) {
  decode_i4b_to_f16<T1, T2, false>(src, dst, N);
}
template <typename T1, typename T2>
__device__ __forceinline__ void decode_i4s_to_f16(T1* src, T2* dst, const int N = 8) {
  decode_i4b_to_f16<T1, T2, true>(src, dst, N);
}

template <typename T1, typename T2, typename T3, bool isSigned>
__device__ __forceinline__ void decode_i4b_to_f16_scale(T1* src, T2* dst, const T3* scale, const int N = 8) {
  const uint32_t w = *reinterpret_cast<const uint32_t*>(src);
  uint32_t* h = reinterpret_cast<uint32_t*>(dst);
  const h2 median = splat((_Float16)(isSigned ? 1032.0f : 1024.0f));
  const h2 s = splat((_Float16)*scale);
#pragma unroll
  for (int i = 0; i < N / 2; ++i) h[i] = as_u32((biased_pair(w, i) - median) * s);
}
template <typename T1, typename T2, typename T3>
__device__ __forceinline__ void decode_i4u_to_f16_scale(T1* src, T2* dst, T3* scale = nullptr, const int N = 8) {
  decode_i4b_to_f16_scale<T1, T2, T3, false>(src, dst, scale, N);
}
template <typename T1, typename T2, typename T3>
__device__ __forceinline__ void decode_i4s_to_f16_scale(T1* src, T2* dst, T3* scale = nullptr, const int N = 8) {
  decode_i4b_to_f16_scale<T1, T2, T3, true>(src, dst, scale, N);
}

template <typename T1, typename T2, typename T3, typename T4>
__device__ __forceinline__ void decode_i4u_to_f16_scale_zeros_original(T1* src, T2* dst, T3* scale = nullptr,
                                                                       T4* zeros = nullptr, const int N = 8) {
  const uint32_t w = *reinterpret_cast<const uint32_t*>(src);
  uint32_t* h = reinterpret_cast<uint32_t*>(dst);
  const h2 k1024 = splat((_Float16)1024.0f), s = splat((_Float16)*scale), z = splat((_Float16)*zeros);
#pragma unroll
  for (int i = 0; i < N / 2; ++i) h[i] = as_u32(((biased_pair(w, i) - k1024) - z) * s);
}

template <typename T1, typename T2, typename T3, typename T4>
__device__ __forceinline__ void decode_i4u_to_f16_scale_zeros_rescale(T1* src, T2* dst, T3* scale = nullptr,
                                                                      T4* zeros = nullptr, const int N = 8) {
  const uint32_t w = *reinterpret_cast<const uint32_t*>(src);
  uint32_t* h = reinterpret_cast<uint32_t*>(dst);
  // the addend is the zero point with its sign bit forced (0x80008000 | zeros, lop3.py:247): -|z|
  const h2 k1024 = splat((_Float16)1024.0f), s = splat((_Float16)*scale), nz = neg_abs(splat((_Float16)*zeros));
#pragma unroll
  for (int i = 0; i < N / 2; ++i) h[i] = as_u32(__builtin_elementwise_fma(biased_pair(w, i) - k1024, s, nz));
}

// zeros points at a 16-bit integer zero point 0..15: 0xe400 | qz is the fp16 number -(1024 + qz)
template <typename T1, typename T2, typename T3, typename T4>
__device__ __forceinline__ void decode_i4u_to_f16_scale_zeros_quantized(T1* src, T2* dst, T3* scale = nullptr,
                                                                        T4* zeros = nullptr, const int N = 8) {
  const uint32_t w = *reinterpret_cast<const uint32_t*>(src);
  uint32_t* h = reinterpret_cast<uint32_t*>(dst);
  const uint32_t qz = (uint32_t)(*reinterpret_cast<const int16_t*>(zeros)) & 0xffffu;
  const h2 median = as_h2(((0xe400u | qz) << 16) | (0xe400u | qz)), s = splat((_Float16)*scale);
#pragma unroll
  for (int i = 0; i < N / 2; ++i) h[i] = as_u32((biased_pair(w, i) + median) * s);
}

// ---- forms with two groups per word: outputs 0..3 (h[0], h[1]) use *scale / *zeros, outputs 4..7 (h[2], h[3]) use
// *(scale + offset) / *(zeros + offset) ----------------------------------------------------------------------
template <typename T1, typename T2, typename T3, bool isSigned>
__device__ __forceinline__ void decode_i4b_to_f16_scale_offset(T1* src, T2* dst, const T3* scale, const int offset,
                                                               const int N = 8) {
  const uint32_t w = *reinterpret_cast<const uint32_t*>(src);
  uint32_t* h = reinterpret_cast<uint32_t*>(dst);
  const h2 median = splat((_Float16)(isSigned ? 1032.0f : 1024.0f));
  const h2 sl = splat((_Float16)*scale), sr = splat((_Float16) * (scale + offset));
#pragma unroll
  for (int i = 0; i < N / 2; ++i) h[i] = as_u32((biased_pair(w, i) - median) * (i < N / 4 ? sl : sr));
}
template <typename T1, typename T2, typename T3>
__device__ __forceinline__ void decode_i4u_to_f16_scale_offset(T1* src, T2* dst, T3* scale = nullptr, const int offset = 0,
                                                               const int N = 8) {
  decode_i4b_to_f16_scale_offset<T1, T2, T3, false>(src, dst, scale, offset, N);
}
template <typename T1, typename T2, typename T3>
__device__ __forceinline__ void decode_i4s_to_f16_scale_offset(T1* src, T2* dst, T3* scale = nullptr, const int offset = 0,
                                                               const int N = 8) {
  decode_i4b_to_f16_scale_offset<T1, T2, T3, true>(src, dst, scale, offset, N);
}

template <typename T1, typename T2, typename T3, typename T4>
__device__ __forceinline__ void decode_i4u_to_f16_scale_zeros_original_offset(T1* src, T2* dst, T3* scale = nullptr,
                                                                              T4* zeros = nullptr, const int offset = 0,
                                                                              const int N = 8) {
  const uint32_t w = *reinterpret_cast<const uint32_t*>(src);
  uint32_t* h = reinterpret_cast<uint32_t*>(dst);
  const h2 k1024 = splat((_Float16)1024.0f);
  const h2 sl = splat((_Float16)*scale), sr = splat((_Float16) * (scale + offset));
  const h2 zl = splat((_Float16)*zeros), zr = splat((_Float16) * (zeros + offset));
#pragma unroll
  for (int i = 0; i < N / 2; ++i) h[i] = as_u32(((biased_pair(w, i) - k1024) - (i < N / 4 ? zl : zr)) * (i < N / 4 ? sl : sr));
}

template <typename T1, typename T2, typename T3, typename T4>
__device__ __forceinline__ void decode_i4u_to_f16_scale_zeros_rescale_offset(T1* src, T2* dst, T3* scale = nullptr,
                                                                             T4* zeros = nullptr, const int offset = 0,
                                                                             const int N = 8) {
  const uint32_t w = *reinterpret_cast<const uint32_t*>(src);
  uint32_t* h = reinterpret_cast<uint32_t*>(dst);
  const h2 k1024 = splat((_Float16)1024.0f);
  const h2 sl = splat((_Float16)*scale), sr = splat((_Float16) * (scale + offset));
  const h2 zl = neg_abs(splat((_Float16)*zeros)), zr = neg_abs(splat((_Float16) * (zeros + offset)));
#pragma unroll
  for (int i = 0; i < N / 2; ++i)
    h[i] = as_u32(__builtin_elementwise_fma(biased_pair(w, i) - k1024, i < N / 4 ? sl : sr, i < N / 4 ? zl : zr));
}

// qzeros holds packed 4-bit zero points in words of the weights' storage type T1: the zero point of the first half
// is field group_offset of qzeros[0], that of the second half field group_offset of qzeros[zero_offset]
template <typename T1, typename T2, typename T3>
__device__ __forceinline__ void decode_i4u_to_f16_scale_zeros_quantized_offset(T1* src, T2* dst, T3* scale = nullptr,
                                                                               T1* qzeros = nullptr, const int scale_offset = 0,
                                                                               const int zero_offset = 0,
                                                                               const int group_offset = 0, const int N = 8) {
  const uint32_t w = *reinterpret_cast<const uint32_t*>(src);
  uint32_t* h = reinterpret_cast<uint32_t*>(dst);
  const h2 sl = splat((_Float16)*scale), sr = splat((_Float16) * (scale + scale_offset));
  const uint32_t ql = (uint32_t)(*qzeros >> (group_offset * 4)) & 0xfu, qr = (uint32_t)(*(qzeros + zero_offset) >> (group_offset * 4)) & 0xfu;
  const h2 ml = as_h2(((0xe400u | ql) << 16) | (0xe400u | ql)), mr = as_h2(((0xe400u | qr) << 16) | (0xe400u | qr));
#pragma unroll
  for (int i = 0; i < N / 2; ++i) h[i] = as_u32((biased_pair(w, i) + (i < N / 4 ? ml : mr)) * (i < N / 4 ? sl : sr));
}

// 16 nibbles -> 16 int8: output word i (i = 0, 1) holds nibbles 4i.. of src word 0 in byte lanes,
// words 2, 3 the same for src word 1.
template <typename T1, typename T2>
__device__ __forceinline__ void decode_i4u_to_i8s(T1* src, T2* dst, const int N = 16) {
  const uint32_t* w = reinterpret_cast<const uint32_t*>(src);
  uint32_t* o = reinterpret_cast<uint32_t*>(dst);
#pragma unroll
  for (int i = 0; i < N / 8; ++i) {
    o[i] = (w[0] >> (4 * i)) & 0x0f0f0f0fu;
    o[i + 2] = (w[1] >> (4 * i)) & 0x0f0f0f0fu;
  }
}
// signed variant: per byte u - 7 (the reference's MEDIAN_NUM is 0x07070707, lop3.py:1007,1019-1020).
// u - 7 lies in -7..8, so the saturating subtraction never saturates; the per-byte subtraction is
// done without borrows between lanes as ((u | 0x80) - 7) ^ 0x80.
template <typename T1, typename T2>
__device__ __forceinline__ void decode_i4s_to_i8s(T1* src, T2* dst, const int N = 16) {
  decode_i4u_to_i8s(src, dst, N);
  uint32_t* o = reinterpret_cast<uint32_t*>(dst);
#pragma unroll
  for (int i = 0; i < N / 4; ++i) o[i] = ((o[i] | 0x80808080u) - 0x07070707u) ^ 0x80808080u;
}

}  // namespace tlq_decode
