// Fast decoders for interleaved 2-bit and 1-bit weights on gfx950 (device functions, header only).
//
// Counterparts of the CUDA lop3 decoders of tilelang/quantize/lop3.py:423-890 (fp16 targets), :892-996 (int8 targets)
// and :1048-1087 (2-bit -> packed 4-bit), with the same names and argument order:
//   decode_i2{u,s}_to_f16(src, dst)                              8 fields of a 16-bit word -> 8 fp16 (signed: u - 2)
//   decode_i2{u,s}_to_f16_scale(src, dst, scale)                 rn(x * s)
//   decode_i2u_to_f16_scale_zeros_original(src, dst, scale, z)   rn(rn(u - z) * s)
//   decode_i2u_to_f16_scale_zeros_rescale(src, dst, scale, z)    rn(rn(u * s) - z)       two roundings (lop3.py:626-627)
//   decode_i2u_to_f16_scale_zeros_quantized(src, dst, scale, qz) rn((u - qz) * s)        qz a 16-bit integer
//   decode_i1{u,s}_to_f16(src, dst)                              8 bits of a byte -> 8 fp16 (signed: 2 u - 1)
//   decode_i1{u,s}_to_f16_scale(src, dst, scale)                 rn(x * s)
//   decode_i1u_to_f16_scale_zeros_original(src, dst, scale, z)   rn(rn(u - z) * s)
//   decode_i1u_to_f16_scale_zeros_rescale(src, dst, scale, z)    fma(u, s, -|z|)         one rounding (lop3.py:870,880)
//   decode_i2{u,s}_to_i8s(src, dst)                              16 fields of a 32-bit word -> 16 int8 (signed: u - 2)
//   decode_i1{u,s}_to_i8s(src, dst)                              16 bits of a 16-bit word -> 16 int8 (signed: 2 u - 1)
//   decode_i2{u,s}_to_i4s(src, dst)                              16 fields of a 32-bit word -> 16 nibbles in two words
//                                                                (the signed form subtracts nothing: lop3.py:1067-1072)
// Output order (what the interleaved storage is made for): with f_j field j of the source, counted from bit 0,
//   fp16 targets   out = f0 f4 f1 f5 f2 f6 f3 f7            (a shift by one field and one AND-OR give two outputs)
//   2-bit -> int8  out word i, byte lane b = f(4b + i)
//   1-bit -> int8  out word i, byte lanes  = bit i, bit 8 + i, bit 4 + i, bit 12 + i
//   2-bit -> int4  out word i, nibble n    = f(2n + i),  i = 0, 1
#pragma once
#include "decode_i4.h"

namespace tlq_decode {

// (1024 + lo, 1024 + hi) from the fields at bits `bits * i` of the two halves of a spread word
template <uint32_t MASK>
__device__ __forceinline__ h2 biased_fields(uint32_t spread, int shift) {
  return as_h2(((spread >> shift) & MASK) | 0x64006400u);
}
// a 16-bit source: its low byte at bits 0..7, its high byte at bits 16..23 (lop3.py:439-440)
template <typename T1>
__device__ __forceinline__ uint32_t spread_i2(const T1* src) {
  const uint32_t w = (uint32_t)(*reinterpret_cast<const uint16_t*>(src));
  return (w & 0x00ffu) | ((w & 0xff00u) << 8);
}
// an 8-bit source: its low nibble at bits 0..3, its high nibble at bits 16..19 (lop3.py:703-704)
template <typename T1>
__device__ __forceinline__ uint32_t spread_i1(const T1* src) {
  const uint32_t w = (uint32_t)(*reinterpret_cast<const uint8_t*>(src));
  return (w & 0x0fu) | ((w & 0xf0u) << 12);
}

// ---- 2-bit -> fp16 --------------------------------------------------------------------------------------------------
template <typename T1, typename T2, bool isSigned>
__device__ __forceinline__ void decode_i2b_to_f16(T1* src, T2* dst, const int N = 8) {
  const uint32_t w = spread_i2(src);
  uint32_t* h = reinterpret_cast<uint32_t*>(dst);
  const h2 median = splat((_Float16)(isSigned ? 1026.0f : 1024.0f));
#pragma unroll
  for (int i = 0; i < N / 2; ++i) h[i] = as_u32(biased_fields<0x00030003u>(w, 2 * i) - median);
}
template <typename T1, typename T2>
__device__ __forceinline__ void decode_i2s_to_f16(T1* src, T2* dst, const int N = 8) {
  decode_i2b_to_f16<T1, T2, true>(src, dst, N);
}
template <typename T1, typename T2>
__device__ __forceinline__ void decode_i2u_to_f16(T1* src, T2* dst, const int N = 8) {
  decode_i2b_to_f16<T1, T2, false>(src, dst, N);
}

template <typename T1, typename T2, typename T3, bool isSigned>
__device__ __forceinline__ void decode_i2b_to_f16_scale(T1* src, T2* dst, const T3* scale, const int N = 8) {
  const uint32_t w = spread_i2(src);
  uint32_t* h = reinterpret_cast<uint32_t*>(dst);
  const h2 median = splat((_Float16)(isSigned ? 1026.0f : 1024.0f)), s = splat((_Float16)*scale);
#pragma unroll
  for (int i = 0; i < N / 2; ++i) h[i] = as_u32((biased_fields<0x00030003u>(w, 2 * i) - median) * s);
}
template <typename T1, typename T2, typename T3>
__device__ __forceinline__ void decode_i2s_to_f16_scale(T1* src, T2* dst, T3* scale, const int N = 8) {
  decode_i2b_to_f16_scale<T1, T2, T3, true>(src, dst, scale, N);
}
template <typename T1, typename T2, typename T3>
__device__ __forceinline__ void decode_i2u_to_f16_scale(T1* src, T2* dst, T3* scale, const int N = 8) {
  decode_i2b_to_f16_scale<T1, T2, T3, false>(src, dst, scale, N);
}

template <typename T1, typename T2, typename T3>
__device__ __forceinline__ void decode_i2u_to_f16_scale_zeros_original(T1* src, T2* dst, T3* scale, T3* zeros, const int N = 8) {
  const uint32_t w = spread_i2(src);
  uint32_t* h = reinterpret_cast<uint32_t*>(dst);
  const h2 k1024 = splat((_Float16)1024.0f), s = splat((_Float16)*scale), z = splat((_Float16)*zeros);
#pragma unroll
  for (int i = 0; i < N / 2; ++i) h[i] = as_u32(((biased_fields<0x00030003u>(w, 2 * i) - k1024) - z) * s);
}

// the product is rounded before the zero point is subtracted (a multiply-add with a zero addend, then a subtraction)
template <typename T1, typename T2, typename T3>
__device__ __forceinline__ void decode_i2u_to_f16_scale_zeros_rescale(T1* src, T2* dst, T3* scale, T3* zeros, const int N = 8) {
  const uint32_t w = spread_i2(src);
  uint32_t* h = reinterpret_cast<uint32_t*>(dst);
  const h2 k1024 = splat((_Float16)1024.0f), s = splat((_Float16)*scale), z = splat((_Float16)*zeros);
#pragma unroll
  for (int i = 0; i < N / 2; ++i) h[i] = as_u32(((biased_fields<0x00030003u>(w, 2 * i) - k1024) * s) - z);
}

// zeros points at a 16-bit integer zero point: 0xe400 | qz is the fp16 number -(1024 + qz) for qz in 0..1023
template <typename T1, typename T2, typename T3, typename T4>
__device__ __forceinline__ void decode_i2u_to_f16_scale_zeros_quantized(T1* src, T2* dst, T3* scale = nullptr,
                                                                        T4* zeros = nullptr, const int N = 8) {
  const uint32_t w = spread_i2(src);
  uint32_t* h = reinterpret_cast<uint32_t*>(dst);
  const uint32_t qz = (uint32_t)(*reinterpret_cast<const int16_t*>(zeros)) & 0xffffu;
  const h2 median = as_h2(((0xe400u | qz) << 16) | (0xe400u | qz)), s = splat((_Float16)*scale);
#pragma unroll
  for (int i = 0; i < N / 2; ++i) h[i] = as_u32((biased_fields<0x00030003u>(w, 2 * i) + median) * s);
}

// ---- 1-bit -> fp16 --------------------------------------------------------------------------------------------------
// signed: 2 u - 1, as x + x and then + (-1) (both exact)
template <typename T1, typename T2, bool isSigned>
__device__ __forceinline__ void decode_i1b_to_f16(T1* src, T2* dst, const int N = 8) {
  const uint32_t w = spread_i1(src);
  uint32_t* h = reinterpret_cast<uint32_t*>(dst);
  const h2 k1024 = splat((_Float16)1024.0f), minus1 = splat((_Float16)-1.0f);
#pragma unroll
  for (int i = 0; i < N / 2; ++i) {
    h2 x = biased_fields<0x00010001u>(w, i) - k1024;
    if (isSigned) x = (x + x) + minus1;
    h[i] = as_u32(x);
  }
}
template <typename T1, typename T2>
__device__ __forceinline__ void decode_i1s_to_f16(T1* src, T2* dst, const int N = 8) {
  decode_i1b_to_f16<T1, T2, true>(src, dst, N);
}
template <typename T1, typename T2>
__device__ __forceinline__ void decode_i1u_to_f16(T1* src, T2* dst, const int N = 8) {
  decode_i1b_to_f16<T1, T2, false>(src, dst, N);
}

template <typename T1, typename T2, typename T3, bool isSigned>
__device__ __forceinline__ void decode_i1b_to_f16_scale(T1* src, T2* dst, const T3* scale, const int N = 8) {
  const uint32_t w = spread_i1(src);
  uint32_t* h = reinterpret_cast<uint32_t*>(dst);
  const h2 k1024 = splat((_Float16)1024.0f), minus1 = splat((_Float16)-1.0f), s = splat((_Float16)*scale);
#pragma unroll
  for (int i = 0; i < N / 2; ++i) {
    h2 x = biased_fields<0x00010001u>(w, i) - k1024;
    if (isSigned) x = (x + x) + minus1;
    h[i] = as_u32(x * s);
  }
}
template <typename T1, typename T2, typename T3>
__device__ __forceinline__ void decode_i1u_to_f16_scale(T1* src, T2* dst, T3* scale = nullptr, const int N = 8) {
  decode_i1b_to_f16_scale<T1, T2, T3, false>(src, dst, scale, N);
}
template <typename T1, typename T2, typename T3>
__device__ __forceinline__ void decode_i1s_to_f16_scale(T1* src, T2* dst, T3* scale = nullptr, const int N = 8) {
  decode_i1b_to_f16_scale<T1, T2, T3, true>(src, dst, scale, N);
}

template <typename T1, typename T2, typename T3, typename T4>
__device__ __forceinline__ void decode_i1u_to_f16_scale_zeros_original(T1* src, T2* dst, T3* scale = nullptr,
                                                                       T4* zeros = nullptr, const int N = 8) {
  const uint32_t w = spread_i1(src);
  uint32_t* h = reinterpret_cast<uint32_t*>(dst);
  const h2 k1024 = splat((_Float16)1024.0f), s = splat((_Float16)*scale), z = splat((_Float16)*zeros);
#pragma unroll
  for (int i = 0; i < N / 2; ++i) h[i] = as_u32(((biased_fields<0x00010001u>(w, i) - k1024) - z) * s);
}

// the addend of the multiply-add is the zero point with its sign bit forced (0x80008000 | zeros): -|z|
template <typename T1, typename T2, typename T3, typename T4>
__device__ __forceinline__ void decode_i1u_to_f16_scale_zeros_rescale(T1* src, T2* dst, T3* scale = nullptr,
                                                                      T4* zeros = nullptr, const int N = 8) {
  const uint32_t w = spread_i1(src);
  uint32_t* h = reinterpret_cast<uint32_t*>(dst);
  const h2 k1024 = splat((_Float16)1024.0f), s = splat((_Float16)*scale), nz = neg_abs(splat((_Float16)*zeros));
#pragma unroll
  for (int i = 0; i < N / 2; ++i) h[i] = as_u32(__builtin_elementwise_fma(biased_fields<0x00010001u>(w, i) - k1024, s, nz));
}

// ---- integer targets ------------------------------------------------------------------------------------------------
// 16 two-bit fields of a 32-bit word -> 16 int8: output word i holds fields i, 4 + i, 8 + i, 12 + i in its byte lanes
template <typename T1, typename T2>
__device__ __forceinline__ void decode_i2u_to_i8s(T1* src, T2* dst, const int N = 16) {
  const uint32_t w = *reinterpret_cast<const uint32_t*>(src);
  uint32_t* o = reinterpret_cast<uint32_t*>(dst);
#pragma unroll
  for (int i = 0; i < N / 4; ++i) o[i] = (w >> (2 * i)) & 0x03030303u;
}
// signed: per byte u - 2 (no borrow between lanes: ((u | 0x80) - 2) ^ 0x80)
template <typename T1, typename T2>
__device__ __forceinline__ void decode_i2s_to_i8s(T1* src, T2* dst, const int N = 16) {
  decode_i2u_to_i8s(src, dst, N);
  uint32_t* o = reinterpret_cast<uint32_t*>(dst);
#pragma unroll
  for (int i = 0; i < N / 4; ++i) o[i] = ((o[i] | 0x80808080u) - 0x02020202u) ^ 0x80808080u;
}

// 16 bits of a 16-bit word -> 16 int8: the word's nibbles are spread to bits 0, 8, 16, 24 (low nibbles of the two bytes,
// then their high nibbles: lop3.py:899-900), output word i holds bits i, 8 + i, 4 + i, 12 + i in its byte lanes
template <typename T1, typename T2>
__device__ __forceinline__ void decode_i1u_to_i8s(T1* src, T2* dst, const int N = 16) {
  const uint32_t w16 = (uint32_t)(*reinterpret_cast<const uint16_t*>(src));
  const uint32_t w = (w16 & 0x0f0fu) | ((w16 & 0xf0f0u) << 12);
  uint32_t* o = reinterpret_cast<uint32_t*>(dst);
#pragma unroll
  for (int i = 0; i < N / 4; ++i) o[i] = (w >> i) & 0x01010101u;
}
// signed: per byte 2 u - 1, i.e. 0 -> 0xff, 1 -> 0x01
template <typename T1, typename T2>
__device__ __forceinline__ void decode_i1s_to_i8s(T1* src, T2* dst, const int N = 16) {
  decode_i1u_to_i8s(src, dst, N);
  uint32_t* o = reinterpret_cast<uint32_t*>(dst);
#pragma unroll
  for (int i = 0; i < N / 4; ++i) o[i] = ((0x01010101u ^ o[i]) * 0xffu) | o[i];
}

// 16 two-bit fields of a 32-bit word -> 16 nibbles in two words: nibble n of output word i holds field 2 n + i.
// The reference's signed form subtracts nothing (its body is a comment, lop3.py:1067-1072): the two are the same.
template <typename T1, typename T2>
__device__ __forceinline__ void decode_i2u_to_i4s(T1* src, T2* dst, const int N = 16) {
  const uint32_t* w = reinterpret_cast<const uint32_t*>(src);
  uint32_t* o = reinterpret_cast<uint32_t*>(dst);
#pragma unroll
  for (int i = 0; i < N / 8; ++i) o[i] = (w[i / 2] >> (2 * (i % 2))) & 0x33333333u;
}
template <typename T1, typename T2>
__device__ __forceinline__ void decode_i2s_to_i4s(T1* src, T2* dst, const int N = 16) {
  decode_i2u_to_i4s(src, dst, N);
}

}  // namespace tlq_decode
