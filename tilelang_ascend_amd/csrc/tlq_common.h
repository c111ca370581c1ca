// Shared host/device helpers of libtlq (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "tlq.h"
#include "tlq_debug.h"

namespace tlq {

// ---- error reporting (thread local, read back through tlq_last_error) -------------------
void set_error(const char* fmt, ...);
bool check_launch(const char* what, const char* detail = nullptr);
uint64_t launch_count();

#define TLQ_REQUIRE(cond, ...)      \
  do {                              \
    if (!(cond)) {                  \
      ::tlq::set_error(__VA_ARGS__); \
      return 1;                     \
    }                               \
  } while (0)

// ---- vector types ---------------------------------------------------------------------
typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16_t;
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef int int4_t __attribute__((ext_vector_type(4)));
typedef unsigned int uint4_t __attribute__((ext_vector_type(4)));
typedef unsigned int uint2_t __attribute__((ext_vector_type(2)));

template <typename To, typename From>
__device__ __forceinline__ To bitcast(const From& v) {
  static_assert(sizeof(To) == sizeof(From), "bitcast size mismatch");
  return __builtin_bit_cast(To, v);
}

// Nibble-pair extraction constants, made opaque to the optimiser so that
// (x & mask) | (magic & ~mask) is selected as one v_bfi_b32 with register operands (gfx9 VOP3
// encodings cannot carry literals; with visible constants the compiler emits v_and + v_or).
//   lo: bits 0..3 and 16..19  ->  fp16 1024 + u     hi: bits 4..7 and 20..23  ->  fp16 64 + u
struct NibbleMagic {
  uint32_t m_lo, b_lo, m_hi, b_hi;
};
__device__ __forceinline__ uint32_t opaque_u32(uint32_t v) {
  asm volatile("" : "+v"(v));
  return v;
}
__device__ __forceinline__ NibbleMagic make_nibble_magic() {
  NibbleMagic m;
  m.m_lo = opaque_u32(0x000f000fu);
  m.b_lo = opaque_u32(0x64006400u);
  m.m_hi = opaque_u32(0x00f000f0u);
  m.b_hi = opaque_u32(0x54005400u);
  return m;
}
__device__ __forceinline__ uint32_t bfi(uint32_t mask, uint32_t x, uint32_t y) { return (x & mask) | (y & ~mask); }

// ---- 16-bit float helpers ----------------------------------------------------------------
// bfloat16 <-> float.  The narrowing is round-to-nearest-even (what torch's .to(bfloat16)
// and the reference's CAST_RINT do).
__device__ __forceinline__ float bf16_bits_to_float(uint32_t bits16) { return bitcast<float>(bits16 << 16); }
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f) {
  return (uint32_t)bitcast<uint16_t>((bf16_t)f);  // v_cvt_pk_bf16_f32: round to nearest even
}
// two floats -> packed bf16x2 (lo in bits 0..15)
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef float float2_t __attribute__((ext_vector_type(2)));
  float2_t f = {lo, hi};
  return bitcast<uint32_t>(__builtin_convertvector(f, bf16x2_t));
}
// byte B of x as float (v_cvt_f32_ubyteB); asm so that the optimiser keeps the one-op form
template <int B>
__device__ __forceinline__ float ubyte_to_float(uint32_t x) {
  float r;
  if (B == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(r) : "v"(x));
  if (B == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(r) : "v"(x));
  if (B == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(r) : "v"(x));
  if (B == 3) asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(r) : "v"(x));
  return r;
}
// value of a float after rounding it to bfloat16
__device__ __forceinline__ float round_to_bf16(float f) { return bitcast<float>(float_to_bf16_bits(f) << 16); }

// Generic load of a 16-bit float T (half_t or bf16_t) as float, and store with RNE.
// Tells the compiler that a pointer is the same in every lane, so that address = scalar base +
// 32-bit lane offset stays in that form (one VGPR per access instead of a 64-bit pair).
__device__ __forceinline__ const uint8_t* uniform_ptr(const uint8_t* p) {
  const uint64_t a = (uint64_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
  return (const uint8_t*)(((uint64_t)hi << 32) | lo);
}

template <typename T>
__device__ __forceinline__ float to_float(T v);
template <>
__device__ __forceinline__ float to_float<half_t>(half_t v) {
  return (float)v;
}
template <>
__device__ __forceinline__ float to_float<bf16_t>(bf16_t v) {
  return bf16_bits_to_float(bitcast<uint16_t>(v));
}

// Store one fp32 value as out_dtype (TLQ_F16 / TLQ_BF16 / TLQ_F32) at element index idx.
__device__ __forceinline__ void store_out(void* base, int64_t idx, float v, int out_dtype) {
  if (out_dtype == TLQ_F32) {
    ((float*)base)[idx] = v;
  } else if (out_dtype == TLQ_F16) {
    ((half_t*)base)[idx] = (half_t)v;
  } else {
    ((uint16_t*)base)[idx] = (uint16_t)float_to_bf16_bits(v);
  }
}

// ---- dequantisation of one nibble --------------------------------------------------------
// W = rn_T( rn_T(T(u) - z) * s ) with one rounding per operation.
template <typename T>
struct Dequant;

template <>
struct Dequant<half_t> {
  // native binary16 subtract and multiply round once each
  static __device__ __forceinline__ half_t apply(uint32_t u, half_t s, half_t z) {
    half_t d = (half_t)(float)u - z;
    return d * s;
  }
};
template <>
struct Dequant<bf16_t> {
  // float arithmetic on bfloat16 inputs followed by RNE narrowing == one bfloat16 rounding
  // per operation (the float result of the product is exact, of the difference it is exact
  // or harmlessly pre-rounded: 24 >= 2*8+2).
  static __device__ __forceinline__ bf16_t apply(uint32_t u, bf16_t s, bf16_t z) {
    float d = round_to_bf16((float)u - to_float(z));
    float w = d * to_float(s);
    return bitcast<bf16_t>((uint16_t)float_to_bf16_bits(w));
  }
};

template <typename T>
__device__ __forceinline__ T from_float(float f);
template <>
__device__ __forceinline__ half_t from_float<half_t>(float f) {
  return (half_t)f;
}
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float f) {
  return bitcast<bf16_t>((uint16_t)float_to_bf16_bits(f));
}

// int4 sign conventions
__device__ __forceinline__ int nibble_to_int(uint32_t u, int sign_mode) {
  switch (sign_mode) {
    case TLQ_S4_TWOS:
      return u >= 8 ? (int)u - 16 : (int)u;
    case TLQ_S4_OFFSET8:
      return (int)u - 8;
    case TLQ_S4_OFFSET7:
      return (int)u - 7;
    default:
      return (int)u;
  }
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace tlq
