// Eight packed int4 weights (one 32-bit word) -> eight fp16 / bf16 values in k order, dequantised exactly as the
// stand-alone kernel does: rn_T(rn_T(T(u) - z) * s).  Shared by the W4A16 tile, streaming and skinny kernels, the
// dequantisation pass and the bf16 GEMV.
// LAYOUT 0: nibble k of the word is element k (general_compress, tilelang/quantize/utils.py:53-69).
// LAYOUT 1: the word went through interleave_weight for the fp16 target (utils.py:73-101): nibbles hold elements
//           0, 2, 4, 6, 1, 3, 5, 7, so that the two nibbles a 16-bit lane pair picks up are neighbours in k and the
//           fp16 decode needs no byte permutes (13 instead of 17 instructions per word).
#pragma once
#include "tlq_common.h"

namespace tlq {

// FOLD is a compile-time flag: the decision is taken once per stage, not per element.
template <typename T, bool FOLD, int LAYOUT = 0>
struct Expand8;

template <bool FOLD, int LAYOUT>
struct Expand8<half_t, FOLD, LAYOUT> {
  half2_t s2, z2, b_lo, b_hi;
  float sf, c_lo, c_hi;
  NibbleMagic mg;
  Expand8() = default;
  __device__ __forceinline__ Expand8(half_t s, half_t z, const NibbleMagic& mg_) : mg(mg_) {
    s2 = half2_t{s, s};
    z2 = half2_t{z, z};
    // with an integer zero point 1024+z and 64+z are exact binary16 values
    const half_t zl = FOLD ? (half_t)(1024.0f + (float)z) : (half_t)1024.0f;
    const half_t zh = FOLD ? (half_t)(64.0f + (float)z) : (half_t)64.0f;
    b_lo = half2_t{zl, zl};
    b_hi = half2_t{zh, zh};
    // (1024 + z) * s and (64 + z) * s are exact in fp32 (11 x 11 significant bits)
    sf = (float)s;
    c_lo = -((1024.0f + (float)z) * sf);
    c_hi = -((64.0f + (float)z) * sf);
  }
  // one value with an integer zero point: fma(1024 + u, s, -(1024 + z) s) is (u - z) s exactly in fp32 (at most 20
  // significant bits), rounded to binary16 once -- the rounding of the product in rn(rn(u - z) * s), whose difference
  // is exact.  One v_fma_mixlo/hi_f16 per value, written straight into its half of the operand register.
  static __device__ __forceinline__ half_t mix(half_t biased, float sf_, float c) { return (half_t)__builtin_fmaf((float)biased, sf_, c); }
  // A folded word comes in two independent halves: part p takes bytes p and p + 2 of the word (nibbles 2p, 2p + 1,
  // 2p + 4, 2p + 5) and gives two operand words -- in plain layout words p and p + 2 (values k 2p, 2p + 1 | 2p + 4, 2p + 5),
  // in interleaved layout words 2p and 2p + 1; place() puts them there.
  static constexpr bool SPLITS = FOLD;
  __device__ __forceinline__ uint2_t part(uint32_t v, int p) const {
    const uint32_t vv = p == 0 ? v : v >> 8;
    const half2_t q0 = bitcast<half2_t>(bfi(mg.m_lo, vv, mg.b_lo));
    const half2_t q1 = bitcast<half2_t>(bfi(mg.m_hi, vv, mg.b_hi));
    if (LAYOUT == 1) {
      const half2_t a{mix(q0.x, sf, c_lo), mix(q0.y, sf, c_lo)}, b{mix(q1.x, sf, c_hi), mix(q1.y, sf, c_hi)};
      return uint2_t{bitcast<uint32_t>(a), bitcast<uint32_t>(b)};
    }
    const half2_t a{mix(q0.x, sf, c_lo), mix(q1.x, sf, c_hi)}, b{mix(q0.y, sf, c_lo), mix(q1.y, sf, c_hi)};
    return uint2_t{bitcast<uint32_t>(a), bitcast<uint32_t>(b)};
  }
  static __device__ __forceinline__ void place(uint4_t& o, const uint2_t& h, int p) {
    if (LAYOUT == 1) {
      if (p == 0) o.x = h.x, o.y = h.y; else o.z = h.x, o.w = h.y;
    } else {
      if (p == 0) o.x = h.x, o.z = h.y; else o.y = h.x, o.w = h.y;
    }
  }
  // part() cut into four pieces of two or three instructions, for callers that interleave them with MFMAs by hand:
  // piece 0 picks the nibbles up, pieces 1 and 2 make the values of the two operand words in fp32 (exact), piece 3 rounds
  // and packs them (v_cvt_pk_f16_f32; measured faster in that setting than v_fma_mixlo/hi_f16 pairs writing the halves
  // of one register)
  struct Pieces {
    half2_t q0, q1;
    float f0, f1, f2, f3;
    uint32_t a, b;
    // An empty volatile statement that "rewrites" what piece i made: volatile statements keep their order, so a caller
    // that puts pin(i) behind its next MFMA statement keeps piece i ahead of that point and piece i + 1 behind it.
    __device__ __forceinline__ void pin(int i) {
      if (i == 0) asm volatile("" : "+v"(q0), "+v"(q1));
      if (i == 1) asm volatile("" : "+v"(q0), "+v"(q1), "+v"(f0), "+v"(f1));  // (also what piece 2 reads: it must not move ahead of this point)
      if (i == 2) asm volatile("" : "+v"(f0), "+v"(f1), "+v"(f2), "+v"(f3));  // (all four: piece 3 packs both words)
      if (i == 3) asm volatile("" : "+v"(a), "+v"(b));
    }
  };
  static __device__ __forceinline__ float mixf(half_t biased, float sf_, float c) { return __builtin_fmaf((float)biased, sf_, c); }
  static __device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
    typedef float float2_t __attribute__((ext_vector_type(2)));
    const float2_t f = {lo, hi};
    return bitcast<uint32_t>(__builtin_convertvector(f, half2_t));
  }
  __device__ __forceinline__ void piece(Pieces& st, uint32_t v, int p, int i) const {
    if (i == 0) {
      const uint32_t vv = p == 0 ? v : v >> 8;
      st.q0 = bitcast<half2_t>(bfi(mg.m_lo, vv, mg.b_lo));
      st.q1 = bitcast<half2_t>(bfi(mg.m_hi, vv, mg.b_hi));
    } else if (i == 1) {
      st.f0 = mixf(st.q0.x, sf, c_lo);
      st.f1 = LAYOUT == 1 ? mixf(st.q0.y, sf, c_lo) : mixf(st.q1.x, sf, c_hi);
    } else if (i == 2) {
      st.f2 = LAYOUT == 1 ? mixf(st.q1.x, sf, c_hi) : mixf(st.q0.y, sf, c_lo);
      st.f3 = mixf(st.q1.y, sf, c_hi);
    } else {
      st.a = pack_f16x2(st.f0, st.f1);
      st.b = pack_f16x2(st.f2, st.f3);
    }
  }
  __device__ __forceinline__ uint4_t operator()(uint32_t v) const {
    const uint32_t v8 = v >> 8;
    if (FOLD && LAYOUT == 0) {
      const half2_t q0 = bitcast<half2_t>(bfi(mg.m_lo, v, mg.b_lo));   // 1024 + (k0, k4)
      const half2_t q1 = bitcast<half2_t>(bfi(mg.m_hi, v, mg.b_hi));   // 64 + (k1, k5)
      const half2_t q2 = bitcast<half2_t>(bfi(mg.m_lo, v8, mg.b_lo));  // 1024 + (k2, k6)
      const half2_t q3 = bitcast<half2_t>(bfi(mg.m_hi, v8, mg.b_hi));  // 64 + (k3, k7)
      const half2_t o0{mix(q0.x, sf, c_lo), mix(q1.x, sf, c_hi)}, o1{mix(q2.x, sf, c_lo), mix(q3.x, sf, c_hi)};
      const half2_t o2{mix(q0.y, sf, c_lo), mix(q1.y, sf, c_hi)}, o3{mix(q2.y, sf, c_lo), mix(q3.y, sf, c_hi)};
      return uint4_t{bitcast<uint32_t>(o0), bitcast<uint32_t>(o1), bitcast<uint32_t>(o2), bitcast<uint32_t>(o3)};
    }
    half2_t p0 = bitcast<half2_t>(bfi(mg.m_lo, v, mg.b_lo)) - b_lo;   // (k0, k4)
    half2_t p1 = bitcast<half2_t>(bfi(mg.m_hi, v, mg.b_hi)) - b_hi;   // (k1, k5)
    half2_t p2 = bitcast<half2_t>(bfi(mg.m_lo, v8, mg.b_lo)) - b_lo;  // (k2, k6)
    half2_t p3 = bitcast<half2_t>(bfi(mg.m_hi, v8, mg.b_hi)) - b_hi;  // (k3, k7)
    if (!FOLD) {
      p0 = p0 - z2;
      p1 = p1 - z2;
      p2 = p2 - z2;
      p3 = p3 - z2;
    }
    p0 = p0 * s2;
    p1 = p1 * s2;
    p2 = p2 * s2;
    p3 = p3 * s2;
    const uint32_t a0 = bitcast<uint32_t>(p0), a1 = bitcast<uint32_t>(p1);
    const uint32_t a2 = bitcast<uint32_t>(p2), a3 = bitcast<uint32_t>(p3);
    if (LAYOUT == 1) return uint4_t{a0, a1, a2, a3};  // the pairs are (k0, k1), (k2, k3), (k4, k5), (k6, k7) already
    uint4_t o;
    o.x = __builtin_amdgcn_perm(a1, a0, 0x05040100u);  // (k0, k1)
    o.y = __builtin_amdgcn_perm(a3, a2, 0x05040100u);  // (k2, k3)
    o.z = __builtin_amdgcn_perm(a1, a0, 0x07060302u);  // (k4, k5)
    o.w = __builtin_amdgcn_perm(a3, a2, 0x07060302u);  // (k6, k7)
    return o;
  }
};

template <bool FOLD, int LAYOUT>
struct Expand8<bf16_t, FOLD, LAYOUT> {
  float sf, zf, c_lo, c_hi;
  NibbleMagic mg;
  Expand8() = default;
  __device__ __forceinline__ Expand8(bf16_t s, bf16_t z, const NibbleMagic& mg_) : mg(mg_) {
    sf = to_float(s);
    zf = to_float(z);
    // exact in fp32 for a small integer zero point (11 x 8 significant bits)
    c_lo = -((1024.0f + zf) * sf);
    c_hi = -((64.0f + zf) * sf);
  }
  // With an integer zero point the nibbles are picked up in pairs as binary16 values 1024 + u / 64 + u (the fp16
  // decoder's bit trick) and fma(1024 + u, s, -(1024 + z) s) is (u - z) s exactly in fp32 (at most 17 significant
  // bits): one v_fma_mix_f32 per value, then one rounding to bfloat16 -- the value rn(rn(u - z) * s), whose difference
  // is exact.  17 instead of 23 instructions per word.
  static __device__ __forceinline__ float mix(half_t biased, float sf_, float c) { return __builtin_fmaf((float)biased, sf_, c); }
  __device__ __forceinline__ float one(float u) const { return round_to_bf16(u - zf) * sf; }
  // halves of a folded word, as in the binary16 decoder above
  static constexpr bool SPLITS = FOLD;
  __device__ __forceinline__ uint2_t part(uint32_t v, int p) const {
    const uint32_t vv = p == 0 ? v : v >> 8;
    const half2_t q0 = bitcast<half2_t>(bfi(mg.m_lo, vv, mg.b_lo));
    const half2_t q1 = bitcast<half2_t>(bfi(mg.m_hi, vv, mg.b_hi));
    if (LAYOUT == 1) return uint2_t{pack_bf16x2(mix(q0.x, sf, c_lo), mix(q0.y, sf, c_lo)), pack_bf16x2(mix(q1.x, sf, c_hi), mix(q1.y, sf, c_hi))};
    return uint2_t{pack_bf16x2(mix(q0.x, sf, c_lo), mix(q1.x, sf, c_hi)), pack_bf16x2(mix(q0.y, sf, c_lo), mix(q1.y, sf, c_hi))};
  }
  static __device__ __forceinline__ void place(uint4_t& o, const uint2_t& h, int p) {
    if (LAYOUT == 1) {
      if (p == 0) o.x = h.x, o.y = h.y; else o.z = h.x, o.w = h.y;
    } else {
      if (p == 0) o.x = h.x, o.z = h.y; else o.y = h.x, o.w = h.y;
    }
  }
  // part() cut into four pieces of two or three instructions, for callers that interleave them with MFMAs by hand:
  // piece 0 picks the nibbles up, pieces 1 and 2 make the values of the two operand words, piece 3 rounds and packs them
  struct Pieces {
    half2_t q0, q1;
    float f0, f1, f2, f3;
    uint32_t a, b;
    // (see the binary16 decoder)
    __device__ __forceinline__ void pin(int i) {
      if (i == 0) asm volatile("" : "+v"(q0), "+v"(q1));
      if (i == 1) asm volatile("" : "+v"(q0), "+v"(q1), "+v"(f0), "+v"(f1));  // (also what piece 2 reads: it must not move ahead of this point)
      if (i == 2) asm volatile("" : "+v"(f0), "+v"(f1), "+v"(f2), "+v"(f3));  // (all four: piece 3 packs both words)
      if (i == 3) asm volatile("" : "+v"(a), "+v"(b));
    }
  };
  __device__ __forceinline__ void piece(Pieces& st, uint32_t v, int p, int i) const {
    if (i == 0) {
      const uint32_t vv = p == 0 ? v : v >> 8;
      st.q0 = bitcast<half2_t>(bfi(mg.m_lo, vv, mg.b_lo));
      st.q1 = bitcast<half2_t>(bfi(mg.m_hi, vv, mg.b_hi));
    } else if (i == 1) {
      st.f0 = mix(st.q0.x, sf, c_lo);
      st.f1 = LAYOUT == 1 ? mix(st.q0.y, sf, c_lo) : mix(st.q1.x, sf, c_hi);
    } else if (i == 2) {
      st.f2 = LAYOUT == 1 ? mix(st.q1.x, sf, c_hi) : mix(st.q0.y, sf, c_lo);
      st.f3 = mix(st.q1.y, sf, c_hi);
    } else {
      st.a = pack_bf16x2(st.f0, st.f1);
      st.b = pack_bf16x2(st.f2, st.f3);
    }
  }
  __device__ __forceinline__ uint4_t operator()(uint32_t v) const {
    uint4_t o;
    if (FOLD) {
      const uint32_t v8 = v >> 8;
      const half2_t q0 = bitcast<half2_t>(bfi(mg.m_lo, v, mg.b_lo));   // 1024 + nibbles (0, 4)
      const half2_t q1 = bitcast<half2_t>(bfi(mg.m_hi, v, mg.b_hi));   // 64 + nibbles (1, 5)
      const half2_t q2 = bitcast<half2_t>(bfi(mg.m_lo, v8, mg.b_lo));  // 1024 + nibbles (2, 6)
      const half2_t q3 = bitcast<half2_t>(bfi(mg.m_hi, v8, mg.b_hi));  // 64 + nibbles (3, 7)
      if (LAYOUT == 1) {  // nibbles hold elements 0, 2, 4, 6, 1, 3, 5, 7
        o.x = pack_bf16x2(mix(q0.x, sf, c_lo), mix(q0.y, sf, c_lo));
        o.y = pack_bf16x2(mix(q1.x, sf, c_hi), mix(q1.y, sf, c_hi));
        o.z = pack_bf16x2(mix(q2.x, sf, c_lo), mix(q2.y, sf, c_lo));
        o.w = pack_bf16x2(mix(q3.x, sf, c_hi), mix(q3.y, sf, c_hi));
        return o;
      }
      o.x = pack_bf16x2(mix(q0.x, sf, c_lo), mix(q1.x, sf, c_hi));
      o.y = pack_bf16x2(mix(q2.x, sf, c_lo), mix(q3.x, sf, c_hi));
      o.z = pack_bf16x2(mix(q0.y, sf, c_lo), mix(q1.y, sf, c_hi));
      o.w = pack_bf16x2(mix(q2.y, sf, c_lo), mix(q3.y, sf, c_hi));
      return o;
    }
    const uint32_t lo = v & 0x0f0f0f0fu;         // bytes k0, k2, k4, k6 (interleaved: k0, k4, k1, k5)
    const uint32_t hi = (v >> 4) & 0x0f0f0f0fu;  // bytes k1, k3, k5, k7 (interleaved: k2, k6, k3, k7)
    if (LAYOUT == 1) {
      o.x = pack_bf16x2(one(ubyte_to_float<0>(lo)), one(ubyte_to_float<2>(lo)));
      o.y = pack_bf16x2(one(ubyte_to_float<0>(hi)), one(ubyte_to_float<2>(hi)));
      o.z = pack_bf16x2(one(ubyte_to_float<1>(lo)), one(ubyte_to_float<3>(lo)));
      o.w = pack_bf16x2(one(ubyte_to_float<1>(hi)), one(ubyte_to_float<3>(hi)));
      return o;
    }
    o.x = pack_bf16x2(one(ubyte_to_float<0>(lo)), one(ubyte_to_float<0>(hi)));
    o.y = pack_bf16x2(one(ubyte_to_float<1>(lo)), one(ubyte_to_float<1>(hi)));
    o.z = pack_bf16x2(one(ubyte_to_float<2>(lo)), one(ubyte_to_float<2>(hi)));
    o.w = pack_bf16x2(one(ubyte_to_float<3>(lo)), one(ubyte_to_float<3>(hi)));
    return o;
  }
};

}  // namespace tlq
