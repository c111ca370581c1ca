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
  NibbleMagic mg;
  __device__ __forceinline__ Expand8(half_t s, half_t z, const NibbleMagic& mg_) : mg(mg_) {
    s2 = half2_t{s, s};
    z2 = half2_t{z, z};
    // with an integer zero point 1024+z and 64+z are exact binary16 values
    const half_t zl = FOLD ? (half_t)(1024.0f + (float)z) : (half_t)1024.0f;
    const half_t zh = FOLD ? (half_t)(64.0f + (float)z) : (half_t)64.0f;
    b_lo = half2_t{zl, zl};
    b_hi = half2_t{zh, zh};
  }
  __device__ __forceinline__ uint4_t operator()(uint32_t v) const {
    const uint32_t v8 = v >> 8;
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
  float sf, zf, c;
  __device__ __forceinline__ Expand8(bf16_t s, bf16_t z, const NibbleMagic&) {
    sf = to_float(s);
    zf = to_float(z);
    c = -(zf * sf);  // exact in fp32 for a small integer zero point (8 x 8 significant bits)
  }
  __device__ __forceinline__ float one(float u) const {
    // fold: (u - z) is an exact small integer, (u - z) * s = fma(u, s, -z*s) exactly
    if (FOLD) return __builtin_fmaf(u, sf, c);
    return round_to_bf16(u - zf) * sf;
  }
  __device__ __forceinline__ uint4_t operator()(uint32_t v) const {
    const uint32_t lo = v & 0x0f0f0f0fu;         // bytes k0, k2, k4, k6 (interleaved: k0, k4, k1, k5)
    const uint32_t hi = (v >> 4) & 0x0f0f0f0fu;  // bytes k1, k3, k5, k7 (interleaved: k2, k6, k3, k7)
    uint4_t o;
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
