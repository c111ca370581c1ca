// Eight packed int4 weights (one 32-bit word, nibble k = element k) -> eight fp16 / bf16 values in k order,
// dequantised exactly as the stand-alone kernel does: rn_T(rn_T(T(u) - z) * s).  Shared by the W4A16 tile and
// skinny kernels and the bf16 GEMV.
#pragma once
#include "tlq_common.h"

namespace tlq {

// FOLD is a compile-time flag: the decision is taken once per stage, not per element.
template <typename T, bool FOLD>
struct Expand8;

template <bool FOLD>
struct Expand8<half_t, FOLD> {
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
    uint4_t o;
    o.x = __builtin_amdgcn_perm(a1, a0, 0x05040100u);  // (k0, k1)
    o.y = __builtin_amdgcn_perm(a3, a2, 0x05040100u);  // (k2, k3)
    o.z = __builtin_amdgcn_perm(a1, a0, 0x07060302u);  // (k4, k5)
    o.w = __builtin_amdgcn_perm(a3, a2, 0x07060302u);  // (k6, k7)
    return o;
  }
};

template <bool FOLD>
struct Expand8<bf16_t, FOLD> {
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
    const uint32_t lo = v & 0x0f0f0f0fu;         // bytes k0, k2, k4, k6
    const uint32_t hi = (v >> 4) & 0x0f0f0f0fu;  // bytes k1, k3, k5, k7
    uint4_t o;
    o.x = pack_bf16x2(one(ubyte_to_float<0>(lo)), one(ubyte_to_float<0>(hi)));
    o.y = pack_bf16x2(one(ubyte_to_float<1>(lo)), one(ubyte_to_float<1>(hi)));
    o.z = pack_bf16x2(one(ubyte_to_float<2>(lo)), one(ubyte_to_float<2>(hi)));
    o.w = pack_bf16x2(one(ubyte_to_float<3>(lo)), one(ubyte_to_float<3>(hi)));
    return o;
  }
};

}  // namespace tlq
