// W4A16 prefill GEMM: packed-int4 weights are dequantised on their way from global memory
// into the LDS weight tile, then fp16 / bf16 MFMA with fp32 accumulation.
//
//   W[n, k] = rn_T( rn_T(T(u) - z) * s ),  C[m, n] = rn_out( sum_k A[m, k] * W[n, k] )
//
// The dequantised tile holds exactly the values of the stand-alone dequantisation kernel
// (one rounding per operation), so the GEMM result equals "dequantise, then fp32-accumulated
// matmul" up to summation order.
//
// One stage is 64 values of K: 32 packed bytes per weight row.  A thread loads 16 packed
// bytes (32 weights of one quantisation group) plus that group's scale / zero, and later
// expands them to four 16-byte LDS chunks.
//
// fp16 expansion, per 32-bit word (8 nibbles k0..k7):
//   (x    & 0x000f000f) | 0x64006400 -> half2 (1024+k0, 1024+k4)     one v_bfi_b32 each
//   (x    & 0x00f000f0) | 0x54005400 -> half2 (  64+k1,   64+k5)
//   (x>>8 & ...) likewise             -> (k2, k6), (k3, k7)
//   packed subtract of the bias (and of an integer zero point folded into it, exact), packed
//   multiply by the scale, then four v_perm_b32 put the halves back into k order.
// bf16 expansion: v_cvt_f32_ubyteN on the masked nibbles, fp32 fma / sub+mul with explicit
// bfloat16 roundings, v_cvt_pk_bf16_f32 to pack pairs in k order.
#include "gemm_core.h"

namespace tlq {

template <typename T>
struct Expand8;

template <>
struct Expand8<half_t> {
  half2_t s2, z2, b_lo, b_hi;
  NibbleMagic mg;
  bool fold;
  __device__ __forceinline__ Expand8(half_t s, half_t z, bool fold_, const NibbleMagic& mg_) : mg(mg_), fold(fold_) {
    s2 = half2_t{s, s};
    z2 = half2_t{z, z};
    // with an integer zero point 1024+z and 64+z are exact binary16 values
    const half_t zl = fold_ ? (half_t)(1024.0f + (float)z) : (half_t)1024.0f;
    const half_t zh = fold_ ? (half_t)(64.0f + (float)z) : (half_t)64.0f;
    b_lo = half2_t{zl, zl};
    b_hi = half2_t{zh, zh};
  }
  __device__ __forceinline__ uint4_t operator()(uint32_t v) const {
    const uint32_t v8 = v >> 8;
    half2_t p0 = bitcast<half2_t>(bfi(mg.m_lo, v, mg.b_lo)) - b_lo;   // (k0, k4)
    half2_t p1 = bitcast<half2_t>(bfi(mg.m_hi, v, mg.b_hi)) - b_hi;   // (k1, k5)
    half2_t p2 = bitcast<half2_t>(bfi(mg.m_lo, v8, mg.b_lo)) - b_lo;  // (k2, k6)
    half2_t p3 = bitcast<half2_t>(bfi(mg.m_hi, v8, mg.b_hi)) - b_hi;  // (k3, k7)
    if (!fold) {
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

template <>
struct Expand8<bf16_t> {
  float sf, zf, c;
  bool fold;
  __device__ __forceinline__ Expand8(bf16_t s, bf16_t z, bool fold_, const NibbleMagic&) : fold(fold_) {
    sf = to_float(s);
    zf = to_float(z);
    c = -(zf * sf);  // exact in fp32 for a small integer zero point (8 x 8 significant bits)
  }
  __device__ __forceinline__ float one(float u) const {
    // fold: (u - z) is an exact small integer, (u - z) * s = fma(u, s, -z*s) exactly
    if (fold) return __builtin_fmaf(u, sf, c);
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

template <typename T, int ROWS, int NT>
struct W4Loader {
  static constexpr int SLOTS = ROWS * 2;  // 16-byte packed loads per stage
  static constexpr int PASSES = (SLOTS + NT - 1) / NT;
  static constexpr bool PARTIAL = SLOTS % NT != 0;
  struct Params {
    const uint8_t* wp;
    const T* scales;
    const T* zeros;
    int64_t row_bytes;  // K / 2
    int groups;         // K / group
    int group;
    float zero_scalar;
    int fold;  // 1: zero point is one integer for the whole matrix and is folded into the bias
  };
  struct Regs {
    uint4_t v[PASSES];
    T s[PASSES], z[PASSES];
  };
  Params p;
  const uint8_t* base;
  int row0, rows_valid;
  NibbleMagic mg;

  __device__ __forceinline__ W4Loader(const Params& pp, int /*batch*/, int row0_, int rows_total)
      : p(pp), base(pp.wp + (int64_t)row0_ * pp.row_bytes), row0(row0_), rows_valid(rows_total - row0_),
        mg(make_nibble_magic()) {}

  __device__ __forceinline__ void gload(Regs& r, int kt, int tid) const {
    const T one = from_float<T>(1.0f);
    const T zs = from_float<T>(p.zero_scalar);
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      const int slot = ps * NT + tid;
      int row = slot >> 1;
      const int half = slot & 1;
      row = row < rows_valid ? row : rows_valid - 1;
      const int kb = kt * 32 + half * 16;
      uint4_t v = {0u, 0u, 0u, 0u};
      T s = one, z = zs;
      if (kb < p.row_bytes && (!PARTIAL || slot < SLOTS)) {
        v = *(const uint4_t*)(base + (int64_t)row * p.row_bytes + kb);
        const int64_t gi = (int64_t)(row0 + row) * p.groups + (kb * 2) / p.group;
        if (p.scales) s = p.scales[gi];
        if (p.zeros) z = p.zeros[gi];
      }
      r.v[ps] = v;
      r.s[ps] = s;
      r.z[ps] = z;
    }
  }
  __device__ __forceinline__ void lstore(const Regs& r, uint8_t* lds, int tid) const {
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      const int slot = ps * NT + tid;
      if (PARTIAL && slot >= SLOTS) continue;
      const int row = slot >> 1;
      const int half = slot & 1;
      const Expand8<T> ex(r.s[ps], r.z[ps], p.fold != 0, mg);
      *(uint4_t*)(lds + lds_off(row, half * 4 + 0)) = ex(r.v[ps].x);
      *(uint4_t*)(lds + lds_off(row, half * 4 + 1)) = ex(r.v[ps].y);
      *(uint4_t*)(lds + lds_off(row, half * 4 + 2)) = ex(r.v[ps].z);
      *(uint4_t*)(lds + lds_off(row, half * 4 + 3)) = ex(r.v[ps].w);
    }
  }
};

template <typename T>
struct MmaOf;
template <>
struct MmaOf<half_t> {
  typedef MmaF16 type;
};
template <>
struct MmaOf<bf16_t> {
  typedef MmaBF16 type;
};

template <typename T, int BM, int BN, int WM, int WN>
static int run_w4a16(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t N,
                     int64_t K, int64_t group, float zero_scalar, int fold, int out_dtype, hipStream_t st) {
  constexpr int NT = WM * WN * 64;
  typedef RowLoader<BM, NT> AL;
  typedef W4Loader<T, BN, NT> WL;
  typename AL::Params pa{(const uint8_t*)A, K * 2, 0, K * 2};
  typename WL::Params pw{(const uint8_t*)Wp, (const T*)scales, (const T*)zeros, K / 2, (int)(K / group), (int)group,
                         zero_scalar,        fold};
  EpiFloat::Params pe{C, N, 0, out_dtype};
  return launch_gemm<typename MmaOf<T>::type, AL, WL, EpiFloat, BM, BN, WM, WN>(pa, pw, pe, 1, M, N, K * 2, st,
                                                                               "tlq_gemm_w4a16(mfma)");
}

// tile override for tuning runs (0 = automatic)
static int g_w4a16_tile = 0;

template <typename T>
static int dispatch_w4a16(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M,
                          int64_t N, int64_t K, int64_t group, float zero_scalar, int fold, int out_dtype,
                          hipStream_t st) {
  int tile = g_w4a16_tile;
  if (tile == 0) {
    if (M <= 16)
      tile = 16;
    else if (M <= 32)
      tile = 32;
    else if (M <= 64)
      tile = 64;
    else if (M <= 128 || ceil_div(M, 256) * ceil_div(N, 256) < 128)
      tile = 128;
    else
      tile = 256;
  }
#define TLQ_RUN(BM, BN, WM, WN) \
  return run_w4a16<T, BM, BN, WM, WN>(A, Wp, scales, zeros, C, M, N, K, group, zero_scalar, fold, out_dtype, st)
  switch (tile) {
    case 16:
      TLQ_RUN(16, 64, 1, 4);
    case 32:
      TLQ_RUN(32, 128, 1, 4);
    case 64:
      TLQ_RUN(64, 256, 1, 4);
    case 128:
      TLQ_RUN(128, 128, 2, 2);
    case 512:
      TLQ_RUN(256, 256, 2, 4);
    default:
      TLQ_RUN(256, 256, 2, 2);
  }
#undef TLQ_RUN
}

int gemm_w4a16_mfma(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t N,
                    int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, hipStream_t st) {
  // An integer zero point shared by the whole matrix folds exactly into the unpack bias.
  const int fold = (zeros == nullptr && zero_scalar == (float)(int)zero_scalar && zero_scalar >= -256.0f &&
                    zero_scalar <= 256.0f)
                       ? 1
                       : 0;
  if (in_dtype == TLQ_F16)
    return dispatch_w4a16<half_t>(A, Wp, scales, zeros, C, M, N, K, group, zero_scalar, fold, out_dtype, st);
  return dispatch_w4a16<bf16_t>(A, Wp, scales, zeros, C, M, N, K, group, zero_scalar, fold, out_dtype, st);
}

}  // namespace tlq

extern "C" {
// Tuning hook used by the benchmark sweeps: forces the activation-tile height (16, 32, 64,
// 128, 256) of the W4A16 MFMA kernel; 0 restores the automatic choice.
void tlq_tune_w4a16_tile(int block_m) { tlq::g_w4a16_tile = block_m; }
}
