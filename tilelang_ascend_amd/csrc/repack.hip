// Offline weight preparation on the GPU: symmetric 4-bit group quantisation of a 16-bit weight matrix
// and packing of 4-bit values into bytes / interleaved 32-bit words.  Both are HBM-bound byte work:
// every element is read once and written once.
#include "tlq_common.h"

namespace tlq {

// ---- packing -------------------------------------------------------------------------------
// Eight values (one per byte of lo, hi) -> one 32-bit word, value k at bits 4k.  The values are NOT
// masked: a value outside 0..15 spills into its neighbours exactly as in the byte-wise OR of the
// reference (tilelang/quantize/utils.py:53-69 accumulates `w << 4k` in an int8).
__device__ __forceinline__ uint32_t pack8(uint32_t lo, uint32_t hi) {
  // bytes b0..b3 of lo, b4..b7 of hi, each sign-extended before the shift like an int8 operand
  uint32_t w = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t src = j < 2 ? lo : hi;
    const int e0 = (int)(int8_t)(src >> (16 * (j & 1)));
    const int e1 = (int)(int8_t)(src >> (16 * (j & 1) + 8));
    w |= ((uint32_t)(e0 | (e1 << 4)) & 0xffu) << (8 * j);
  }
  return w;
}

// Field permutation of tilelang/quantize/utils.py:73-101 for 4-bit fields: field i of the word moves to
// bit (i % G) * stride + (i / G) * 4 with stride 16, G 2 (fp16 target) or stride 8, G 4 (int8 target).
template <int MODE>
__device__ __forceinline__ uint32_t interleave8(uint32_t w) {
  if (MODE == 0) return w;
  uint32_t out = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int shift = MODE == 1 ? (i % 2) * 16 + (i / 2) * 4 : (i % 4) * 8 + (i / 4) * 4;
    out |= ((w >> (4 * i)) & 0xfu) << shift;
  }
  return out;
}

template <int MODE>
__global__ __launch_bounds__(256) void pack_int4_kernel(const uint8_t* __restrict__ src, uint32_t* __restrict__ dst,
                                                       int64_t n_words) {
  // a thread packs 16 values (one 16-byte load) into two words (one 8-byte store)
  const int64_t pairs = n_words >> 1;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < pairs; i += (int64_t)gridDim.x * blockDim.x) {
    const uint4_t v = ((const uint4_t*)src)[i];
    uint2_t o;
    o.x = interleave8<MODE>(pack8(v.x, v.y));
    o.y = interleave8<MODE>(pack8(v.z, v.w));
    ((uint2_t*)dst)[i] = o;
  }
  if ((n_words & 1) && blockIdx.x == 0 && threadIdx.x == 0) {  // odd word count: the last word
    const uint2_t v = ((const uint2_t*)src)[n_words - 1];
    dst[n_words - 1] = interleave8<MODE>(pack8(v.x, v.y));
  }
}

// ---- symmetric 4-bit group quantisation -----------------------------------------------------------
// s = max|w| * 0.125 over a group (rounded to T), q = clamp(rint(rn_T(w / s)) + 8, 0, 16), output q - 8.
// (tilelang/quantize/utils.py:5-50; the upper clamp is 16 there, reached only by the +max element.)
// A group of all zeros has s = 0 and every quotient is NaN, which the reference's int conversion turns
// into the most negative integer: q = 0, output -8.
template <typename T>
__device__ __forceinline__ float round_T(float v);
template <>
__device__ __forceinline__ float round_T<half_t>(float v) {
  return (float)(half_t)v;
}
template <>
__device__ __forceinline__ float round_T<bf16_t>(float v) {
  return round_to_bf16(v);
}

template <typename T>
__device__ __forceinline__ void widen8(const uint4_t& v, float (&f)[8]);
template <>
__device__ __forceinline__ void widen8<half_t>(const uint4_t& v, float (&f)[8]) {
  const half8_t h = bitcast<half8_t>(v);
#pragma unroll
  for (int i = 0; i < 8; ++i) f[i] = (float)h[i];
}
template <>
__device__ __forceinline__ void widen8<bf16_t>(const uint4_t& v, float (&f)[8]) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = bitcast<float>(w[i] << 16);
    f[2 * i + 1] = bitcast<float>(w[i] & 0xffff0000u);
  }
}

template <typename T>
__device__ __forceinline__ int quant_one(float w, float s) {
  if (s == 0.f) return -8;
  const float q = __builtin_rintf(round_T<T>(w / s));  // the quotient is rounded to the weight type first, as in torch
  const float c = fminf(fmaxf(q + 8.f, 0.f), 16.f);
  return (int)c - 8;
}

// LPG = lanes per group (group / 8), a power of two <= 64: the group maximum is a butterfly over LPG lanes.
template <typename T>
__global__ __launch_bounds__(256) void quantize_sym4_kernel(const T* __restrict__ W, int8_t* __restrict__ Q,
                                                           T* __restrict__ S, int64_t n_chunks, int lpg) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  // n_chunks is a multiple of lpg and the grid stride a multiple of 64, so the lanes of a group stay together
  for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c < ((n_chunks + 63) & ~(int64_t)63); c += stride) {
    const bool live = c < n_chunks;
    float f[8];
    float amax = 0.f;
    if (live) {
      widen8<T>(((const uint4_t*)W)[c], f);
#pragma unroll
      for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(f[i]));
    }
    for (int off = 1; off < lpg; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    const float s = round_T<T>(amax * 0.125f);
    if (live) {
      if ((c & (lpg - 1)) == 0) S[c / lpg] = from_float<T>(s);
      uint32_t o[2] = {0, 0};
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i >> 2] |= ((uint32_t)quant_one<T>(f[i], s) & 0xffu) << (8 * (i & 3));
      ((uint2_t*)Q)[c] = uint2_t{o[0], o[1]};
    }
  }
}

// any group size that is a multiple of 8: one wavefront per group, two passes over it
template <typename T>
__global__ __launch_bounds__(256) void quantize_sym4_generic_kernel(const T* __restrict__ W, int8_t* __restrict__ Q,
                                                                   T* __restrict__ S, int64_t n_groups, int group) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int64_t waves = (int64_t)gridDim.x * (blockDim.x >> 6);
  const int cpg = group >> 3;
  for (int64_t g = wave; g < n_groups; g += waves) {
    const uint4_t* w = (const uint4_t*)(W + g * group);
    float amax = 0.f;
    for (int c = lane; c < cpg; c += 64) {
      float f[8];
      widen8<T>(w[c], f);
#pragma unroll
      for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(f[i]));
    }
    for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    const float s = round_T<T>(amax * 0.125f);
    if (lane == 0) S[g] = from_float<T>(s);
    for (int c = lane; c < cpg; c += 64) {
      float f[8];
      widen8<T>(w[c], f);
      uint32_t o[2] = {0, 0};
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i >> 2] |= ((uint32_t)quant_one<T>(f[i], s) & 0xffu) << (8 * (i & 3));
      ((uint2_t*)(Q + g * group))[c] = uint2_t{o[0], o[1]};
    }
  }
}

template <typename T>
static int run_quantize(const void* W, void* Q, void* S, int64_t N, int64_t K, int64_t group, hipStream_t st) {
  const int64_t n_chunks = N * K / 8, lpg = group / 8;
  if (lpg <= 64 && (lpg & (lpg - 1)) == 0) {
    const int64_t want = ceil_div(n_chunks, (int64_t)256);
    quantize_sym4_kernel<T><<<(int)(want > 262144 ? 262144 : want), 256, 0, st>>>((const T*)W, (int8_t*)Q, (T*)S, n_chunks, (int)lpg);
  } else {
    const int64_t n_groups = N * (K / group), want = ceil_div(n_groups, (int64_t)4);
    quantize_sym4_generic_kernel<T><<<(int)(want > 262144 ? 262144 : want), 256, 0, st>>>((const T*)W, (int8_t*)Q, (T*)S, n_groups,
                                                                                         (int)group);
  }
  return check_launch("tlq_quantize_sym4") ? 0 : 1;
}

}  // namespace tlq

using namespace tlq;

extern "C" {

int tlq_pack_int4(const void* values, void* packed, int64_t N, int64_t K, int interleave, void* stream) {
  TLQ_REQUIRE(N >= 0 && K >= 0 && N < ((int64_t)1 << 31) && K < ((int64_t)1 << 31), "tlq_pack_int4: bad shape N=%lld K=%lld",
              (long long)N, (long long)K);
  TLQ_REQUIRE(interleave >= 0 && interleave <= 2, "tlq_pack_int4: interleave must be 0 (none), 1 (fp16 order) or 2 (int8 order)");
  if (N == 0 || K == 0) return 0;
  TLQ_REQUIRE(K % 8 == 0, "tlq_pack_int4: K=%lld must be a multiple of 8", (long long)K);
  TLQ_REQUIRE(values && packed, "tlq_pack_int4: null pointer");
  TLQ_REQUIRE(((uintptr_t)values & 15) == 0 && ((uintptr_t)packed & 7) == 0, "tlq_pack_int4: values must be 16-byte and packed 8-byte aligned");
  const int64_t n_words = N * K / 8;
  const int64_t want = ceil_div((n_words >> 1) + 1, (int64_t)256);
  const int blocks = (int)(want > 262144 ? 262144 : want);
  hipStream_t st = (hipStream_t)stream;
  if (interleave == 0)
    pack_int4_kernel<0><<<blocks, 256, 0, st>>>((const uint8_t*)values, (uint32_t*)packed, n_words);
  else if (interleave == 1)
    pack_int4_kernel<1><<<blocks, 256, 0, st>>>((const uint8_t*)values, (uint32_t*)packed, n_words);
  else
    pack_int4_kernel<2><<<blocks, 256, 0, st>>>((const uint8_t*)values, (uint32_t*)packed, n_words);
  return check_launch("tlq_pack_int4") ? 0 : 1;
}

int tlq_quantize_sym4(const void* W, void* q_minus8, void* scales, int64_t N, int64_t K, int64_t group, int dtype, void* stream) {
  TLQ_REQUIRE(N >= 0 && K >= 0 && N < ((int64_t)1 << 31) && K < ((int64_t)1 << 31), "tlq_quantize_sym4: bad shape N=%lld K=%lld",
              (long long)N, (long long)K);
  TLQ_REQUIRE(dtype == TLQ_F16 || dtype == TLQ_BF16, "tlq_quantize_sym4: dtype must be float16 or bfloat16 (got %d)", dtype);
  if (N == 0 || K == 0) return 0;
  TLQ_REQUIRE(group > 0 && group % 8 == 0 && K % group == 0, "tlq_quantize_sym4: group=%lld must be a multiple of 8 that divides K=%lld",
              (long long)group, (long long)K);
  TLQ_REQUIRE(W && q_minus8 && scales, "tlq_quantize_sym4: null pointer");
  TLQ_REQUIRE(((uintptr_t)W & 15) == 0 && ((uintptr_t)q_minus8 & 7) == 0 && ((uintptr_t)scales & 1) == 0, "tlq_quantize_sym4: misaligned pointer");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TLQ_F16) return run_quantize<half_t>(W, q_minus8, scales, N, K, group, st);
  return run_quantize<bf16_t>(W, q_minus8, scales, N, K, group, st);
}

}  // extern "C"
