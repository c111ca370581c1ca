// Stand-alone nibble unpack and per-group dequantisation kernels (HBM-bound streaming).
//
// Fast path: one lane turns 4 packed bytes (8 weights) into 16 bytes (fp16/bf16) or 8 bytes
// (int8) per step, so a wavefront reads 256 contiguous bytes and writes 1024 (512)
// contiguous bytes per instruction.  Shapes that do not fit (K % 8 != 0, group % 8 != 0)
// take a one-element-per-lane kernel.
#include "expand8.h"
#include "tlq_common.h"

namespace tlq {

// ---- unpack to int8 / fp16 / bf16 without scales --------------------------------------
template <typename OutT>
__device__ __forceinline__ OutT convert_nibble(uint32_t u, int sign_mode);
template <>
__device__ __forceinline__ int8_t convert_nibble<int8_t>(uint32_t u, int sign_mode) {
  return (int8_t)nibble_to_int(u, sign_mode);
}
template <>
__device__ __forceinline__ half_t convert_nibble<half_t>(uint32_t u, int sign_mode) {
  return (half_t)(float)nibble_to_int(u, sign_mode);
}
template <>
__device__ __forceinline__ bf16_t convert_nibble<bf16_t>(uint32_t u, int sign_mode) {
  return from_float<bf16_t>((float)nibble_to_int(u, sign_mode));
}

template <typename OutT>
__global__ __launch_bounds__(256) void unpack_int4_vec8(const uint32_t* __restrict__ wp, OutT* __restrict__ out,
                                                        int64_t n_words, int sign_mode) {
  struct alignas(8 * sizeof(OutT)) Vec {
    OutT v[8];
  };
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_words; i += (int64_t)gridDim.x * blockDim.x) {
    uint32_t x = wp[i];
    Vec r;
#pragma unroll
    for (int j = 0; j < 8; ++j) r.v[j] = convert_nibble<OutT>((x >> (4 * j)) & 0xF, sign_mode);
    ((Vec*)out)[i] = r;
  }
}

template <typename OutT>
__global__ __launch_bounds__(256) void unpack_int4_scalar(const uint8_t* __restrict__ wp, OutT* __restrict__ out,
                                                          int64_t n_elems, int sign_mode) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_elems; i += (int64_t)gridDim.x * blockDim.x) {
    uint32_t b = wp[i >> 1];
    out[i] = convert_nibble<OutT>((b >> (4 * (i & 1))) & 0xF, sign_mode);
  }
}

// ---- per-group dequantisation -----------------------------------------------------------
// One lane dequantises a 32-bit word (8 weights) with the expander the GEMM kernels use (bit-identical to the
// element-wise Dequant<T>::apply, a third of its instructions); a zero point that is a small integer folds into
// the unpack bias.  LAYOUT as in expand8.h (0 plain, 1 words permuted by interleave_weight for the fp16 target).
template <typename T, int LAYOUT>
__global__ __launch_bounds__(256) void dequant_w4_vec8(const uint32_t* __restrict__ wp, const T* __restrict__ scales,
                                                       const T* __restrict__ zeros, T* __restrict__ out,
                                                       int64_t n_words, int words_per_row, int group, int groups_per_row,
                                                       float zero_scalar) {
  const T one = from_float<T>(1.0f);
  const T zs = from_float<T>(zero_scalar);
  const NibbleMagic mg = make_nibble_magic();
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_words; i += (int64_t)gridDim.x * blockDim.x) {
    int64_t row = i / words_per_row;
    int k = (int)(i - row * words_per_row) * 8;
    int64_t gi = row * groups_per_row + k / group;
    T s = scales ? scales[gi] : one;
    T z = zeros ? zeros[gi] : zs;
    const uint32_t x = wp[i];
    const float zf = to_float(z);
    uint4_t r;
    if (zf == __builtin_rintf(zf) && zf >= -256.0f && zf <= 256.0f)
      r = Expand8<T, true, LAYOUT>(s, z, mg)(x);
    else
      r = Expand8<T, false, LAYOUT>(s, z, mg)(x);
    ((uint4_t*)out)[i] = r;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void dequant_w4_scalar(const uint8_t* __restrict__ wp, const T* __restrict__ scales,
                                                         const T* __restrict__ zeros, T* __restrict__ out, int64_t N,
                                                         int64_t K, int group, float zero_scalar) {
  const T one = from_float<T>(1.0f);
  const T zs = from_float<T>(zero_scalar);
  int64_t total = N * K;
  int64_t G = K / group;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    int64_t row = i / K;
    int64_t k = i - row * K;
    int64_t gi = row * G + k / group;
    T s = scales ? scales[gi] : one;
    T z = zeros ? zeros[gi] : zs;
    uint32_t b = wp[i >> 1];
    out[i] = Dequant<T>::apply((b >> (4 * (i & 1))) & 0xF, s, z);
  }
}

static int grid_for(int64_t items) {
  int64_t blocks = ceil_div(items, 256);
  const int64_t cap = 256 * 32;  // 256 CUs x 32 resident blocks is plenty for a streaming loop
  return (int)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

template <typename OutT>
static int launch_unpack(const void* wp, void* out, int64_t N, int64_t K, int sign_mode, hipStream_t st) {
  if (N * K == 0) return 0;
  const bool aligned = ((uintptr_t)wp % 4 == 0) && ((uintptr_t)out % (8 * sizeof(OutT)) == 0);
  if (K % 8 == 0 && aligned) {
    int64_t n_words = N * K / 8;
    unpack_int4_vec8<OutT><<<grid_for(n_words), 256, 0, st>>>((const uint32_t*)wp, (OutT*)out, n_words, sign_mode);
  } else {
    unpack_int4_scalar<OutT><<<grid_for(N * K), 256, 0, st>>>((const uint8_t*)wp, (OutT*)out, N * K, sign_mode);
  }
  return check_launch("tlq_unpack_int4") ? 0 : 1;
}

template <typename T>
static int launch_dequant(const void* wp, const void* scales, const void* zeros, void* out, int64_t N, int64_t K,
                          int64_t group, float zero_scalar, int w_layout, hipStream_t st) {
  if (N * K == 0) return 0;
  const bool aligned = ((uintptr_t)wp % 4 == 0) && ((uintptr_t)out % 16 == 0);
  if (K % 8 == 0 && group % 8 == 0 && aligned) {
    int64_t n_words = N * K / 8;
    if (w_layout == TLQ_W_INTERLEAVED_F16)
      dequant_w4_vec8<T, 1><<<grid_for(n_words), 256, 0, st>>>((const uint32_t*)wp, (const T*)scales, (const T*)zeros, (T*)out, n_words,
                                                              (int)(K / 8), (int)group, (int)(K / group), zero_scalar);
    else
      dequant_w4_vec8<T, 0><<<grid_for(n_words), 256, 0, st>>>((const uint32_t*)wp, (const T*)scales, (const T*)zeros, (T*)out, n_words,
                                                              (int)(K / 8), (int)group, (int)(K / group), zero_scalar);
  } else {
    if (w_layout != TLQ_W_PLAIN) {
      set_error("tlq_dequant_w4_layout: interleaved weights need K %% 8 == 0, group %% 8 == 0, 4-byte aligned words and a 16-byte aligned output");
      return 1;
    }
    dequant_w4_scalar<T><<<grid_for(N * K), 256, 0, st>>>((const uint8_t*)wp, (const T*)scales, (const T*)zeros, (T*)out,
                                                         N, K, (int)group, zero_scalar);
  }
  return check_launch("tlq_dequant_w4", "dequant_w4_vec8") ? 0 : 1;
}

}  // namespace tlq

extern "C" {

int tlq_unpack_int4(const void* w_packed, void* out, int64_t N, int64_t K, int out_dtype, int sign_mode, void* stream) {
  using namespace tlq;
  TLQ_REQUIRE(N >= 0 && K >= 0, "tlq_unpack_int4: negative shape N=%lld K=%lld", (long long)N, (long long)K);
  TLQ_REQUIRE(K % 2 == 0, "tlq_unpack_int4: K=%lld must be even (two int4 per byte)", (long long)K);
  TLQ_REQUIRE(sign_mode >= TLQ_U4 && sign_mode <= TLQ_S4_OFFSET7, "tlq_unpack_int4: bad sign_mode %d", sign_mode);
  TLQ_REQUIRE(N * K == 0 || (w_packed && out), "tlq_unpack_int4: null pointer");
  TLQ_REQUIRE(N * K < (int64_t)1 << 40, "tlq_unpack_int4: shape too large");
  hipStream_t st = (hipStream_t)stream;
  switch (out_dtype) {
    case TLQ_I8:
      return launch_unpack<int8_t>(w_packed, out, N, K, sign_mode, st);
    case TLQ_F16:
      return launch_unpack<half_t>(w_packed, out, N, K, sign_mode, st);
    case TLQ_BF16:
      return launch_unpack<bf16_t>(w_packed, out, N, K, sign_mode, st);
    default:
      set_error("tlq_unpack_int4: unsupported out_dtype %d", out_dtype);
      return 1;
  }
}

int tlq_dequant_w4_layout(const void* w_packed, const void* scales, const void* zeros, void* out, int64_t N, int64_t K,
                          int64_t group, float zero_scalar, int dtype, int w_layout, void* stream) {
  using namespace tlq;
  TLQ_REQUIRE(N >= 0 && K >= 0, "tlq_dequant_w4: negative shape");
  TLQ_REQUIRE(K % 2 == 0, "tlq_dequant_w4: K=%lld must be even", (long long)K);
  TLQ_REQUIRE(w_layout == TLQ_W_PLAIN || w_layout == TLQ_W_INTERLEAVED_F16, "tlq_dequant_w4: bad weight layout %d", w_layout);
  if (N * K == 0) return 0;
  TLQ_REQUIRE(group > 0 && K % group == 0, "tlq_dequant_w4: group=%lld must divide K=%lld", (long long)group,
              (long long)K);
  TLQ_REQUIRE(w_packed && out, "tlq_dequant_w4: null pointer");
  TLQ_REQUIRE(N * K < (int64_t)1 << 40, "tlq_dequant_w4: shape too large");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TLQ_F16) return launch_dequant<half_t>(w_packed, scales, zeros, out, N, K, group, zero_scalar, w_layout, st);
  if (dtype == TLQ_BF16) return launch_dequant<bf16_t>(w_packed, scales, zeros, out, N, K, group, zero_scalar, w_layout, st);
  set_error("tlq_dequant_w4: unsupported dtype %d", dtype);
  return 1;
}

int tlq_dequant_w4(const void* w_packed, const void* scales, const void* zeros, void* out, int64_t N, int64_t K,
                   int64_t group, float zero_scalar, int dtype, void* stream) {
  return tlq_dequant_w4_layout(w_packed, scales, zeros, out, N, K, group, zero_scalar, dtype, TLQ_W_PLAIN, stream);
}

}  // extern "C"
