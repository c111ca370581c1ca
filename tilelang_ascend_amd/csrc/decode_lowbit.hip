// Stand-alone kernel around the interleaved 2-bit / 1-bit fast decoders (decode_lowbit.h): one lane decodes one unit,
// 16 bytes of output -- 8 fp16 from 16 (2-bit) or 8 (1-bit) source bits, 16 int8 from 32 or 16 source bits -- or, for the
// packed 4-bit target, 16 nibbles (8 bytes) from 32 source bits.
#include "decode_lowbit.h"
#include "tlq_common.h"

namespace tlq {

enum { LB_ZEROS_NONE = 0, LB_ZEROS_ORIGINAL = 1, LB_ZEROS_RESCALE = 2, LB_ZEROS_QUANTIZED = 3 };

template <int BITS, bool SIGNED, bool SCALE, int ZMODE>
__global__ __launch_bounds__(256) void decode_lowbit_f16_kernel(const uint8_t* __restrict__ src, const half_t* __restrict__ scales,
                                                                const void* __restrict__ zeros, uint4_t* __restrict__ out,
                                                                int64_t n_units, int units_per_group) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_units; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t g = i / units_per_group;
    uint4_t r;
    if constexpr (BITS == 2) {
      uint16_t w = ((const uint16_t*)src)[i];
      if constexpr (ZMODE == LB_ZEROS_ORIGINAL)
        tlq_decode::decode_i2u_to_f16_scale_zeros_original(&w, &r, scales + g, (const half_t*)zeros + g);
      else if constexpr (ZMODE == LB_ZEROS_RESCALE)
        tlq_decode::decode_i2u_to_f16_scale_zeros_rescale(&w, &r, scales + g, (const half_t*)zeros + g);
      else if constexpr (ZMODE == LB_ZEROS_QUANTIZED)
        tlq_decode::decode_i2u_to_f16_scale_zeros_quantized(&w, &r, scales + g, (const int16_t*)zeros + g);
      else if constexpr (SCALE)
        tlq_decode::decode_i2b_to_f16_scale<uint16_t, uint4_t, half_t, SIGNED>(&w, &r, scales + g);
      else
        tlq_decode::decode_i2b_to_f16<uint16_t, uint4_t, SIGNED>(&w, &r);
    } else {
      uint8_t w = src[i];
      if constexpr (ZMODE == LB_ZEROS_ORIGINAL)
        tlq_decode::decode_i1u_to_f16_scale_zeros_original(&w, &r, scales + g, (const half_t*)zeros + g);
      else if constexpr (ZMODE == LB_ZEROS_RESCALE)
        tlq_decode::decode_i1u_to_f16_scale_zeros_rescale(&w, &r, scales + g, (const half_t*)zeros + g);
      else if constexpr (SCALE)
        tlq_decode::decode_i1b_to_f16_scale<uint8_t, uint4_t, half_t, SIGNED>(&w, &r, scales + g);
      else
        tlq_decode::decode_i1b_to_f16<uint8_t, uint4_t, SIGNED>(&w, &r);
    }
    out[i] = r;
  }
}

template <int BITS, bool SIGNED>
__global__ __launch_bounds__(256) void decode_lowbit_i8_kernel(const uint8_t* __restrict__ src, uint4_t* __restrict__ out, int64_t n_units) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_units; i += (int64_t)gridDim.x * blockDim.x) {
    uint4_t r;
    if constexpr (BITS == 2) {
      uint32_t w = ((const uint32_t*)src)[i];
      if (SIGNED) tlq_decode::decode_i2s_to_i8s(&w, &r); else tlq_decode::decode_i2u_to_i8s(&w, &r);
    } else {
      uint16_t w = ((const uint16_t*)src)[i];
      if (SIGNED) tlq_decode::decode_i1s_to_i8s(&w, &r); else tlq_decode::decode_i1u_to_i8s(&w, &r);
    }
    out[i] = r;
  }
}

template <bool SIGNED>
__global__ __launch_bounds__(256) void decode_i2_i4_kernel(const uint32_t* __restrict__ src, uint2_t* __restrict__ out, int64_t n_units) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_units; i += (int64_t)gridDim.x * blockDim.x) {
    uint32_t w = src[i];
    uint2_t r;
    if (SIGNED) tlq_decode::decode_i2s_to_i4s(&w, &r); else tlq_decode::decode_i2u_to_i4s(&w, &r);
    out[i] = r;
  }
}

static int lb_grid_for(int64_t n) { return (n + 255) / 256 > 65535 ? 65535 : (int)((n + 255) / 256); }

template <int BITS>
static void launch_f16(const uint8_t* w, const half_t* s, const void* zeros, uint4_t* o, int64_t n, int upg, bool is_signed, int zmode,
                       hipStream_t st) {
  const int g = lb_grid_for(n);
  if (zmode == LB_ZEROS_ORIGINAL) { decode_lowbit_f16_kernel<BITS, false, true, LB_ZEROS_ORIGINAL><<<g, 256, 0, st>>>(w, s, zeros, o, n, upg); return; }
  if (zmode == LB_ZEROS_RESCALE) { decode_lowbit_f16_kernel<BITS, false, true, LB_ZEROS_RESCALE><<<g, 256, 0, st>>>(w, s, zeros, o, n, upg); return; }
  if constexpr (BITS == 2)
    if (zmode == LB_ZEROS_QUANTIZED) { decode_lowbit_f16_kernel<2, false, true, LB_ZEROS_QUANTIZED><<<g, 256, 0, st>>>(w, s, zeros, o, n, upg); return; }
  if (s) {
    if (is_signed) decode_lowbit_f16_kernel<BITS, true, true, LB_ZEROS_NONE><<<g, 256, 0, st>>>(w, s, zeros, o, n, upg);
    else decode_lowbit_f16_kernel<BITS, false, true, LB_ZEROS_NONE><<<g, 256, 0, st>>>(w, s, zeros, o, n, upg);
  } else {
    if (is_signed) decode_lowbit_f16_kernel<BITS, true, false, LB_ZEROS_NONE><<<g, 256, 0, st>>>(w, s, zeros, o, n, upg);
    else decode_lowbit_f16_kernel<BITS, false, false, LB_ZEROS_NONE><<<g, 256, 0, st>>>(w, s, zeros, o, n, upg);
  }
}

}  // namespace tlq

using namespace tlq;

extern "C" int tlq_decode_lowbit_interleaved(const void* src, const void* scales, const void* zeros, void* out, int64_t n_units,
                                             int64_t units_per_group, int source_bit, int out_bits, int is_signed, int zeros_mode,
                                             void* stream) {
  const char* me = "tlq_decode_lowbit_interleaved";
  TLQ_REQUIRE(source_bit == 2 || source_bit == 1, "%s: source_bit must be 2 or 1 (got %d; 4-bit sources: tlq_decode_i4_interleaved)", me, source_bit);
  TLQ_REQUIRE(out_bits == 16 || out_bits == 8 || out_bits == 4, "%s: out_bits must be 16 (fp16), 8 (int8) or 4 (packed nibbles), got %d", me, out_bits);
  TLQ_REQUIRE(!(out_bits == 4 && source_bit != 2), "%s: the packed 4-bit target takes 2-bit sources only", me);
  TLQ_REQUIRE(n_units >= 0 && n_units < ((int64_t)1 << 40), "%s: bad n_units %lld", me, (long long)n_units);
  TLQ_REQUIRE(zeros_mode >= LB_ZEROS_NONE && zeros_mode <= LB_ZEROS_QUANTIZED, "%s: bad zeros_mode %d", me, zeros_mode);
  TLQ_REQUIRE(!(zeros_mode == LB_ZEROS_QUANTIZED && source_bit == 1), "%s: 1-bit sources have no decoder for quantized zeros", me);
  TLQ_REQUIRE(!(zeros_mode != LB_ZEROS_NONE && is_signed), "%s: zeros are not supported for signed sources", me);
  TLQ_REQUIRE(!(zeros_mode != LB_ZEROS_NONE && (!scales || !zeros)), "%s: zeros_mode needs scales and zeros", me);
  TLQ_REQUIRE(!(out_bits != 16 && (scales || zeros_mode != LB_ZEROS_NONE)), "%s: the integer targets take no scales / zeros", me);
  if (n_units == 0) return 0;
  TLQ_REQUIRE(src && out, "%s: null pointer", me);
  // bytes of source per unit: 8 outputs (fp16 target) or 16 outputs (integer targets) x source_bit bits
  const int src_bytes = (out_bits == 16 ? 8 : 16) * source_bit / 8;
  TLQ_REQUIRE(((uintptr_t)src & (uintptr_t)(src_bytes - 1)) == 0 && ((uintptr_t)out & (out_bits == 4 ? 7 : 15)) == 0 &&
                  ((uintptr_t)scales & 1) == 0 && ((uintptr_t)zeros & 1) == 0, "%s: misaligned pointer", me);
  TLQ_REQUIRE(!scales || (units_per_group > 0 && units_per_group < ((int64_t)1 << 31)), "%s: units_per_group must be positive", me);
  hipStream_t st = (hipStream_t)stream;
  const int upg = scales ? (int)units_per_group : 1;
  if (out_bits == 16) {
    if (source_bit == 2)
      launch_f16<2>((const uint8_t*)src, (const half_t*)scales, zeros, (uint4_t*)out, n_units, upg, is_signed != 0, zeros_mode, st);
    else
      launch_f16<1>((const uint8_t*)src, (const half_t*)scales, zeros, (uint4_t*)out, n_units, upg, is_signed != 0, zeros_mode, st);
  } else if (out_bits == 8) {
    const int g = lb_grid_for(n_units);
    if (source_bit == 2) {
      if (is_signed) decode_lowbit_i8_kernel<2, true><<<g, 256, 0, st>>>((const uint8_t*)src, (uint4_t*)out, n_units);
      else decode_lowbit_i8_kernel<2, false><<<g, 256, 0, st>>>((const uint8_t*)src, (uint4_t*)out, n_units);
    } else {
      if (is_signed) decode_lowbit_i8_kernel<1, true><<<g, 256, 0, st>>>((const uint8_t*)src, (uint4_t*)out, n_units);
      else decode_lowbit_i8_kernel<1, false><<<g, 256, 0, st>>>((const uint8_t*)src, (uint4_t*)out, n_units);
    }
  } else {
    const int g = lb_grid_for(n_units);
    if (is_signed) decode_i2_i4_kernel<true><<<g, 256, 0, st>>>((const uint32_t*)src, (uint2_t*)out, n_units);
    else decode_i2_i4_kernel<false><<<g, 256, 0, st>>>((const uint32_t*)src, (uint2_t*)out, n_units);
  }
  return check_launch(me) ? 0 : 1;
}
