// Stand-alone kernel around the interleaved-weight fast decoders (decode_i4.h): one lane decodes
// one 32-bit word (8 weights -> 16 bytes of fp16) or two words (16 weights -> 16 bytes of int8).
#include "decode_i4.h"
#include "tlq_common.h"

namespace tlq {

enum { ZEROS_NONE = 0, ZEROS_ORIGINAL = 1, ZEROS_RESCALE = 2, ZEROS_QUANTIZED = 3 };

template <bool SIGNED, bool SCALE, int ZMODE>
__global__ __launch_bounds__(256) void decode_i4_f16_kernel(const uint32_t* __restrict__ words,
                                                            const half_t* __restrict__ scales,
                                                            const void* __restrict__ zeros, uint4_t* __restrict__ out,
                                                            int64_t n_words, int words_per_group) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_words; i += (int64_t)gridDim.x * blockDim.x) {
    uint32_t w = words[i];
    const int64_t g = i / words_per_group;
    uint4_t r;
    if (ZMODE == ZEROS_ORIGINAL) {
      tlq_decode::decode_i4u_to_f16_scale_zeros_original(&w, &r, scales + g, (const half_t*)zeros + g);
    } else if (ZMODE == ZEROS_RESCALE) {
      tlq_decode::decode_i4u_to_f16_scale_zeros_rescale(&w, &r, scales + g, (const half_t*)zeros + g);
    } else if (ZMODE == ZEROS_QUANTIZED) {
      tlq_decode::decode_i4u_to_f16_scale_zeros_quantized(&w, &r, scales + g, (const int16_t*)zeros + g);
    } else if (SCALE) {
      if (SIGNED)
        tlq_decode::decode_i4s_to_f16_scale(&w, &r, scales + g);
      else
        tlq_decode::decode_i4u_to_f16_scale(&w, &r, scales + g);
    } else {
      if (SIGNED)
        tlq_decode::decode_i4s_to_f16(&w, &r);
      else
        tlq_decode::decode_i4u_to_f16(&w, &r);
    }
    out[i] = r;
  }
}

// The two-group forms: word i uses group g = i / words_per_group for its first four outputs and group g + offset for the
// last four.  With ZEROS_QUANTIZED the zero points are 4-bit fields of 32-bit words: field group_offset of word g and
// of word g + zero_offset.
template <bool SIGNED, int ZMODE>
__global__ __launch_bounds__(256) void decode_i4_f16_offset_kernel(const uint32_t* __restrict__ words,
                                                                   const half_t* __restrict__ scales,
                                                                   const void* __restrict__ zeros, uint4_t* __restrict__ out,
                                                                   int64_t n_words, int words_per_group, int offset,
                                                                   int zero_offset, int group_offset) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_words; i += (int64_t)gridDim.x * blockDim.x) {
    uint32_t w = words[i];
    const int64_t g = i / words_per_group;
    uint4_t r;
    if (ZMODE == ZEROS_ORIGINAL) {
      tlq_decode::decode_i4u_to_f16_scale_zeros_original_offset(&w, &r, scales + g, (const half_t*)zeros + g, offset);
    } else if (ZMODE == ZEROS_RESCALE) {
      tlq_decode::decode_i4u_to_f16_scale_zeros_rescale_offset(&w, &r, scales + g, (const half_t*)zeros + g, offset);
    } else if (ZMODE == ZEROS_QUANTIZED) {
      const uint32_t* wq = &w;
      tlq_decode::decode_i4u_to_f16_scale_zeros_quantized_offset(wq, &r, scales + g, (const uint32_t*)zeros + g, offset,
                                                                 zero_offset, group_offset);
    } else if (SIGNED) {
      tlq_decode::decode_i4s_to_f16_scale_offset(&w, &r, scales + g, offset);
    } else {
      tlq_decode::decode_i4u_to_f16_scale_offset(&w, &r, scales + g, offset);
    }
    out[i] = r;
  }
}

template <bool SIGNED>
__global__ __launch_bounds__(256) void decode_i4_i8_kernel(const uint2_t* __restrict__ words, uint4_t* __restrict__ out,
                                                           int64_t n_pairs) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_pairs; i += (int64_t)gridDim.x * blockDim.x) {
    uint2_t w = words[i];
    uint4_t r;
    if (SIGNED)
      tlq_decode::decode_i4s_to_i8s(&w, &r);
    else
      tlq_decode::decode_i4u_to_i8s(&w, &r);
    out[i] = r;
  }
}

static int grid_for(int64_t n) { return (int)(n + 255) / 256 > 65535 ? 65535 : (int)((n + 255) / 256); }

}  // namespace tlq

using namespace tlq;

extern "C" int tlq_decode_i4_interleaved(const void* words, const void* scales, const void* zeros, void* out,
                                         int64_t n_words, int64_t words_per_group, int out_dtype, int is_signed,
                                         int zeros_mode, void* stream) {
  TLQ_REQUIRE(n_words >= 0 && n_words < ((int64_t)1 << 40), "tlq_decode_i4_interleaved: bad n_words %lld", (long long)n_words);
  TLQ_REQUIRE(out_dtype == TLQ_F16 || out_dtype == TLQ_I8, "tlq_decode_i4_interleaved: out_dtype must be float16 or int8 (got %d)",
              out_dtype);
  TLQ_REQUIRE(zeros_mode >= ZEROS_NONE && zeros_mode <= ZEROS_QUANTIZED, "tlq_decode_i4_interleaved: bad zeros_mode %d",
              zeros_mode);
  TLQ_REQUIRE(!(zeros_mode != ZEROS_NONE && is_signed), "tlq_decode_i4_interleaved: zeros are not supported for signed sources");
  TLQ_REQUIRE(!(zeros_mode != ZEROS_NONE && (!scales || !zeros)), "tlq_decode_i4_interleaved: zeros_mode needs scales and zeros");
  TLQ_REQUIRE(!(out_dtype == TLQ_I8 && (scales || zeros_mode != ZEROS_NONE)),
              "tlq_decode_i4_interleaved: the int8 decoders take no scales / zeros");
  TLQ_REQUIRE(!(out_dtype == TLQ_I8 && n_words % 2), "tlq_decode_i4_interleaved: the int8 decoders need an even word count");
  if (n_words == 0) return 0;
  TLQ_REQUIRE(words && out, "tlq_decode_i4_interleaved: null pointer");
  TLQ_REQUIRE(((uintptr_t)words & 7) == 0 && ((uintptr_t)out & 15) == 0, "tlq_decode_i4_interleaved: misaligned pointer");
  TLQ_REQUIRE(!scales || words_per_group > 0, "tlq_decode_i4_interleaved: words_per_group must be positive");
  hipStream_t st = (hipStream_t)stream;
  const int wpg = scales ? (int)words_per_group : 1;
  const uint32_t* w = (const uint32_t*)words;
  const half_t* s = (const half_t*)scales;
  uint4_t* o = (uint4_t*)out;
  if (out_dtype == TLQ_I8) {
    const int64_t pairs = n_words / 2;
    if (is_signed)
      decode_i4_i8_kernel<true><<<grid_for(pairs), 256, 0, st>>>((const uint2_t*)words, o, pairs);
    else
      decode_i4_i8_kernel<false><<<grid_for(pairs), 256, 0, st>>>((const uint2_t*)words, o, pairs);
    return check_launch("tlq_decode_i4_interleaved") ? 0 : 1;
  }
  const int g = grid_for(n_words);
  switch (zeros_mode) {
    case ZEROS_ORIGINAL: decode_i4_f16_kernel<false, true, ZEROS_ORIGINAL><<<g, 256, 0, st>>>(w, s, zeros, o, n_words, wpg); break;
    case ZEROS_RESCALE: decode_i4_f16_kernel<false, true, ZEROS_RESCALE><<<g, 256, 0, st>>>(w, s, zeros, o, n_words, wpg); break;
    case ZEROS_QUANTIZED: decode_i4_f16_kernel<false, true, ZEROS_QUANTIZED><<<g, 256, 0, st>>>(w, s, zeros, o, n_words, wpg); break;
    default:
      if (scales) {
        if (is_signed)
          decode_i4_f16_kernel<true, true, ZEROS_NONE><<<g, 256, 0, st>>>(w, s, zeros, o, n_words, wpg);
        else
          decode_i4_f16_kernel<false, true, ZEROS_NONE><<<g, 256, 0, st>>>(w, s, zeros, o, n_words, wpg);
      } else {
        if (is_signed)
          decode_i4_f16_kernel<true, false, ZEROS_NONE><<<g, 256, 0, st>>>(w, s, zeros, o, n_words, wpg);
        else
          decode_i4_f16_kernel<false, false, ZEROS_NONE><<<g, 256, 0, st>>>(w, s, zeros, o, n_words, wpg);
      }
  }
  return check_launch("tlq_decode_i4_interleaved") ? 0 : 1;
}

extern "C" int tlq_decode_i4_interleaved_offset(const void* words, const void* scales, const void* zeros, void* out,
                                                int64_t n_words, int64_t words_per_group, int64_t n_scales, int64_t n_zeros,
                                                int offset, int zero_offset, int group_offset, int is_signed, int zeros_mode,
                                                void* stream) {
  const char* me = "tlq_decode_i4_interleaved_offset";
  TLQ_REQUIRE(n_words >= 0 && n_words < ((int64_t)1 << 40), "%s: bad n_words %lld", me, (long long)n_words);
  TLQ_REQUIRE(zeros_mode >= ZEROS_NONE && zeros_mode <= ZEROS_QUANTIZED, "%s: bad zeros_mode %d", me, zeros_mode);
  TLQ_REQUIRE(!(zeros_mode != ZEROS_NONE && is_signed), "%s: zeros are not supported for signed sources", me);
  TLQ_REQUIRE(scales != nullptr, "%s: the two-group decoders need scales", me);
  TLQ_REQUIRE(!(zeros_mode != ZEROS_NONE && !zeros), "%s: zeros_mode needs zeros", me);
  TLQ_REQUIRE(words_per_group > 0 && words_per_group < ((int64_t)1 << 31), "%s: words_per_group must be positive", me);
  TLQ_REQUIRE(offset >= 0 && zero_offset >= 0 && group_offset >= 0 && group_offset < 8,
              "%s: offsets must not be negative and group_offset must be in 0..7", me);
  if (n_words == 0) return 0;
  // every index the kernel forms: group of the last word, plus the offset of the second half
  const int64_t groups = (n_words + words_per_group - 1) / words_per_group;
  TLQ_REQUIRE(groups + offset <= n_scales, "%s: %lld groups + offset %d need %lld scales, got %lld", me, (long long)groups, offset,
              (long long)(groups + offset), (long long)n_scales);
  if (zeros_mode == ZEROS_ORIGINAL || zeros_mode == ZEROS_RESCALE)
    TLQ_REQUIRE(groups + offset <= n_zeros, "%s: %lld groups + offset %d need %lld zeros, got %lld", me, (long long)groups, offset,
                (long long)(groups + offset), (long long)n_zeros);
  if (zeros_mode == ZEROS_QUANTIZED)
    TLQ_REQUIRE(groups + zero_offset <= n_zeros, "%s: %lld groups + zero_offset %d need %lld words of zero points, got %lld", me,
                (long long)groups, zero_offset, (long long)(groups + zero_offset), (long long)n_zeros);
  TLQ_REQUIRE(words && out, "%s: null pointer", me);
  TLQ_REQUIRE(((uintptr_t)words & 3) == 0 && ((uintptr_t)out & 15) == 0 && ((uintptr_t)scales & 1) == 0 &&
                  ((uintptr_t)zeros & (zeros_mode == ZEROS_QUANTIZED ? 3 : 1)) == 0, "%s: misaligned pointer", me);
  hipStream_t st = (hipStream_t)stream;
  const uint32_t* w = (const uint32_t*)words;
  const half_t* s = (const half_t*)scales;
  uint4_t* o = (uint4_t*)out;
  const int g = grid_for(n_words), wpg = (int)words_per_group;
  switch (zeros_mode) {
    case ZEROS_ORIGINAL:
      decode_i4_f16_offset_kernel<false, ZEROS_ORIGINAL><<<g, 256, 0, st>>>(w, s, zeros, o, n_words, wpg, offset, zero_offset, group_offset);
      break;
    case ZEROS_RESCALE:
      decode_i4_f16_offset_kernel<false, ZEROS_RESCALE><<<g, 256, 0, st>>>(w, s, zeros, o, n_words, wpg, offset, zero_offset, group_offset);
      break;
    case ZEROS_QUANTIZED:
      decode_i4_f16_offset_kernel<false, ZEROS_QUANTIZED><<<g, 256, 0, st>>>(w, s, zeros, o, n_words, wpg, offset, zero_offset, group_offset);
      break;
    default:
      if (is_signed)
        decode_i4_f16_offset_kernel<true, ZEROS_NONE><<<g, 256, 0, st>>>(w, s, zeros, o, n_words, wpg, offset, zero_offset, group_offset);
      else
        decode_i4_f16_offset_kernel<false, ZEROS_NONE><<<g, 256, 0, st>>>(w, s, zeros, o, n_words, wpg, offset, zero_offset, group_offset);
  }
  return check_launch(me) ? 0 : 1;
}
