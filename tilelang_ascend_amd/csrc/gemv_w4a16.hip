// Decode GEMV / skinny GEMM for packed-int4 weights (M <= 16): HBM-bound.
//
//   C[m, n] = sum_k A[m, k] * W[n, k],   W[n, k] = (u[n, k] - z[n, k/g]) * s[n, k/g]
//
// Work split: one wavefront owns R consecutive weight rows.  K is split across the 64
// lanes in chunks of 32 weights (16 packed bytes): lane l takes chunks l, l+64, ...  so each
// wave-wide load instruction covers 1024 contiguous bytes of a row.  The chunk is unpacked
// in registers, multiplied with the matching activation slice and the 64 partial sums are
// combined with a cross-lane butterfly at the end (split-K inside the wavefront).
//
// fp16 path: two nibbles at a time are turned into a half2 with one v_and_or_b32
// ((x & 0x000f000f) | 0x64006400 = 1024+u, (x & 0x00f000f0) | 0x54005400 = 64+u), the bias
// is removed exactly with one packed subtract and v_dot2_f32_f16 accumulates in fp32.  Scale
// and zero point are applied once per chunk in fp32:  s * (sum A*u - z * sum A), which is
// at least as accurate as multiplying rounded fp16 weights.
// bf16 path: weights are dequantised element-wise with bfloat16 rounding after each step
// (bf16 keeps only 8 mantissa bits, so skipping those roundings would be visible).
#include "tlq_common.h"

namespace tlq {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// ---- fp16: activations kept as half2 pairs in the order the nibble unpack produces ----------
// pair p = 4*j + i of a 32-element chunk holds elements (8*j + i, 8*j + i + 4).
struct ActF16 {
  half2_t a[16];
  float sum;
};

__device__ __forceinline__ void load_act(ActF16& r, const half_t* __restrict__ A, int64_t off) {
  const uint4_t* p = (const uint4_t*)(A + off);
  float s = 0.f;
  const half2_t ones = {(half_t)1.0f, (half_t)1.0f};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    uint4_t v = p[j];  // elements 8j .. 8j+7 as (0,1)(2,3)(4,5)(6,7)
    half2_t q0 = bitcast<half2_t>(v.x), q1 = bitcast<half2_t>(v.y);
    half2_t q2 = bitcast<half2_t>(v.z), q3 = bitcast<half2_t>(v.w);
    r.a[4 * j + 0] = half2_t{q0.x, q2.x};
    r.a[4 * j + 1] = half2_t{q0.y, q2.y};
    r.a[4 * j + 2] = half2_t{q1.x, q3.x};
    r.a[4 * j + 3] = half2_t{q1.y, q3.y};
#pragma unroll
    for (int i = 0; i < 4; ++i) s = __builtin_amdgcn_fdot2(r.a[4 * j + i], ones, s, false);
  }
  r.sum = s;
}

// sum over the chunk of A[k] * u[k] (u = raw nibble value), fp32
__device__ __forceinline__ float dot_chunk(const uint4_t& w, const ActF16& act) {
  const half2_t b1024 = {(half_t)1024.0f, (half_t)1024.0f};
  const half2_t b64 = {(half_t)64.0f, (half_t)64.0f};
  float acc = 0.f;
  const uint32_t x[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    uint32_t v = x[j];
    uint32_t v8 = v >> 8;
    half2_t p0 = bitcast<half2_t>(and_or(v, 0x000f000fu, 0x64006400u)) - b1024;   // (k0, k4)
    half2_t p1 = bitcast<half2_t>(and_or(v, 0x00f000f0u, 0x54005400u)) - b64;     // (k1, k5)
    half2_t p2 = bitcast<half2_t>(and_or(v8, 0x000f000fu, 0x64006400u)) - b1024;  // (k2, k6)
    half2_t p3 = bitcast<half2_t>(and_or(v8, 0x00f000f0u, 0x54005400u)) - b64;    // (k3, k7)
    acc = __builtin_amdgcn_fdot2(p0, act.a[4 * j + 0], acc, false);
    acc = __builtin_amdgcn_fdot2(p1, act.a[4 * j + 1], acc, false);
    acc = __builtin_amdgcn_fdot2(p2, act.a[4 * j + 2], acc, false);
    acc = __builtin_amdgcn_fdot2(p3, act.a[4 * j + 3], acc, false);
  }
  return acc;
}

__device__ __forceinline__ float chunk_term(const uint4_t& w, const ActF16& act, half_t s, half_t z) {
  float d = dot_chunk(w, act);
  return (float)s * (d - (float)z * act.sum);
}

// ---- bf16: activations as floats, element-wise exact dequantisation ----------------------------
struct ActBF16 {
  float a[32];
};

__device__ __forceinline__ void load_act(ActBF16& r, const bf16_t* __restrict__ A, int64_t off) {
  const uint4_t* p = (const uint4_t*)(A + off);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    uint4_t v = p[j];
    const uint32_t x[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      r.a[8 * j + 2 * i] = bitcast<float>(x[i] << 16);
      r.a[8 * j + 2 * i + 1] = bitcast<float>(x[i] & 0xffff0000u);
    }
  }
}

__device__ __forceinline__ float chunk_term(const uint4_t& w, const ActBF16& act, bf16_t s, bf16_t z) {
  const float sf = to_float(s), zf = to_float(z);
  const uint32_t x[4] = {w.x, w.y, w.z, w.w};
  float acc = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float u = (float)((x[j] >> (4 * i)) & 0xFu);
      float d = round_to_bf16(u - zf);
      float wv = round_to_bf16(d * sf);
      acc = __builtin_fmaf(act.a[8 * j + i], wv, acc);
    }
  }
  return acc;
}

template <typename T>
struct ActOf;
template <>
struct ActOf<half_t> {
  typedef ActF16 type;
};
template <>
struct ActOf<bf16_t> {
  typedef ActBF16 type;
};

// R weight rows per wavefront, MT activation rows per pass.
template <typename T, int R, int MT>
__global__ __launch_bounds__(256) void gemv_w4a16_kernel(const T* __restrict__ A, const uint8_t* __restrict__ Wp,
                                                         const T* __restrict__ scales, const T* __restrict__ zeros,
                                                         void* __restrict__ C, int m_count, int N, int K, int group,
                                                         float zero_scalar, int out_dtype) {
  typedef typename ActOf<T>::type Act;
  // blockIdx.y selects one of gridDim.y independent problems stacked contiguously
  {
    const int64_t b = blockIdx.y;
    const int64_t gsz = (int64_t)N * (K / group);
    A += b * m_count * K;
    Wp += b * N * (int64_t)(K >> 1);
    if (scales) scales += b * gsz;
    if (zeros) zeros += b * gsz;
    const int64_t coff = b * m_count * N;
    C = out_dtype == TLQ_F32 ? (void*)((float*)C + coff) : (void*)((uint16_t*)C + coff);
  }
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int waves_per_block = blockDim.x >> 6;
  const int row0 = (blockIdx.x * waves_per_block + wave) * R;
  if (row0 >= N) return;  // whole wavefront leaves together

  const int chunks = K >> 5;
  const int groups = K / group;
  const int64_t row_bytes = K >> 1;
  const T one = from_float<T>(1.0f);
  const T zs = from_float<T>(zero_scalar);

  int rows[R];
#pragma unroll
  for (int r = 0; r < R; ++r) rows[r] = (row0 + r < N) ? row0 + r : N - 1;  // clamp: loads stay in bounds

  for (int m0 = 0; m0 < m_count; m0 += MT) {
    float acc[R][MT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < MT; ++m) acc[r][m] = 0.f;

    for (int c = lane; c < chunks; c += 64) {
      uint4_t w[R];
      T s[R], z[R];
      const int g = (c << 5) / group;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        w[r] = *(const uint4_t*)(Wp + rows[r] * row_bytes + ((int64_t)c << 4));
        s[r] = scales ? scales[(int64_t)rows[r] * groups + g] : one;
        z[r] = zeros ? zeros[(int64_t)rows[r] * groups + g] : zs;
      }
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const int mm = (m0 + m < m_count) ? m0 + m : m_count - 1;
        Act act;
        load_act(act, A, (int64_t)mm * K + ((int64_t)c << 5));
#pragma unroll
        for (int r = 0; r < R; ++r) acc[r][m] += chunk_term(w[r], act, s[r], z[r]);
      }
    }

#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        float v = wave_sum(acc[r][m]);
        if (lane == 0 && row0 + r < N && m0 + m < m_count) store_out(C, (int64_t)(m0 + m) * N + row0 + r, v, out_dtype);
      }
  }
}

template <typename T, int R, int MT>
static void launch_gemv(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int batch, int M,
                        int N, int K, int group, float zero_scalar, int out_dtype, int waves_per_block, hipStream_t st) {
  const int rows_per_block = R * waves_per_block;
  const int blocks = (int)ceil_div(N, rows_per_block);
  gemv_w4a16_kernel<T, R, MT><<<dim3(blocks, batch), 64 * waves_per_block, 0, st>>>((const T*)A, (const uint8_t*)Wp, (const T*)scales,
                                                                     (const T*)zeros, C, M, N, K, group, zero_scalar,
                                                                     out_dtype);
}

// rows-per-wave / waves-per-block overrides for tuning runs (0 = automatic)
static int g_gemv_rows = 0, g_gemv_waves = 0;

int gemv_w4a16(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t batch, int64_t M,
               int64_t N, int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, hipStream_t st) {
  int R = g_gemv_rows ? g_gemv_rows : 2;
  int wpb = g_gemv_waves ? g_gemv_waves : 4;
  const bool f16 = in_dtype == TLQ_F16;
#define TLQ_GEMV_CASE(RR, MTT)                                                                                       \
  if (f16)                                                                                                           \
    launch_gemv<half_t, RR, MTT>(A, Wp, scales, zeros, C, (int)batch, (int)M, (int)N, (int)K, (int)group, zero_scalar, out_dtype, \
                                 wpb, st);                                                                           \
  else                                                                                                               \
    launch_gemv<bf16_t, RR, MTT>(A, Wp, scales, zeros, C, (int)batch, (int)M, (int)N, (int)K, (int)group, zero_scalar, out_dtype, \
                                 wpb, st)
  if (M == 1) {
    if (R == 1) {
      TLQ_GEMV_CASE(1, 1);
    } else if (R == 4) {
      TLQ_GEMV_CASE(4, 1);
    } else {
      TLQ_GEMV_CASE(2, 1);
    }
  } else {
    if (R >= 2) {
      TLQ_GEMV_CASE(2, 2);
    } else {
      TLQ_GEMV_CASE(1, 2);
    }
  }
#undef TLQ_GEMV_CASE
  return check_launch("tlq_gemm_w4a16(gemv)") ? 0 : 1;
}

}  // namespace tlq

extern "C" {
// Tuning hook used by the benchmark sweeps: rows per wavefront (1, 2, 4) and wavefronts per
// block (1..4) of the GEMV kernel; 0 restores the automatic choice.
void tlq_tune_gemv(int rows_per_wave, int waves_per_block) {
  tlq::g_gemv_rows = rows_per_wave;
  tlq::g_gemv_waves = (waves_per_block < 0 || waves_per_block > 4) ? 0 : waves_per_block;
}
}
