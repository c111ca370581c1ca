// Per-token (per-row) int8 activation quantiser, the step that feeds the W8A8 matmuls:
//   amax[m]  = max(max_n |x[m, n]|, 1e-4)
//   scale[m] = amax / 127                      (round_scale: the next power of two, 2^ceil(log2(amax / 127)))
//   y[m, n]  = int8( rint( clamp(x[m, n] / scale[m], -127, 127) ) )      rint = round half to even
// HBM bound: one wavefront (many rows) or one work-group (few or long rows) owns a row, reads it once
// into registers with 16-byte loads, reduces the maximum across lanes, and writes 8 int8 per lane and
// chunk.  Rows longer than 32768 values, or of a length that is no multiple of 8, are read twice.
#include "tlq_common.h"

namespace tlq {

template <>
__device__ __forceinline__ float to_float<float>(float v) {
  return v;
}

// Eight consecutive values, kept as loaded (16 or 32 bytes) and widened to float on use.  The input is read once:
// non-temporal loads (M = 16384, N = 4096: 38.2 instead of 40.0 us; with the resident grid 36.1 us).  The output is
// stored normally: non-temporal stores save another microsecond here and cost the W8A8 GEMM that reads the output next
// 4 - 14 us (16384 x 4096 x 4096: quantiser + GEMM 291 against 279 us).
template <typename T>
struct Raw8;
template <>
struct Raw8<half_t> {
  half8_t v;
  __device__ __forceinline__ void load(const half_t* p) { v = __builtin_nontemporal_load((const half8_t*)p); }
  __device__ __forceinline__ float get(int i) const { return (float)v[i]; }
};
template <>
struct Raw8<bf16_t> {
  uint32_t w[4];
  __device__ __forceinline__ void load(const bf16_t* p) {
    const uint4_t q = __builtin_nontemporal_load((const uint4_t*)p);
    w[0] = q.x, w[1] = q.y, w[2] = q.z, w[3] = q.w;
  }
  __device__ __forceinline__ float get(int i) const {
    return bitcast<float>((i & 1) ? (w[i >> 1] & 0xffff0000u) : (w[i >> 1] << 16));
  }
};
template <>
struct Raw8<float> {
  float4_t a, b;
  __device__ __forceinline__ void load(const float* p) {
    a = __builtin_nontemporal_load((const float4_t*)p);
    b = __builtin_nontemporal_load((const float4_t*)(p + 4));
  }
  __device__ __forceinline__ float get(int i) const { return i < 4 ? a[i] : b[i - 4]; }
};

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

__device__ __forceinline__ float row_scale(float amax, int round_scale) {
  amax = fmaxf(amax, 1e-4f);
  const float s = amax / 127.0f;
  if (!round_scale) return s;
  // 2^ceil(log2(s)) from the bits of s: exponent, plus one when any mantissa bit is set
  const uint32_t bits = bitcast<uint32_t>(s);
  const int e = (int)((bits >> 23) & 0xff) - 127 + ((bits & 0x7fffffu) ? 1 : 0);
  return bitcast<float>((uint32_t)(e + 127) << 23);
}

// x / scale, correctly rounded wherever the quotient matters, from the row's reciprocal
// rcp = fl(1 / scale): q0 = x * rcp is within an ulp, the remainder x - q0 * scale is exact in one
// fma, and one more fma lands on the correctly rounded quotient.  (Only when the remainder
// underflows, |x| < 2^-100 or so, can the last bit differ; such quotients round to 0 either way.)
__device__ __forceinline__ uint32_t quant1(float x, float scale, float rcp) {
  const float q0 = x * rcp;
  const float q1 = __builtin_fmaf(__builtin_fmaf(-q0, scale, x), rcp, q0);
  const float q = __builtin_rintf(fminf(fmaxf(q1, -127.0f), 127.0f));
  return (uint32_t)(int)q & 0xffu;
}

// N % 8 == 0.  WPR wavefronts of a 256-lane work-group share one row (1: four rows per work-group,
// 4: one row); a lane keeps CH chunks of 8 values, so the row length is at most 512 * WPR * CH.
template <typename T, int CH, int WPR>
__global__ __launch_bounds__(256) void act_quant_rows_kernel(const T* __restrict__ X, int8_t* __restrict__ Y,
                                                            float* __restrict__ S, int64_t M, int N, int round_scale) {
  __shared__ float part[2][4];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  constexpr int RPB = 4 / WPR;  // rows per work-group
  const int sub = WPR == 1 ? 0 : wv, lanes = 64 * WPR;
  const int chunks = N >> 3;
  int it = 0;
  // every wavefront of a work-group runs the same number of iterations (the barrier below needs that)
  for (int64_t m0 = (int64_t)blockIdx.x * RPB; m0 < M; m0 += (int64_t)gridDim.x * RPB, it ^= 1) {
    const int64_t m = m0 + (WPR == 1 ? wv : 0);
    const bool live = m < M;
    const T* x = X + m * N;
    Raw8<T> r[CH];
    float amax = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int ci = c * lanes + sub * 64 + lane;
      if (live && ci < chunks) {
        r[c].load(x + ci * 8);
#pragma unroll
        for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(r[c].get(i)));
      }
    }
    amax = wave_max(amax);
    if constexpr (WPR > 1) {
      if (lane == 0) part[it][wv] = amax;
      __syncthreads();  // part[] alternates between iterations, so one barrier per row is enough
      amax = fmaxf(fmaxf(part[it][0], part[it][1]), fmaxf(part[it][2], part[it][3]));
    }
    const float scale = row_scale(amax, round_scale);
    const float rcp = 1.0f / scale;
    if (live && lane == 0 && sub == 0) S[m] = scale;
    int8_t* y = Y + m * N;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int ci = c * lanes + sub * 64 + lane;
      if (live && ci < chunks) {
        uint2_t o;
        o.x = quant1(r[c].get(0), scale, rcp) | quant1(r[c].get(1), scale, rcp) << 8 | quant1(r[c].get(2), scale, rcp) << 16 |
              quant1(r[c].get(3), scale, rcp) << 24;
        o.y = quant1(r[c].get(4), scale, rcp) | quant1(r[c].get(5), scale, rcp) << 8 | quant1(r[c].get(6), scale, rcp) << 16 |
              quant1(r[c].get(7), scale, rcp) << 24;
        *(uint2_t*)(y + ci * 8) = o;  // plain store: the GEMM that follows finds the output in the last-level cache
      }
    }
  }
}

// Any N: two passes over the row, one value per lane and step.
template <typename T>
__global__ __launch_bounds__(256) void act_quant_generic_kernel(const T* __restrict__ X, int8_t* __restrict__ Y,
                                                               float* __restrict__ S, int64_t M, int64_t N,
                                                               int round_scale) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int64_t waves = (int64_t)gridDim.x * (blockDim.x >> 6);
  for (int64_t m = wave; m < M; m += waves) {
    const T* x = X + m * N;
    float amax = 0.f;
    for (int64_t n = lane; n < N; n += 64) amax = fmaxf(amax, fabsf(to_float(x[n])));
    amax = wave_max(amax);
    const float scale = row_scale(amax, round_scale);
    if (lane == 0) S[m] = scale;
    int8_t* y = Y + m * N;
    for (int64_t n = lane; n < N; n += 64) {
      const float q = __builtin_rintf(fminf(fmaxf(to_float(x[n]) / scale, -127.0f), 127.0f));
      y[n] = (int8_t)(int)q;
    }
  }
}

template <typename T, int WPR>
static void launch_rows(const T* X, int8_t* Y, float* S, int64_t M, int N, int round_scale, int per_lane,
                        hipStream_t st) {
  // a resident grid (eight work-groups per CU: every wavefront slot) that walks the rows, instead of a work-group per
  // four rows: 37.0 instead of 40.0 us at M = 16384, N = 4096 (4 and 12 per CU are slower)
  const int64_t want = ceil_div(M, (int64_t)(4 / WPR));
  int cus = tlq_device_cu_count();
  if (cus <= 0) cus = 256;
  const int blocks = (int)(want > (int64_t)cus * 8 ? (int64_t)cus * 8 : want);
#define TLQ_AQ(CH) act_quant_rows_kernel<T, CH, WPR><<<blocks, 256, 0, st>>>(X, Y, S, M, N, round_scale)
  if (per_lane <= 1) TLQ_AQ(1);
  else if (per_lane <= 2) TLQ_AQ(2);
  else if (per_lane <= 4) TLQ_AQ(4);
  else if (per_lane <= 8) TLQ_AQ(8);
  else TLQ_AQ(16);
#undef TLQ_AQ
}

template <typename T>
static int run_act_quant(const void* Xv, void* Yv, void* Sv, int64_t M, int64_t N, int round_scale, hipStream_t st) {
  const T* X = (const T*)Xv;
  int8_t* Y = (int8_t*)Yv;
  float* S = (float*)Sv;
  const bool vec = N % 8 == 0 && ((uintptr_t)X & 15) == 0 && ((uintptr_t)Y & 7) == 0 && N <= 512 * 4 * 16;
  if (vec) {
    // one wavefront per row while a lane then holds at most 8 chunks and there are rows enough to
    // fill the chip that way; otherwise the four wavefronts of a work-group split the row
    const int per_lane1 = (int)ceil_div(N, (int64_t)512);
    const int cap1 = sizeof(T) == 4 ? 4 : 8;
    if (per_lane1 <= cap1 && M >= 4096)
      launch_rows<T, 1>(X, Y, S, M, (int)N, round_scale, per_lane1, st);
    else
      launch_rows<T, 4>(X, Y, S, M, (int)N, round_scale, (int)ceil_div(N, (int64_t)2048), st);
  } else {
    const int64_t want = ceil_div(M, (int64_t)4);
    act_quant_generic_kernel<T><<<(int)(want > 65536 ? 65536 : want), 256, 0, st>>>(X, Y, S, M, N, round_scale);
  }
  return check_launch("tlq_act_quant_i8", "act_quant kernel") ? 0 : 1;
}

}  // namespace tlq

using namespace tlq;

extern "C" int tlq_act_quant_i8(const void* X, void* Y, void* S, int64_t M, int64_t N, int in_dtype, int round_scale,
                                void* stream) {
  TLQ_REQUIRE(M >= 0 && N >= 0 && M < ((int64_t)1 << 40) && N < ((int64_t)1 << 31), "tlq_act_quant_i8: bad shape M=%lld N=%lld",
              (long long)M, (long long)N);
  TLQ_REQUIRE(in_dtype == TLQ_F16 || in_dtype == TLQ_BF16 || in_dtype == TLQ_F32,
              "tlq_act_quant_i8: in_dtype must be float16, bfloat16 or float32 (got %d)", in_dtype);
  if (M == 0) return 0;
  TLQ_REQUIRE(N > 0, "tlq_act_quant_i8: rows are empty");
  TLQ_REQUIRE(X && Y && S, "tlq_act_quant_i8: null pointer");
  TLQ_REQUIRE(((uintptr_t)S & 3) == 0 && ((uintptr_t)X & (in_dtype == TLQ_F32 ? 3 : 1)) == 0, "tlq_act_quant_i8: misaligned pointer");
  hipStream_t st = (hipStream_t)stream;
  if (in_dtype == TLQ_F16) return run_act_quant<half_t>(X, Y, S, M, N, round_scale, st);
  if (in_dtype == TLQ_BF16) return run_act_quant<bf16_t>(X, Y, S, M, N, round_scale, st);
  return run_act_quant<float>(X, Y, S, M, N, round_scale, st);
}
