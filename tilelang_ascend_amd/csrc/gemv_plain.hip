// Plain (non-quantised) GEMV y[N] = A[N, K] . x[K] with fp32 accumulation, for fp16 / bf16 / fp32 operands.
// HBM bound: N * K elements are read once.  A work-group of up to 16 wavefronts owns a contiguous range of
// rows and copies x into LDS once; a wavefront takes two rows at a time and keeps four 16-byte loads per row
// and lane in flight.
#include "tlq_common.h"

namespace tlq {

template <typename T>
struct Dot16;  // fp32 dot product of two 16-byte operand pieces
template <>
struct Dot16<half_t> {
  static __device__ __forceinline__ float run(const uint4_t& a, const uint4_t& x, float acc) {
    acc = __builtin_amdgcn_fdot2(bitcast<half2_t>(a.x), bitcast<half2_t>(x.x), acc, false);
    acc = __builtin_amdgcn_fdot2(bitcast<half2_t>(a.y), bitcast<half2_t>(x.y), acc, false);
    acc = __builtin_amdgcn_fdot2(bitcast<half2_t>(a.z), bitcast<half2_t>(x.z), acc, false);
    acc = __builtin_amdgcn_fdot2(bitcast<half2_t>(a.w), bitcast<half2_t>(x.w), acc, false);
    return acc;
  }
};
template <>
struct Dot16<bf16_t> {
  static __device__ __forceinline__ float run(const uint4_t& a, const uint4_t& x, float acc) {
    const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, xw[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc = __builtin_fmaf(bitcast<float>(aw[i] << 16), bitcast<float>(xw[i] << 16), acc);
      acc = __builtin_fmaf(bitcast<float>(aw[i] & 0xffff0000u), bitcast<float>(xw[i] & 0xffff0000u), acc);
    }
    return acc;
  }
};
template <>
struct Dot16<float> {
  static __device__ __forceinline__ float run(const uint4_t& a, const uint4_t& x, float acc) {
    acc = __builtin_fmaf(bitcast<float>(a.x), bitcast<float>(x.x), acc);
    acc = __builtin_fmaf(bitcast<float>(a.y), bitcast<float>(x.y), acc);
    acc = __builtin_fmaf(bitcast<float>(a.z), bitcast<float>(x.z), acc);
    acc = __builtin_fmaf(bitcast<float>(a.w), bitcast<float>(x.w), acc);
    return acc;
  }
};

__device__ __forceinline__ float wave_sum_all(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// XLDS: x fits LDS (copied once per work-group); otherwise every piece of x is read through the caches.
template <typename T, bool XLDS>
__global__ __launch_bounds__(1024) void gemv_plain_kernel(const uint8_t* __restrict__ x, const uint8_t* __restrict__ A,
                                                         void* __restrict__ y, int N, int64_t row_bytes, int out_dtype,
                                                         int rows_per_block, int nwaves) {
  extern __shared__ __align__(16) uint8_t smem[];
  constexpr int U = 4, R = 2;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int chunks = (int)(row_bytes >> 4);  // 16-byte pieces per row
  const int r0 = blockIdx.x * rows_per_block;
  const int r1 = r0 + rows_per_block < N ? r0 + rows_per_block : N;
  if (XLDS) {
    for (int c = threadIdx.x; c < chunks; c += nwaves << 6) ((uint4_t*)smem)[c] = ((const uint4_t*)x)[c];
    __syncthreads();
  }
  const uint4_t* xs = XLDS ? (const uint4_t*)smem : (const uint4_t*)x;
  for (int row = r0 + wave * R; row < r1; row += nwaves * R) {
    float acc[R];
    const uint8_t* ap[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      acc[r] = 0.f;
      const int rr = row + r < r1 ? row + r : r1 - 1;  // clamp: the second row of the last pair may not exist
      ap[r] = A + (int64_t)rr * row_bytes;
    }
    for (int c0 = 0; c0 < chunks; c0 += 64 * U) {
      uint4_t a[R][U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int c = c0 + u * 64 + lane;
        const int cc = c < chunks ? c : chunks - 1;
#pragma unroll
        // the matrix is read once: non-temporal (N = 11008, K = 4096 fp16: 16.5 instead of 18.0 us)
        for (int r = 0; r < R; ++r) a[r][u] = __builtin_nontemporal_load((const uint4_t*)ap[r] + cc);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int c = c0 + u * 64 + lane;
        if (c < chunks) {
          const uint4_t xv = xs[c];
#pragma unroll
          for (int r = 0; r < R; ++r) acc[r] = Dot16<T>::run(a[r][u], xv, acc[r]);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float v = wave_sum_all(acc[r]);
      if (lane == 0 && row + r < r1) store_out(y, row + r, v, out_dtype);
    }
  }
}

static int cu_count_plain() {
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
    n = 256;
  return n;
}

template <typename T>
static int run_gemv_plain(const void* x, const void* A, void* y, int64_t N, int64_t K, int out_dtype, hipStream_t st) {
  const int64_t row_bytes = K * (int64_t)sizeof(T);
  const int nwaves = 16;
  int blocks = cu_count_plain() * (row_bytes >= 32768 ? 2 : 1);
  int rpb = (int)ceil_div(N, (int64_t)blocks);
  if (rpb < 2) rpb = 2;
  blocks = (int)ceil_div(N, (int64_t)rpb);
  const bool xlds = row_bytes <= 64 * 1024;
  if (xlds)
    gemv_plain_kernel<T, true><<<blocks, 64 * nwaves, (size_t)row_bytes, st>>>((const uint8_t*)x, (const uint8_t*)A, y, (int)N,
                                                                          row_bytes, out_dtype, rpb, nwaves);
  else
    gemv_plain_kernel<T, false><<<blocks, 64 * nwaves, 0, st>>>((const uint8_t*)x, (const uint8_t*)A, y, (int)N, row_bytes,
                                                               out_dtype, rpb, nwaves);
  return check_launch("tlq_gemv") ? 0 : 1;
}

}  // namespace tlq

using namespace tlq;

extern "C" int tlq_gemv(const void* x, const void* A, void* y, int64_t N, int64_t K, int dtype, int out_dtype, void* stream) {
  TLQ_REQUIRE(N >= 0 && K >= 0 && N < ((int64_t)1 << 31) && K < ((int64_t)1 << 31), "tlq_gemv: bad shape N=%lld K=%lld",
              (long long)N, (long long)K);
  TLQ_REQUIRE(dtype == TLQ_F16 || dtype == TLQ_BF16 || dtype == TLQ_F32, "tlq_gemv: dtype must be float16, bfloat16 or float32 (got %d)", dtype);
  TLQ_REQUIRE(out_dtype == TLQ_F16 || out_dtype == TLQ_BF16 || out_dtype == TLQ_F32, "tlq_gemv: bad out_dtype %d", out_dtype);
  if (N == 0) return 0;
  const int64_t elem = dtype == TLQ_F32 ? 4 : 2;
  TLQ_REQUIRE(K > 0 && (K * elem) % 16 == 0, "tlq_gemv: a row of K=%lld values must be a positive multiple of 16 bytes", (long long)K);
  TLQ_REQUIRE(x && A && y, "tlq_gemv: null pointer");
  TLQ_REQUIRE((((uintptr_t)x | (uintptr_t)A) & 15) == 0, "tlq_gemv: x and A must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == TLQ_F16) return run_gemv_plain<half_t>(x, A, y, N, K, out_dtype, st);
  if (dtype == TLQ_BF16) return run_gemv_plain<bf16_t>(x, A, y, N, K, out_dtype, st);
  return run_gemv_plain<float>(x, A, y, N, K, out_dtype, st);
}
