/* TEST INFRASTRUCTURE ONLY -- plain-C restatement of the reference's quantized-matmul
 * arithmetic.  Linked by the tests and by the cpu_baseline leg of the benchmark, never by
 * the shipped library.
 *
 * It is written independently of oracle/ref.py (scalar loops, its own float rounding
 * routine built on nearbyint) so that the two restatements check each other; both are
 * additionally pinned by the reference's [[0x12,0x34]] -> [2,1,4,3] vector, exhaustive
 * nibble tables and closed forms in the test-suite.
 *
 * Reference lines followed (paths relative to the reference checkout):
 *   orc_unpack_u4      examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:10-57
 *   orc_convert_s4     examples/dequantize_gemm/example_dequant_gemm_w4a8.py:124-145
 *   orc_dequant_w4     tilelang/quantize/lop3.py:135-175 ("original" zeros: (u - z) * s, one
 *                      rounding per operation) and tilelang/quantize/utils.py:33
 *   orc_gemm_w4a16     example_dequant_gemm_fine_grained.py:269-289 (fp32 accumulate, cast)
 *   orc_gemm_i8        example_dequant_gemm_fine_grained.py:292-312 (int32 accumulate)
 *   orc_rescale        examples/quant_batch_matmul/example_quant_batch_matmul.py:93-95 and
 *                      examples/deepseek_v4/int8_gemm.py:95-102 (sequential fp32 multiplies)
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

/* ---- correctly rounded conversion of a double to a small binary format (RNE) ---------- */
static double round_to_format(double x, int p, int emin, int emax) {
  if (x == 0.0 || isnan(x) || isinf(x)) return x;
  int e;
  (void)frexp(x, &e); /* x = m * 2^e, 0.5 <= |m| < 1 */
  int ex = e - 1;     /* x = m' * 2^ex, 1 <= |m'| < 2 */
  if (ex < emin) ex = emin;
  double ulp = ldexp(1.0, ex - (p - 1));
  double r = nearbyint(x / ulp) * ulp; /* default rounding mode: ties to even */
  double maxfinite = ldexp(2.0 - ldexp(1.0, -(p - 1)), emax);
  if (fabs(r) > maxfinite) r = (x > 0) ? INFINITY : -INFINITY;
  return r;
}
static double rn_f16(double x) { return round_to_format(x, 11, -14, 15); }
static double rn_bf16(double x) { return round_to_format(x, 8, -126, 127); }
static double rn_f32(double x) { return (double)(float)x; }

static uint16_t f16_bits(double v) { /* v already representable in binary16 */
  if (isnan(v)) return 0x7e00;
  uint16_t s = signbit(v) ? 0x8000 : 0;
  double a = fabs(v);
  if (isinf(a)) return s | 0x7c00;
  if (a == 0.0) return s;
  int e;
  double m = frexp(a, &e);
  int ex = e - 1;
  if (ex < -14) return s | (uint16_t)nearbyint(ldexp(a, 24));
  return s | (uint16_t)((ex + 15) << 10) | (uint16_t)nearbyint((m * 2.0 - 1.0) * 1024.0);
}
static double f16_val(uint16_t b) {
  int s = b >> 15, e = (b >> 10) & 31, m = b & 1023;
  double v = (e == 0) ? ldexp((double)m, -24) : (e == 31) ? (m ? NAN : INFINITY) : ldexp(1.0 + m / 1024.0, e - 15);
  return s ? -v : v;
}
static uint16_t bf16_bits(double v) { /* v already representable in bfloat16 */
  float f = (float)v;
  uint32_t u;
  memcpy(&u, &f, 4);
  return (uint16_t)(u >> 16);
}
static double bf16_val(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return (double)f;
}

/* kind: 0 = float16, 1 = bfloat16 */
static double rn_kind(double x, int kind) { return kind ? rn_bf16(x) : rn_f16(x); }
static uint16_t bits_kind(double v, int kind) { return kind ? bf16_bits(v) : f16_bits(v); }
static double val_kind(uint16_t b, int kind) { return kind ? bf16_val(b) : f16_val(b); }

/* ---- nibble unpack ------------------------------------------------------------------ */
/* out[n*K + k] = (Wp[n*K/2 + k/2] >> 4*(k%2)) & 15, as int8 (0..15) */
void orc_unpack_u4(const uint8_t* wp, int8_t* out, int64_t N, int64_t K) {
  for (int64_t n = 0; n < N; ++n)
    for (int64_t k = 0; k < K; ++k) {
      uint8_t val = wp[n * (K / 2) + k / 2];
      int pos = (int)(k % 2);
      out[n * K + k] = (int8_t)((val >> (pos * 4)) & 0xF);
    }
}
/* two's-complement: ((nibble << 4) as int8) >> 4 */
void orc_convert_s4(const uint8_t* wp, int8_t* out, int64_t N, int64_t K) {
  for (int64_t n = 0; n < N; ++n)
    for (int64_t k = 0; k < K; ++k) {
      int8_t val = (int8_t)wp[n * (K / 2) + k / 2];
      int pos = (int)(k % 2);
      int8_t sh = (int8_t)((val >> (pos * 4)) & 0xF);
      out[n * K + k] = (int8_t)(((int8_t)(sh << 4)) >> 4);
    }
}

/* ---- per-group dequantisation ------------------------------------------------------- */
/* out bits = rn_T( rn_T(u - z) * s ); scales/zeros are [N, K/group] bit patterns of T, or NULL
 * (scale 1, zero = zero_scalar). */
void orc_dequant_w4(const uint8_t* wp, const uint16_t* scales, const uint16_t* zeros, double zero_scalar,
                    uint16_t* out, int64_t N, int64_t K, int64_t group, int kind) {
  int64_t G = K / group;
  for (int64_t n = 0; n < N; ++n)
    for (int64_t k = 0; k < K; ++k) {
      double u = (double)((wp[n * (K / 2) + k / 2] >> (4 * (k % 2))) & 0xF);
      double z = zeros ? val_kind(zeros[n * G + k / group], kind) : rn_kind(zero_scalar, kind);
      double d = rn_kind(u - z, kind);
      if (scales) d = rn_kind(d * val_kind(scales[n * G + k / group], kind), kind);
      out[n * K + k] = bits_kind(d, kind);
    }
}

/* ---- W4A16 GEMM: C = rn_out( sum_k f32(A[m,k]) * f32(W[n,k]) ), fp32 accumulate ------- */
/* A: [M,K] bits of T; W: [N,K] bits of T (already dequantised); out_kind 0/1 = f16/bf16 bits
 * in C16, 2 = fp32 in C32. */
void orc_gemm_w4a16(const uint16_t* A, const uint16_t* W, void* C, int64_t M, int64_t N, int64_t K, int kind,
                    int out_kind) {
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k)
        acc += (float)val_kind(A[m * K + k], kind) * (float)val_kind(W[n * K + k], kind);
      if (out_kind == 2)
        ((float*)C)[m * N + n] = acc;
      else
        ((uint16_t*)C)[m * N + n] = bits_kind(rn_kind((double)acc, out_kind), out_kind);
    }
}

/* ---- int8 GEMM, int32 accumulate (wraps like the hardware would; never reached in tests) -- */
/* b_layout: 0 = B[K,N] (quant_batch_matmul), 1 = B[N,K] (transpose_B) */
void orc_gemm_i8(const int8_t* A, const int8_t* B, int32_t* C, int64_t M, int64_t N, int64_t K, int b_layout) {
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      int64_t acc = 0;
      for (int64_t k = 0; k < K; ++k) {
        int b = b_layout ? B[n * K + k] : B[k * N + n];
        acc += (int64_t)A[m * K + k] * b;
      }
      C[m * N + n] = (int32_t)acc;
    }
}

/* ---- rescale epilogue: out = rn_out( rn_f32( rn_f32(f32(acc) * sa[m]) * sb[n] ) ) -------- */
/* sa may be NULL (skipped); sb has n_sb entries (1 = per-tensor, N = per-channel). */
void orc_rescale(const int32_t* acc, const float* sa, const float* sb, int64_t n_sb, void* out, int64_t M, int64_t N,
                 int out_kind) {
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      double c = rn_f32((double)acc[m * N + n]);
      if (sa) c = rn_f32(c * (double)sa[m]);
      if (sb) c = rn_f32(c * (double)sb[n_sb == 1 ? 0 : n]);
      if (out_kind == 2)
        ((float*)out)[m * N + n] = (float)c;
      else
        ((uint16_t*)out)[m * N + n] = bits_kind(rn_kind(c, out_kind), out_kind);
    }
}

/* ---- per-token int8 activation quantiser (examples/deepseek_v4/act_quant.py:112-142) ----
 * x: float32 [M,N] (bf16 / fp16 inputs are widened by the caller, which is exact).
 * round_scale: smallest power of two >= amax / 127 (:93-105, exponent field plus "mantissa != 0"). */
void orc_act_quant(const float* x, int8_t* y, float* s, int64_t M, int64_t N, int round_scale) {
  for (int64_t m = 0; m < M; ++m) {
    float amax = 0.f;
    for (int64_t n = 0; n < N; ++n) amax = fmaxf(amax, fabsf(x[m * N + n]));
    if (amax < 1e-4f) amax = 1e-4f;
    float sc = amax / 127.0f;
    if (round_scale) {
      uint32_t b;
      memcpy(&b, &sc, 4);
      uint32_t e = ((b >> 23) & 0xffu) + ((b & 0x7fffffu) != 0);
      b = e << 23;
      memcpy(&sc, &b, 4);
    }
    s[m] = sc;
    for (int64_t n = 0; n < N; ++n) {
      float q = x[m * N + n] / sc;
      q = q < -127.f ? -127.f : (q > 127.f ? 127.f : q);
      y[m * N + n] = (int8_t)nearbyintf(q); /* default rounding mode: to nearest, ties to even */
    }
  }
}

/* Checker for the division-free quotient the HIP kernel uses: q0 = x * r, q = fma(fma(-q0, s, x), r, q0)
 * with r = fl(1 / s).  Draws n pseudo-random (x, s) pairs, a third of them within two ulp of a tie
 * (k + 1/2) * s, and counts the pairs whose clamped, rounded integer differs from that of x / s.
 * quotient_mismatches receives the count of raw quotients that differ in any bit. */
int64_t orc_act_quant_quotient_check(int64_t n, uint64_t seed, int64_t* quotient_mismatches) {
  uint64_t st = seed ? seed : 88172645463325252ull;
  int64_t bad_int = 0, bad_q = 0;
#define ORC_RND() (st ^= st << 13, st ^= st >> 7, st ^= st << 17, st)
  for (int64_t i = 0; i < n; ++i) {
    uint32_t ea = 60 + (uint32_t)(ORC_RND() % 190), u = (ea << 23) | (uint32_t)(ORC_RND() & 0x7fffff);
    float amax, sc, x;
    memcpy(&amax, &u, 4);
    if (amax < 1e-4f) amax = 1e-4f;
    sc = amax / 127.0f;
    if (i & 1) {
      memcpy(&u, &sc, 4);
      u = (((u >> 23) & 0xffu) + ((u & 0x7fffffu) != 0)) << 23;
      memcpy(&sc, &u, 4);
    }
    if (i % 3 == 0) {
      x = ((float)(ORC_RND() % 128) + 0.5f) * sc;
      memcpy(&u, &x, 4);
      u += (uint32_t)(ORC_RND() % 5) - 2u;
      memcpy(&x, &u, 4);
    } else {
      uint32_t xb = (uint32_t)ORC_RND(), ex = (uint32_t)(ORC_RND() % (ea + 1));
      u = (ex << 23) | (xb & 0x7fffff);
      memcpy(&x, &u, 4);
    }
    if (x > amax) x = amax;
    if (ORC_RND() & 1) x = -x;
    const float r = 1.0f / sc, q_ref = x / sc, q0 = x * r;
    const float q = fmaf(fmaf(-q0, sc, x), r, q0);
    bad_q += q != q_ref;
    const float a = q_ref < -127.f ? -127.f : (q_ref > 127.f ? 127.f : q_ref);
    const float b = q < -127.f ? -127.f : (q > 127.f ? 127.f : q);
    bad_int += nearbyintf(a) != nearbyintf(b);
  }
#undef ORC_RND
  if (quotient_mismatches) *quotient_mismatches = bad_q;
  return bad_int;
}
