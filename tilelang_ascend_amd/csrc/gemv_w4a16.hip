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
// fp16 path: two nibbles at a time are turned into a half2 with one v_bfi_b32
// ((x & 0x000f000f) | 0x64006400 = 1024+u, (x & 0x00f000f0) | 0x54005400 = 64+u), the bias
// is removed exactly with one packed subtract and v_dot2_f32_f16 accumulates in fp32.  Scale
// and zero point are applied once per chunk in fp32:  s * (sum A*u - z * sum A), which is
// at least as accurate as multiplying rounded fp16 weights.
// bf16 path: weights are dequantised element-wise with bfloat16 rounding after each step
// (bf16 keeps only 8 mantissa bits, so skipping those roundings would be visible).
#include <type_traits>

#include "tlq_common.h"
#include "expand8.h"
#include "gemm_addr.h"

namespace tlq {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// Sum over the 64 lanes with DPP moves (no LDS traffic); the total lands in lane 63.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, bitcast<int>(v), CTRL, ROW_MASK, 0xf, false);
  return v + bitcast<float>(moved);
}
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
  v = dpp_add<0xB1, 0xf>(v);   // quad_perm [1,0,3,2]
  v = dpp_add<0x4E, 0xf>(v);   // quad_perm [2,3,0,1]
  v = dpp_add<0x141, 0xf>(v);  // row_half_mirror
  v = dpp_add<0x140, 0xf>(v);  // row_mirror: every lane of a row holds the row total
  v = dpp_add<0x142, 0xa>(v);  // row_bcast15 into rows 1 and 3
  v = dpp_add<0x143, 0xc>(v);  // row_bcast31 into rows 2 and 3
  return v;
}

// ---- fp16: activations kept as half2 pairs in the order the nibble unpack produces ----------
// pair p = 4*j + i of a 32-element chunk holds elements (8*j + i, 8*j + i + 4).
struct ActF16 {
  half2_t a[16];
  float sum;   // sum of the 32 activations
  float bsum;  // 1024 * (sum over even k) + 64 * (sum over odd k): what the unpack bias adds to the dot
};

__device__ __forceinline__ void load_act(ActF16& r, const half_t* __restrict__ A, int64_t off) {
  const uint4_t* p = (const uint4_t*)(A + off);
  float s = 0.f, se = 0.f;
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
    se = __builtin_amdgcn_fdot2(r.a[4 * j + 0], ones, se, false);  // pairs 0 and 2 hold the even k
    se = __builtin_amdgcn_fdot2(r.a[4 * j + 2], ones, se, false);
  }
  r.sum = s;
  r.bsum = 1024.0f * se + 64.0f * (s - se);
}

// the same from four 16-byte words already loaded.  LAYOUT 1: the weight words went through interleave_weight for the fp16
// target (nibbles hold elements 0, 2, 4, 6, 1, 3, 5, 7): the pair that the low / high nibble mask picks out of a word and of
// the word shifted by 8 is then (0, 1), (2, 3), (4, 5), (6, 7) -- the activations as they lie in memory; pairs 0 and 2 are
// still the ones that carry the bias 1024.
template <int LAYOUT = 0>
__device__ __forceinline__ void permute_act(ActF16& r, const uint4_t (&p)[4]) {
  float s = 0.f, se = 0.f;
  const half2_t ones = {(half_t)1.0f, (half_t)1.0f};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint4_t v = p[j];
    half2_t q0 = bitcast<half2_t>(v.x), q1 = bitcast<half2_t>(v.y);
    half2_t q2 = bitcast<half2_t>(v.z), q3 = bitcast<half2_t>(v.w);
    if (LAYOUT == 1) {
      r.a[4 * j + 0] = q0;
      r.a[4 * j + 1] = q1;
      r.a[4 * j + 2] = q2;
      r.a[4 * j + 3] = q3;
    } else {
      r.a[4 * j + 0] = half2_t{q0.x, q2.x};
      r.a[4 * j + 1] = half2_t{q0.y, q2.y};
      r.a[4 * j + 2] = half2_t{q1.x, q3.x};
      r.a[4 * j + 3] = half2_t{q1.y, q3.y};
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) s = __builtin_amdgcn_fdot2(r.a[4 * j + i], ones, s, false);
    se = __builtin_amdgcn_fdot2(r.a[4 * j + 0], ones, se, false);
    se = __builtin_amdgcn_fdot2(r.a[4 * j + 2], ones, se, false);
  }
  r.sum = s;
  r.bsum = 1024.0f * se + 64.0f * (s - se);
}

// Sum over the chunk of A[k] * (bias_k + u[k]) with the unpack bias left in (1024 for even k,
// 64 for odd k); the caller subtracts act.bsum.  fp32 accumulation keeps the cancellation error
// near 1e-5 relative, far below the fp16 output rounding.
__device__ __forceinline__ float dot_chunk_biased(const uint4_t& w, const ActF16& act, const NibbleMagic& mg) {
  float acc = 0.f;
  const uint32_t x[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t v = x[j];
    const uint32_t v8 = v >> 8;
    acc = __builtin_amdgcn_fdot2(bitcast<half2_t>(bfi(mg.m_lo, v, mg.b_lo)), act.a[4 * j + 0], acc, false);
    acc = __builtin_amdgcn_fdot2(bitcast<half2_t>(bfi(mg.m_hi, v, mg.b_hi)), act.a[4 * j + 1], acc, false);
    acc = __builtin_amdgcn_fdot2(bitcast<half2_t>(bfi(mg.m_lo, v8, mg.b_lo)), act.a[4 * j + 2], acc, false);
    acc = __builtin_amdgcn_fdot2(bitcast<half2_t>(bfi(mg.m_hi, v8, mg.b_hi)), act.a[4 * j + 3], acc, false);
  }
  return acc;
}

// sum over the chunk of A[k] * u[k] (u = raw nibble value), fp32
__device__ __forceinline__ float dot_chunk(const uint4_t& w, const ActF16& act) {
  const NibbleMagic mg = make_nibble_magic();
  const half2_t b1024 = {(half_t)1024.0f, (half_t)1024.0f};
  const half2_t b64 = {(half_t)64.0f, (half_t)64.0f};
  float acc = 0.f;
  const uint32_t x[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    uint32_t v = x[j];
    uint32_t v8 = v >> 8;
    half2_t p0 = bitcast<half2_t>(bfi(mg.m_lo, v, mg.b_lo)) - b1024;   // (k0, k4)
    half2_t p1 = bitcast<half2_t>(bfi(mg.m_hi, v, mg.b_hi)) - b64;     // (k1, k5)
    half2_t p2 = bitcast<half2_t>(bfi(mg.m_lo, v8, mg.b_lo)) - b1024;  // (k2, k6)
    half2_t p3 = bitcast<half2_t>(bfi(mg.m_hi, v8, mg.b_hi)) - b64;    // (k3, k7)
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
// same value through the biased dot: s * (sum A*(bias+u) - sum A*bias - z * sum A)
__device__ __forceinline__ float chunk_term_biased(const uint4_t& w, const ActF16& act, half_t s, half_t z,
                                                   const NibbleMagic& mg) {
  const float d = dot_chunk_biased(w, act, mg);
  return (float)s * (d - __builtin_fmaf((float)z, act.sum, act.bsum));
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

// the same value with the weights dequantised eight at a time (Expand8: bf16((u - z) * s), exact) and the packed
// bf16 dot instruction; `a` holds the chunk's 32 activations in memory order
template <bool FOLD, int LAYOUT = 0>
__device__ __forceinline__ float chunk_term_dot2(const uint4_t& w, const uint4_t (&a)[4], bf16_t s, bf16_t z,
                                                 const NibbleMagic& mg) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  const Expand8<bf16_t, FOLD, LAYOUT> ex(s, z, mg);
  const uint32_t x[4] = {w.x, w.y, w.z, w.w};
  float acc = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint4_t e = ex(x[j]);  // (k0,k1)(k2,k3)(k4,k5)(k6,k7)
    acc = __builtin_amdgcn_fdot2_f32_bf16(bitcast<bf16x2_t>(e.x), bitcast<bf16x2_t>(a[j].x), acc, false);
    acc = __builtin_amdgcn_fdot2_f32_bf16(bitcast<bf16x2_t>(e.y), bitcast<bf16x2_t>(a[j].y), acc, false);
    acc = __builtin_amdgcn_fdot2_f32_bf16(bitcast<bf16x2_t>(e.z), bitcast<bf16x2_t>(a[j].z), acc, false);
    acc = __builtin_amdgcn_fdot2_f32_bf16(bitcast<bf16x2_t>(e.w), bitcast<bf16x2_t>(a[j].w), acc, false);
  }
  return acc;
}

// ---- fp16 kernel: persistent wavefronts, activations pre-processed once per block into LDS -----
// LDS layout for MT activation rows and `chunks` = K/32 chunks:
//   pairs[m][j][c]  uint4  (j = 0..3: pairs 4j..4j+3 of chunk c, in unpack order)   -> lane c reads 16 B
//   sums [m][c]     float2 (sum of the 32 activations of chunk c, bias correction of chunk c)
// so that consecutive lanes read consecutive 16-byte words (no bank conflicts).
//
// A wavefront walks over "steps": step (rg, it) covers R rows (row group rg) x one 16-byte chunk
// per lane (chunk it*64 + lane).  Row groups are dealt round-robin to all wavefronts of the grid.
// The loads of D steps are in flight per wavefront: a problem of a few tens of MB is latency
// bound (bytes in flight / memory latency), so every wavefront requests its first D KB before
// anything else and requests step s + D as soon as step s has been consumed.
template <int R, int MT, int D>
__global__ __launch_bounds__(256, 4) void gemv_w4a16_f16_kernel(const half_t* __restrict__ A,
                                                                const uint8_t* __restrict__ Wp,
                                                                const half_t* __restrict__ scales,
                                                                const half_t* __restrict__ zeros,
                                                                void* __restrict__ C, int m_count, int N, int K,
                                                                int group_shift, float zero_scalar, int out_dtype) {
  extern __shared__ __align__(16) uint8_t smem[];
  const int chunks = K >> 5;
  uint4_t* const lds_pairs = (uint4_t*)smem;                            // [MT][4][chunks]
  float2* const lds_sums = (float2*)(smem + (size_t)MT * chunks * 64);  // [MT][chunks]
  const int groups = K >> group_shift;
  {
    const int64_t b = blockIdx.y;
    const int64_t gsz = (int64_t)N * groups;
    A += b * m_count * K;
    Wp += b * N * (int64_t)(K >> 1);
    if (scales) scales += b * gsz;
    if (zeros) zeros += b * gsz;
    const int64_t coff = b * m_count * N;
    C = out_dtype == TLQ_F32 ? (void*)((float*)C + coff) : (void*)((uint16_t*)C + coff);
  }
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform: row pointers stay scalar
  const int waves_per_block = blockDim.x >> 6;
  const int wave_id = blockIdx.x * waves_per_block + wave;
  const int wave_count = gridDim.x * waves_per_block;
  const int row_groups = (N + R - 1) / R;
  const int row_bytes = K >> 1;
  const int iters = (chunks + 63) >> 6;  // chunk iterations per row
  const half_t one = (half_t)1.0f;
  const half_t zs = (half_t)zero_scalar;

  // Absent scale / zero tensors: read a valid dummy location (the activations) and discard the
  // value, so that the load sequence is branch free.
  const bool has_s = scales != nullptr, has_z = zeros != nullptr;
  const half_t* const sp = has_s ? scales : A;
  const half_t* const zp = has_z ? zeros : A;

  struct Stage {
    uint4_t w[R];
    half_t s[R], z[R];
  };
  struct Cursor {  // wave-uniform position in this wavefront's sequence of steps
    int rg, it;
  };
  auto advance = [&](Cursor& c) {
    if (++c.it == iters) {
      c.it = 0;
      c.rg += wave_count;
    }
  };
  auto issue = [&](Stage& st, const Cursor& at) {
    const int c = (at.it << 6) + lane;
    const bool ok = c < chunks;
    const int cc = ok ? c : chunks - 1;
    const int gi = (cc << 5) >> group_shift;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      int row = at.rg * R + r;
      row = row < N ? row : N - 1;  // clamp: loads stay in bounds
      st.w[r] = __builtin_nontemporal_load((const uint4_t*)(Wp + (uint32_t)(row * row_bytes + (cc << 4))));  // read once
      const uint32_t go = (uint32_t)(row * groups + gi);
      const half_t sv = sp[has_s ? go : 0u];
      const half_t zv = zp[has_z ? go : 0u];
      st.s[r] = ok ? (has_s ? sv : one) : (half_t)0.0f;  // a chunk past the end contributes 0
      st.z[r] = has_z ? zv : zs;
    }
  };

  const NibbleMagic mg = make_nibble_magic();
  Stage st[D];
  Cursor ic = {wave_id, 0};  // next step to request
  auto fill = [&]() {
#pragma unroll
    for (int d = 0; d < D; ++d)
      if (ic.rg < row_groups) {
        issue(st[d], ic);
        advance(ic);
      }
  };
  fill();  // the first weight loads go out before the activation staging

  for (int m0 = 0; m0 < m_count; m0 += MT) {
    if (m0 > 0) __syncthreads();  // previous pass has finished reading LDS
    for (int i = threadIdx.x; i < chunks * MT; i += blockDim.x) {
      const int m = (MT == 1) ? 0 : i / chunks;
      const int c = i - m * chunks;
      const int mm = (m0 + m < m_count) ? m0 + m : m_count - 1;
      ActF16 act;
      load_act(act, A, (int64_t)mm * K + (c << 5));
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint4_t v = {bitcast<uint32_t>(act.a[4 * j + 0]), bitcast<uint32_t>(act.a[4 * j + 1]),
                     bitcast<uint32_t>(act.a[4 * j + 2]), bitcast<uint32_t>(act.a[4 * j + 3])};
        lds_pairs[(m * 4 + j) * chunks + c] = v;
      }
      lds_sums[m * chunks + c] = make_float2(act.sum, act.bsum);
    }
    __syncthreads();

    if (m0 > 0) {
      ic = Cursor{wave_id, 0};
      fill();
    }
    float acc[R][MT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < MT; ++m) acc[r][m] = 0.f;

    Cursor cc = {wave_id, 0};  // step being consumed
    while (cc.rg < row_groups) {
#pragma unroll
      for (int d = 0; d < D; ++d) {
        if (cc.rg >= row_groups) break;
        int c = (cc.it << 6) + lane;
        c = c < chunks ? c : chunks - 1;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          ActF16 act;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const uint4_t v = lds_pairs[(m * 4 + j) * chunks + c];
            act.a[4 * j + 0] = bitcast<half2_t>(v.x);
            act.a[4 * j + 1] = bitcast<half2_t>(v.y);
            act.a[4 * j + 2] = bitcast<half2_t>(v.z);
            act.a[4 * j + 3] = bitcast<half2_t>(v.w);
          }
          const float2 sb = lds_sums[m * chunks + c];
          act.sum = sb.x;
          act.bsum = sb.y;
#pragma unroll
          for (int r = 0; r < R; ++r) acc[r][m] += chunk_term_biased(st[d].w[r], act, st[d].s[r], st[d].z[r], mg);
        }

        if (cc.it == iters - 1) {  // row group finished: reduce over the lanes and store
#pragma unroll
          for (int r = 0; r < R; ++r)
#pragma unroll
            for (int m = 0; m < MT; ++m) {
              const float v = wave_sum_to_lane63(acc[r][m]);
              const int row = cc.rg * R + r;
              if (lane == 63 && row < N && m0 + m < m_count) store_out(C, (int64_t)(m0 + m) * N + row, v, out_dtype);
              acc[r][m] = 0.f;
            }
        }
        advance(cc);
        if (ic.rg < row_groups) {  // the slot just consumed takes the step D ahead
          issue(st[d], ic);
          advance(ic);
        }
      }
    }
  }
}

// ---- fp16, M = 1, short rows: activations in registers --------------------------------------------
// For K <= 2048 * ITERS a lane meets the same ITERS chunks of the activation vector in every row, so
// each wavefront keeps them (permuted, with their sums) in registers.  The work-group is as large as
// the CU takes (up to 16 wavefronts) and owns a contiguous range of rows: it prepares the activations
// ONCE and copies the scales and zero points of its rows (contiguous in memory) into LDS with a few
// wide loads.  The path from L2 to the CUs carries about 15 TB/s on this part: a private copy of the
// activations per wavefront would put more bytes on it than the weights themselves, and one small
// gather per row and tensor costs about as much as a 1 KB weight load.
// A step is a whole row: ITERS 16-byte weight loads per lane.  D rows are in flight per wavefront; the
// staging loads (a few KB the first multiply waits for) are requested first, the first D rows right behind them
// (measured: 6.95 against 7.13 us per launch with the rows first; more rows in flight at the start, up to all of a
// launch's rows, only delay the staging data behind megabytes of weights and were 1 - 2 us slower).  The loop body
// is free of branches (rows past the end are clamped and their results dropped): the compiler then
// keeps exact counts of the loads in flight instead of draining them at every control-flow merge.
// Long rows (ITERS > 2) keep more activations per lane than a 16-wavefront work-group has registers for: those
// instances are built for work-groups of 8 wavefronts (MAXT = 512 threads, 256 registers per lane).
// fp16 multiplies the raw nibbles (unpack bias left in, corrected through the chunk sums); bf16 dequantises
// element by element exactly as the reference does -- bf16((u - z) * s) differs from the exact product in the
// 8th bit, more than the output tolerance allows -- and multiplies with the packed bf16 dot instruction.
template <typename T, int ITERS, int D>
__device__ __forceinline__ void gemv_rows_body(const T* __restrict__ A, const uint8_t* __restrict__ Wp,
                                               const T* __restrict__ scales, const T* __restrict__ zeros,
                                               void* __restrict__ C, int N, int K, int group_shift, float zero_scalar,
                                               int out_dtype, int rows_per_block, int nwaves) {
  constexpr bool F16 = sizeof(T) == 2 && __is_same(T, half_t);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int chunks = K >> 5;
  const int row_bytes = K >> 1;
  const int r0 = blockIdx.x * rows_per_block;
  const int r1 = r0 + rows_per_block < N ? r0 + rows_per_block : N;  // rows [r0, r1) belong to this work-group
  Wp += (int64_t)blockIdx.y * N * (int64_t)row_bytes;
  int cc[ITERS];
  bool ok[ITERS];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int c = (it << 6) + lane;
    ok[it] = c < chunks;
    cc[it] = ok[it] ? c : chunks - 1;
  }
  struct Stage {
    uint4_t w[ITERS];
  };
  auto issue = [&](Stage& st, int row) {
#pragma unroll
    for (int it = 0; it < ITERS; ++it)  // read once: non-temporal (24 weight sets per launch: 94.5 instead of 101.6 us)
      st.w[it] = __builtin_nontemporal_load((const uint4_t*)(Wp + (uint32_t)(row * row_bytes + (cc[it] << 4))));
  };
  Stage st[D];
  int irow = r0 + wave;  // next row to request

  extern __shared__ __align__(16) uint8_t smem[];
  const int groups = K >> group_shift;
  uint4_t* const lds_pairs = (uint4_t*)smem;                       // [4][chunks]
  float2* const lds_sums = (float2*)(smem + (size_t)chunks * 64);  // [chunks]
  T* const lds_s = (T*)(smem + (size_t)chunks * 72);               // [rows_per_block][groups]
  T* const lds_z = lds_s + rows_per_block * groups;                // [rows_per_block][groups] (16-byte aligned: see launcher)
  {
    const int64_t b = blockIdx.y;
    const int64_t gsz = (int64_t)N * groups;
    A += b * K;
    if (scales) scales += b * gsz;
    if (zeros) zeros += b * gsz;
    const int64_t coff = b * N;
    C = out_dtype == TLQ_F32 ? (void*)((float*)C + coff) : (void*)((uint16_t*)C + coff);
  }
  const bool has_s = scales != nullptr, has_z = zeros != nullptr;
  int gsel[ITERS];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) gsel[it] = (cc[it] << 5) >> group_shift;

  // staging loads: thread t < chunks fetches activation chunk t, and all threads copy the scale / zero rows,
  // 16 bytes (or one value) each
  const int tchunk = threadIdx.x < chunks ? threadIdx.x : chunks - 1;
  uint4_t araw[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) araw[j] = ((const uint4_t*)(A + ((int64_t)tchunk << 5)))[j];
  const int n_sz = (r1 - r0) * groups;  // values per tensor
  const int64_t sz0 = (int64_t)r0 * groups;
  // 16-byte pieces: every work-group's values (rows_per_block * groups of them from r0 * groups on, fewer in the last one)
  // and every problem's (N * groups) must be whole pieces -- 28 or 86 groups per row with rows in fours qualify
  const bool wide = ((rows_per_block * groups) & 7) == 0 && (((int64_t)N * groups) & 7) == 0 && (((uintptr_t)scales | (uintptr_t)zeros) & 15) == 0;
  uint4_t s_raw = {0, 0, 0, 0}, z_raw = {0, 0, 0, 0};
  const int t8 = threadIdx.x << 3;
  if (wide && t8 < n_sz) {  // a work-group of 1024 threads covers 8192 values per tensor in one go
    if (has_s) s_raw = *(const uint4_t*)(scales + sz0 + t8);
    if (has_z) z_raw = *(const uint4_t*)(zeros + sz0 + t8);
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int d = 0; d < D; ++d) {
    issue(st[d], irow < r1 ? irow : r1 - 1);
    irow += nwaves;
  }
  __builtin_amdgcn_sched_barrier(0);

  if (threadIdx.x < chunks) {
    if constexpr (F16) {
      ActF16 a;
      permute_act(a, araw);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        lds_pairs[j * chunks + tchunk] = uint4_t{bitcast<uint32_t>(a.a[4 * j + 0]), bitcast<uint32_t>(a.a[4 * j + 1]),
                                                 bitcast<uint32_t>(a.a[4 * j + 2]), bitcast<uint32_t>(a.a[4 * j + 3])};
      lds_sums[tchunk] = make_float2(a.sum, a.bsum);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) lds_pairs[j * chunks + tchunk] = araw[j];  // natural order, no sums needed
    }
  }
  if (wide) {
    if (t8 < n_sz) {
      if (has_s) *(uint4_t*)(lds_s + t8) = s_raw;
      if (has_z) *(uint4_t*)(lds_z + t8) = z_raw;
    }
    for (int i = t8 + (int)((nwaves << 6) << 3); i < n_sz; i += (int)((nwaves << 6) << 3)) {  // more than 8192 values
      if (has_s) *(uint4_t*)(lds_s + i) = *(const uint4_t*)(scales + sz0 + i);
      if (has_z) *(uint4_t*)(lds_z + i) = *(const uint4_t*)(zeros + sz0 + i);
    }
  } else {
    for (int i = threadIdx.x; i < n_sz; i += (nwaves << 6)) {
      if (has_s) lds_s[i] = scales[sz0 + i];
      if (has_z) lds_z[i] = zeros[sz0 + i];
    }
  }
  __syncthreads();
  ActF16 act[F16 ? ITERS : 1];      // fp16: pairs in unpack order and the chunk sums
  uint4_t actn[F16 ? 1 : ITERS][4];  // bf16: the 32 activations of a chunk as loaded
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    if constexpr (F16) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint4_t v = lds_pairs[j * chunks + cc[it]];
        act[it].a[4 * j + 0] = bitcast<half2_t>(v.x);
        act[it].a[4 * j + 1] = bitcast<half2_t>(v.y);
        act[it].a[4 * j + 2] = bitcast<half2_t>(v.z);
        act[it].a[4 * j + 3] = bitcast<half2_t>(v.w);
      }
      const float2 sb = lds_sums[cc[it]];
      act[it].sum = sb.x;
      act[it].bsum = sb.y;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) actn[it][j] = lds_pairs[j * chunks + cc[it]];
    }
  }

  const NibbleMagic mg = make_nibble_magic();
  const T one = from_float<T>(1.0f), zs = from_float<T>(zero_scalar);
  const int my_rows = r0 + wave < r1 ? (r1 - r0 - wave + nwaves - 1) / nwaves : 0;
  int row = r0 + wave;
  for (int round = 0; round * D < my_rows; ++round) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int lrow = (row < r1 ? row : r1 - 1) - r0;
      float acc = 0.f;
      if constexpr (F16) {
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
          const half_t sv = has_s ? lds_s[lrow * groups + gsel[it]] : one;
          const half_t z = has_z ? lds_z[lrow * groups + gsel[it]] : zs;
          const half_t s = ok[it] ? sv : (half_t)0.0f;  // a chunk past the end contributes 0
          acc += chunk_term_biased(st[d].w[it], act[it], s, z, mg);
        }
      } else {
        T sv[ITERS], zv[ITERS];
        bool integral = true;  // small integer zero points fold exactly into one fused multiply-add per weight
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
          const T s0 = has_s ? lds_s[lrow * groups + gsel[it]] : one;
          zv[it] = has_z ? lds_z[lrow * groups + gsel[it]] : zs;
          sv[it] = ok[it] ? s0 : from_float<T>(0.0f);
          const float zf = to_float(zv[it]);
          integral = integral && zf == __builtin_rintf(zf) && zf >= -256.0f && zf <= 256.0f;
        }
        if (__builtin_amdgcn_ballot_w64(integral) == ~0ull) {
#pragma unroll
          for (int it = 0; it < ITERS; ++it) acc += chunk_term_dot2<true>(st[d].w[it], actn[it], sv[it], zv[it], mg);
        } else {
#pragma unroll
          for (int it = 0; it < ITERS; ++it) acc += chunk_term_dot2<false>(st[d].w[it], actn[it], sv[it], zv[it], mg);
        }
      }
      const float v = wave_sum_to_lane63(acc);
      if (lane == 63 && row < r1) store_out(C, row, v, out_dtype);
      row += nwaves;
      issue(st[d], irow < r1 ? irow : r1 - 1);  // the slot just consumed takes the row D ahead
      irow += nwaves;
    }
  }
}

template <int ITERS, int D, int MAXT>
__global__ __launch_bounds__(MAXT) void gemv_w4a16_f16_rows_kernel(const half_t* __restrict__ A,
                                                                  const uint8_t* __restrict__ Wp,
                                                                  const half_t* __restrict__ scales,
                                                                  const half_t* __restrict__ zeros,
                                                                  void* __restrict__ C, int N, int K, int group_shift,
                                                                  float zero_scalar, int out_dtype, int rows_per_block,
                                                                  int nwaves) {
  gemv_rows_body<half_t, ITERS, D>(A, Wp, scales, zeros, C, N, K, group_shift, zero_scalar, out_dtype, rows_per_block, nwaves);
}

template <int ITERS, int D, int MAXT>
__global__ __launch_bounds__(MAXT) void gemv_w4a16_bf16_rows_kernel(const bf16_t* __restrict__ A,
                                                                   const uint8_t* __restrict__ Wp,
                                                                   const bf16_t* __restrict__ scales,
                                                                   const bf16_t* __restrict__ zeros,
                                                                   void* __restrict__ C, int N, int K, int group_shift,
                                                                   float zero_scalar, int out_dtype, int rows_per_block,
                                                                   int nwaves) {
  gemv_rows_body<bf16_t, ITERS, D>(A, Wp, scales, zeros, C, N, K, group_shift, zero_scalar, out_dtype, rows_per_block, nwaves);
}

// ---- ring kernel: the rows kernel's arithmetic with every global read a direct global -> LDS load ----
// Loads that return into registers move about 14 bytes per clock and CU through the address unit, direct loads about 30;
// a single problem of a few tens of MB is over before the stream settles, so the rate at which a CU can put its
// requests out is what its time depends on.  Here every wavefront asks for its first `D` rows (all of its rows for the
// shapes this is used for) before anything else happens, the staging data (activations, scales, zero points of the
// work-group's rows) travels the same way ahead of them, and a row is read back from the wavefront's private LDS slot
// by the lane that asked for it.  Same sums in the same order as the rows kernel: the results are the same bits.
// MT = 2 activation rows (fp16): a row's nibbles are expanded once and multiplied with both activation rows, whose
// prepared chunks the wavefront keeps in registers (36 per activation row and 2048 values of K).  Every further
// activation row costs about 2 us on the cfg-2 shape: from three rows on the decode kernel (matrix cores) is ahead.
template <typename T, int ITERS, int D, int MT, int LAYOUT = 0>
__global__ __launch_bounds__(1024) void gemv_w4a16_ring_kernel(const T* __restrict__ A, const uint8_t* __restrict__ Wp,
                                                                             const T* __restrict__ scales,
                                                                             const T* __restrict__ zeros, void* __restrict__ C,
                                                                             int N, int K, int group_shift, float zero_scalar,
                                                                             int out_dtype, int rows_per_block) {
  constexpr bool F16 = __is_same(T, half_t);
  static_assert(MT == 1 || (F16 && MT == 2), "two activation rows: fp16 only");
  typedef __attribute__((address_space(3))) uint8_t* lptr_t;
  extern __shared__ __align__(16) uint8_t smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nwaves = blockDim.x >> 6;
  const int chunks = K >> 5, row_bytes = K >> 1, groups = K >> group_shift;
  const int r0 = blockIdx.x * rows_per_block;
  const int r1 = r0 + rows_per_block < N ? r0 + rows_per_block : N;
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lptr_t)smem);
  const addr::RingLayout L = addr::ring_layout(nwaves, D, ITERS, K, rows_per_block, groups, MT);
  const bool has_s = scales != nullptr, has_z = zeros != nullptr;
  auto dma16 = [&](uint32_t lds_addr, uint32_t voff, const uint8_t* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
  };
  // the packed weights are read once: non-temporal, so that they do not displace what the caches hold for later
  // (single launch of 22.5 MB: 6.46 instead of 7.18 us)
  auto dma16_once = [&](uint32_t lds_addr, uint32_t voff, const uint8_t* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
  };
  auto wait_vm = [&](int outstanding) {  // a wavefront-uniform count, 0 .. ITERS * D
    static_assert(ITERS * D <= 6, "cases below");
    switch (outstanding) {
      case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
      case 5: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
      case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
      case 3: asm volatile("s_waitcnt vmcnt(3)" ::: "memory"); break;
      case 2: asm volatile("s_waitcnt vmcnt(2)" ::: "memory"); break;
      case 1: asm volatile("s_waitcnt vmcnt(1)" ::: "memory"); break;
      default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
  };

  // ---- staging data first (loads retire in issue order: once only a wavefront's weight rows are outstanding its
  // staging loads have landed), then the first D rows ----
  const int a_pieces = chunks * 4 * MT;  // the activation rows are contiguous
  for (int p0 = wave * 64; p0 < a_pieces; p0 += nwaves * 64)
    dma16(lds0 + L.act + (uint32_t)p0 * 16u, addr::ring_act_voff(p0, lane, a_pieces), (const uint8_t*)A);
  const int sz_pieces = ((r1 - r0) * groups) >> 3;  // groups is a multiple of 8
  const uint8_t* const s_base = uniform_ptr((const uint8_t*)(scales + (int64_t)r0 * groups));
  const uint8_t* const z_base = uniform_ptr((const uint8_t*)(zeros + (int64_t)r0 * groups));
  for (int p0 = wave * 64; p0 < sz_pieces; p0 += nwaves * 64) {
    const uint32_t voff = addr::ring_stage_voff(p0, lane, sz_pieces);
    if (has_s) dma16(lds0 + L.s + (uint32_t)p0 * 16u, voff, s_base);
    if (has_z) dma16(lds0 + L.z + (uint32_t)p0 * 16u, voff, z_base);
  }
  uint32_t voff_w[ITERS];
  int cc[ITERS], gsel[ITERS];
  bool ok[ITERS];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int c = (it << 6) + lane;
    ok[it] = c < chunks;
    cc[it] = ok[it] ? c : chunks - 1;
    gsel[it] = (cc[it] << 5) >> group_shift;
    voff_w[it] = addr::ring_w_voff(lane, it, chunks);
  }
  const int my_rows = addr::ring_my_rows(r1 - r0, wave, nwaves);
  auto issue = [&](int i, int slot) {  // the wavefront's i-th row into ring slot `slot`
    const uint8_t* const base = uniform_ptr(Wp + (int64_t)(r0 + wave + i * nwaves) * row_bytes);
#pragma unroll
    for (int it = 0; it < ITERS; ++it) dma16_once(lds0 + L.ring + addr::ring_w_lds(wave, slot, it, D, ITERS), voff_w[it], base);
  };
#pragma unroll
  for (int d = 0; d < D; ++d)
    if (d < my_rows) issue(d, d);
  wait_vm(ITERS * (my_rows < D ? my_rows : D));
  __syncthreads();

  // every wavefront prepares the activations of its lanes' chunks itself (fp16: pairs in unpack order and the chunk
  // sums; bf16: the 32 values as they are)
  ActF16 act[MT][F16 ? ITERS : 1];
  uint4_t actn[F16 ? 1 : ITERS][4];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      uint4_t raw[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) raw[j] = *(const uint4_t*)(smem + L.act + addr::ring_act_lds(m * chunks + cc[it], j));
      if constexpr (F16) {
        permute_act<LAYOUT>(act[m][it], raw);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) actn[it][j] = raw[j];
      }
    }
  const T* const lds_s = (const T*)(smem + L.s);
  const T* const lds_z = (const T*)(smem + L.z);
  const NibbleMagic mg = make_nibble_magic();
  const T one = from_float<T>(1.0f), zs = from_float<T>(zero_scalar);
  int slot = 0;
  for (int i = 0; i < my_rows; ++i) {
    wait_vm(ITERS * addr::ring_younger_rows(i, my_rows, D));
    const int lrow = wave + i * nwaves;
    uint4_t w[ITERS];
#pragma unroll
    for (int it = 0; it < ITERS; ++it)
      w[it] = *(const uint4_t*)(smem + L.ring + addr::ring_w_lds(wave, slot, it, D, ITERS) + (uint32_t)lane * 16u);
    T sv[ITERS], zv[ITERS];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const T s0 = has_s ? lds_s[lrow * groups + gsel[it]] : one;
      sv[it] = ok[it] ? s0 : from_float<T>(0.0f);  // a chunk past the end contributes 0
      zv[it] = has_z ? lds_z[lrow * groups + gsel[it]] : zs;
    }
    if (i + D < my_rows) {  // the slot takes the row D ahead once this row's words are in registers
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      issue(i + D, slot);
    }
    float acc = 0.f;
    if constexpr (F16 && MT > 1) {
      float accm[MT];
#pragma unroll
      for (int m = 0; m < MT; ++m) accm[m] = 0.f;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        half2_t e[16];  // the chunk's 32 nibbles with the unpack bias left in, once for all activation rows
        const uint32_t x[4] = {w[it].x, w[it].y, w[it].z, w[it].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t v = x[j], v8 = v >> 8;
          e[4 * j + 0] = bitcast<half2_t>(bfi(mg.m_lo, v, mg.b_lo));
          e[4 * j + 1] = bitcast<half2_t>(bfi(mg.m_hi, v, mg.b_hi));
          e[4 * j + 2] = bitcast<half2_t>(bfi(mg.m_lo, v8, mg.b_lo));
          e[4 * j + 3] = bitcast<half2_t>(bfi(mg.m_hi, v8, mg.b_hi));
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          float d = 0.f;
#pragma unroll
          for (int p = 0; p < 16; ++p) d = __builtin_amdgcn_fdot2(e[p], act[m][it].a[p], d, false);
          accm[m] += (float)sv[it] * (d - __builtin_fmaf((float)zv[it], act[m][it].sum, act[m][it].bsum));
        }
      }
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const float v = wave_sum_to_lane63(accm[m]);
        if (lane == 63) store_out(C, (int64_t)m * N + r0 + lrow, v, out_dtype);
      }
      slot = slot + 1 == D ? 0 : slot + 1;
      continue;
    } else if constexpr (F16) {
#pragma unroll
      for (int it = 0; it < ITERS; ++it) acc += chunk_term_biased(w[it], act[0][it], sv[it], zv[it], mg);
    } else {
      bool integral = true;  // small integer zero points fold exactly into one fused multiply-add per weight
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const float zf = to_float(zv[it]);
        integral = integral && zf == __builtin_rintf(zf) && zf >= -256.0f && zf <= 256.0f;
      }
      if (__builtin_amdgcn_ballot_w64(integral) == ~0ull) {
#pragma unroll
        for (int it = 0; it < ITERS; ++it) acc += chunk_term_dot2<true, LAYOUT>(w[it], actn[it], sv[it], zv[it], mg);
      } else {
#pragma unroll
        for (int it = 0; it < ITERS; ++it) acc += chunk_term_dot2<false, LAYOUT>(w[it], actn[it], sv[it], zv[it], mg);
      }
    }
    const float v = wave_sum_to_lane63(acc);
    if (lane == 63) store_out(C, r0 + lrow, v, out_dtype);
    slot = slot + 1 == D ? 0 : slot + 1;
  }
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
        w[r] = __builtin_nontemporal_load((const uint4_t*)(Wp + rows[r] * row_bytes + ((int64_t)c << 4)));  // read once
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

// A few weight rows (the last N % 16 of a matrix whose row count is no multiple of 16) against ALL activation rows, written
// into an output whose rows lie `ldc` elements apart, from column `col0` on: one wavefront per activation row, the generic
// kernel's arithmetic (every weight dequantised as the reference rounds it, fp32 sums).
// A 32-bit word of interleave_weight's float16 layout (field j holds element (0, 2, 4, 6, 1, 3, 5, 7)[j]) back in plain order.
__device__ __forceinline__ uint32_t plain_word_of_interleaved(uint32_t v) {
  const uint32_t lo = v & 0xffffu, hi = v >> 16;  // even elements | odd elements
  const uint32_t even = ((lo & 0xf000u) << 12) | ((lo & 0x0f00u) << 8) | ((lo & 0x00f0u) << 4) | (lo & 0x000fu);
  const uint32_t odd = ((hi & 0xf000u) << 12) | ((hi & 0x0f00u) << 8) | ((hi & 0x00f0u) << 4) | (hi & 0x000fu);
  return even | (odd << 4);
}
template <typename T, int LAYOUT>
__global__ __launch_bounds__(256) void w4a16_tail_rows_kernel(const T* __restrict__ A, const uint8_t* __restrict__ Wp,
                                                              const T* __restrict__ scales, const T* __restrict__ zeros,
                                                              void* __restrict__ C, int M, int rows, int K, int group,
                                                              float zero_scalar, int out_dtype, int64_t ldc, int64_t col0) {
  typedef typename ActOf<T>::type Act;
  const int lane = threadIdx.x & 63;
  const int64_t m = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (m >= M) return;  // whole wavefront leaves together
  const int chunks = K >> 5;
  const int groups = K / group;
  const int64_t row_bytes = K >> 1;
  const T one = from_float<T>(1.0f);
  const T zs = from_float<T>(zero_scalar);
  for (int r = 0; r < rows; ++r) {
    float acc = 0.f;
    for (int c = lane; c < chunks; c += 64) {
      uint4_t w = *(const uint4_t*)(Wp + r * row_bytes + ((int64_t)c << 4));
      if constexpr (LAYOUT == 1) w = uint4_t{plain_word_of_interleaved(w.x), plain_word_of_interleaved(w.y), plain_word_of_interleaved(w.z), plain_word_of_interleaved(w.w)};
      const int g = (c << 5) / group;
      const T s = scales ? scales[(int64_t)r * groups + g] : one;
      const T z = zeros ? zeros[(int64_t)r * groups + g] : zs;
      Act act;
      load_act(act, A, m * K + ((int64_t)c << 5));
      acc += chunk_term(w, act, s, z);
    }
    const float v = wave_sum(acc);
    if (lane == 0) store_out(C, m * ldc + col0 + r, v, out_dtype);
  }
}

// Wp, scales and zeros point at the first of the `rows` weight rows.
int w4a16_tail_rows(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t rows, int64_t K,
                    int64_t group, float zero_scalar, int in_dtype, int out_dtype, int w_layout, int64_t ldc, int64_t col0, hipStream_t st) {
  if (M < 1 || rows < 1 || rows > 64 || K < 32 || K % 32 != 0 || group < 1 || K % group != 0 || group % 32 != 0 || M > 0x7fffffff || K > 0x7fffffff) {
    set_error("tlq_gemm_w4a16 (last weight rows): bad shape M=%lld rows=%lld K=%lld group=%lld", (long long)M, (long long)rows, (long long)K, (long long)group);
    return 1;
  }
  const unsigned blocks = (unsigned)ceil_div(M, (int64_t)4);
#define TLQ_TAIL_CASE(TT, LL)                                                                                                        \
  w4a16_tail_rows_kernel<TT, LL><<<blocks, 256, 0, st>>>((const TT*)A, (const uint8_t*)Wp, (const TT*)scales, (const TT*)zeros, C, (int)M, \
                                                         (int)rows, (int)K, (int)group, zero_scalar, out_dtype, ldc, col0)
  if (in_dtype == TLQ_F16) {
    if (w_layout == TLQ_W_PLAIN) TLQ_TAIL_CASE(half_t, 0);
    else TLQ_TAIL_CASE(half_t, 1);
  } else {
    if (w_layout == TLQ_W_PLAIN) TLQ_TAIL_CASE(bf16_t, 0);
    else TLQ_TAIL_CASE(bf16_t, 1);
  }
#undef TLQ_TAIL_CASE
  return check_launch("tlq_gemm_w4a16 (last weight rows)", "w4a16_tail_rows_kernel") ? 0 : 1;
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

// rows-per-wave / waves-per-block / blocks-per-CU overrides for tuning runs (0 = automatic)
static thread_local int g_gemv_rows = 0, g_gemv_waves = 0, g_gemv_waves16 = 0, g_gemv_unroll = 0, g_gemv_depth = 0;

static int cu_count() {
  static int n = 0;
  if (n == 0) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
  }
  return n;
}

template <int R, int MT, int D>
static int launch_gemv_f16(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int batch,
                           int M, int N, int K, int group_shift, float zero_scalar, int out_dtype, int waves_per_block,
                           int blocks_per_cu, hipStream_t st) {
  const size_t lds = (size_t)MT * (K / 32) * 72;
  if (lds > 64 * 1024) {
    set_error("tlq_gemm_w4a16(gemv): K=%d needs %zu bytes of LDS for the activations (limit 65536)", K, lds);
    return 1;
  }
  const int row_groups = (int)ceil_div(N, R);
  int blocks = (int)ceil_div(row_groups, waves_per_block);
  const int cap = (int)ceil_div((int64_t)cu_count() * blocks_per_cu, batch);
  if (blocks > cap) blocks = cap < 1 ? 1 : cap;
  gemv_w4a16_f16_kernel<R, MT, D><<<dim3(blocks, batch), 64 * waves_per_block, lds, st>>>(
      (const half_t*)A, (const uint8_t*)Wp, (const half_t*)scales, (const half_t*)zeros, C, M, N, K, group_shift,
      zero_scalar, out_dtype);
  return 0;
}

// Launch geometry of the rows kernel: work-groups of `waves_per_block` wavefronts, each owning `rows_per_block`
// consecutive rows whose scales and zero points it keeps in LDS next to the prepared activations; at least
// `blocks_per_cu` work-groups per CU when there are rows enough.  Everything a work-group keeps in LDS must fit the
// 64 KB a kernel gets without asking for more: 72 bytes per 32 activations, 4 bytes per row and group.
struct RowsPlan {
  int rows_per_block, blocks;
  size_t lds_bytes;
  bool fits;
};
static RowsPlan plan_gemv_rows(int batch, int N, int K, int group_shift, int waves_per_block, int blocks_per_cu, int cus) {
  RowsPlan p{0, 0, 0, false};
  const int groups = K >> group_shift;
  const size_t act_bytes = (size_t)(K / 32) * 72;
  if (groups < 1 || act_bytes >= 64 * 1024) return p;
  int blocks = (int)ceil_div((int64_t)cus * blocks_per_cu, batch);
  if (blocks < 1) blocks = 1;
  int rpb = (int)ceil_div(N, blocks);
  if (rpb < waves_per_block) rpb = waves_per_block;
  int rpb_max = (int)((64 * 1024 - act_bytes) / ((size_t)4 * groups));
  if (rpb_max > (48 * 1024) / (4 * groups)) rpb_max = (48 * 1024) / (4 * groups);  // at most 48 KB of scales and zero points
  rpb_max &= ~3;
  if (rpb_max < waves_per_block) return p;
  // more rows per work-group than LDS holds: an equal number of smaller work-groups for every CU instead of full ones and a
  // short last round (N = 28672, K = 8192, groups of 64: 312 work-groups of 92 rows on 256 CUs took 31.7 us, the same
  // matrix with groups of 128 -- 256 work-groups of 112 rows -- 23.3 us)
  // (one problem per launch only: with many, the work-groups of all problems share the rounds, and full ones were faster --
  // 24 problems of N = 11008, K = 4096: 94 us with 29 work-groups of 384 rows each, 104 us with 33 of 336)
  if (rpb > rpb_max && batch == 1) rpb = (int)ceil_div(N, (int64_t)blocks * ceil_div(rpb, rpb_max));
  if (rpb < waves_per_block) rpb = waves_per_block;
  rpb = (rpb + 3) & ~3;  // keeps the zero-point block of LDS 16-byte aligned for any group count
  if (rpb > rpb_max) rpb = rpb_max;
  p.rows_per_block = rpb;
  p.blocks = (int)ceil_div(N, rpb);
  p.lds_bytes = act_bytes + (size_t)rpb * groups * 4;
  p.fits = p.lds_bytes <= 64 * 1024;
  return p;
}

template <typename T, int ITERS, int D, int MAXT>
static int launch_gemv_rows(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int batch,
                            int N, int K, int group_shift, float zero_scalar, int out_dtype, int waves_per_block,
                            int blocks_per_cu, hipStream_t st) {
  const RowsPlan plan = plan_gemv_rows(batch, N, K, group_shift, waves_per_block, blocks_per_cu, cu_count());
  if (!plan.fits) {
    set_error("tlq_gemm_w4a16(gemv): K=%d with groups of %d does not fit the rows kernel's 64 KB of LDS", K, 1 << group_shift);
    return 1;
  }
  const int rpb = plan.rows_per_block, blocks = plan.blocks;
  const size_t lds = plan.lds_bytes;
  if constexpr (__is_same(T, half_t))
    gemv_w4a16_f16_rows_kernel<ITERS, D, MAXT><<<dim3(blocks, batch), 64 * waves_per_block, lds, st>>>(
        (const half_t*)A, (const uint8_t*)Wp, (const half_t*)scales, (const half_t*)zeros, C, N, K, group_shift,
        zero_scalar, out_dtype, rpb, waves_per_block);
  else
    gemv_w4a16_bf16_rows_kernel<ITERS, D, MAXT><<<dim3(blocks, batch), 64 * waves_per_block, lds, st>>>(
        (const bf16_t*)A, (const uint8_t*)Wp, (const bf16_t*)scales, (const bf16_t*)zeros, C, N, K, group_shift,
        zero_scalar, out_dtype, rpb, waves_per_block);
  return 0;
}

// Launch geometry of the ring kernel: one work-group of 16 wavefronts per CU, every wavefront's rows in flight from the
// start where the LDS has room for them (three slots of a row per wavefront at most).  One problem per launch, rows of
// up to 4096 values, group counts that are multiples of 8 (the staging loads move 16 bytes).
struct RingPlan {
  bool ok;
  int iters, depth, waves, rows_per_block, blocks;
  uint32_t lds_bytes;
};
static RingPlan plan_gemv_ring(int64_t batch, int64_t M, int64_t N, int64_t K, int group_shift, int cus) {
  RingPlan p{false, 0, 0, 0, 0, 0, 0};
  if (batch != 1 || M < 1 || M > 2 || N < 1 || N > 0x7fffffff || K < 32 || K % 32 != 0 || K > 4096 || group_shift < 5 || cus < 1) return p;
  const int groups = (int)(K >> group_shift);
  if (groups < 8 || groups % 8 != 0 || ((int64_t)groups << group_shift) != K) return p;
  p.waves = (g_gemv_waves16 >= 1 && g_gemv_waves16 <= 16) ? g_gemv_waves16 : 16;
  p.iters = K > 2048 ? 2 : 1;
  // work-groups per CU (tlq_tune_gemv_unroll): two of 16 wavefronts fit a CU's registers and LDS, and are slower, as every
  // other way of putting more requests in flight was: N = 11008, K = 4096: 6.8 us with one, 7.5 with two, 8.8 with three
  const int per_cu = (g_gemv_unroll >= 1 && g_gemv_unroll <= 4) ? g_gemv_unroll : 1;
  int64_t rpb = ceil_div(N, (int64_t)cus * per_cu);
  if (rpb < p.waves) rpb = p.waves;
  if (rpb * groups * 2 > 24 * 1024) return p;  // scales and zero points of the rows: at most 24 KB each
  p.rows_per_block = (int)rpb;
  p.blocks = (int)ceil_div(N, rpb);
  // one row in flight per wavefront: 16 wavefronts on 256 CUs ask for 8 MB at a time, about what the memory system
  // holds in flight at its full rate; with two or three rows per wavefront the same launch measured 3 - 17 % slower
  const int per_wave = (int)ceil_div(rpb, (int64_t)p.waves);
  // (from about 64 MB of weights on the launch is long enough for two rows in flight to be level or 2 - 4 % ahead)
  const int want = (g_gemv_depth >= 1 && g_gemv_depth <= 3) ? g_gemv_depth : (N * (K / 2) > ((int64_t)64 << 20) ? 2 : 1);
  p.depth = per_wave < want ? per_wave : want;
  if (M > 1 && p.depth > 2) p.depth = 2;
  p.lds_bytes = addr::ring_layout(p.waves, p.depth, p.iters, (int)K, p.rows_per_block, groups, (int)M).total;
  p.ok = p.lds_bytes <= 160 * 1024;
  return p;
}

template <typename T, int ITERS, int D, int MT, int LAYOUT>
static int launch_gemv_ring(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int N, int K,
                            int group_shift, float zero_scalar, int out_dtype, const RingPlan& p, hipStream_t st) {
  auto kern = gemv_w4a16_ring_kernel<T, ITERS, D, MT, LAYOUT>;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) {
      set_error("tlq_gemm_w4a16(gemv): cannot reserve the ring kernel's LDS: %s", hipGetErrorString(e));
      return 1;
    }
    attr_set = true;
  }
  kern<<<p.blocks, 64 * p.waves, p.lds_bytes, st>>>((const T*)A, (const uint8_t*)Wp, (const T*)scales, (const T*)zeros, C, N, K,
                                                  group_shift, zero_scalar, out_dtype, p.rows_per_block);
  return check_launch("tlq_gemm_w4a16(gemv)", LAYOUT == 1 ? "gemv_w4a16_ring_kernel, interleaved words" : "gemv_w4a16_ring_kernel") ? 0 : 1;
}

// 1 (default): the ring kernel where it applies; 0: never
static thread_local int g_gemv_ring = 1;

template <typename T, int MT, int LAYOUT = 0>
static int dispatch_gemv_ring(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int N, int K,
                              int group_shift, float zero_scalar, int out_dtype, const RingPlan& p, hipStream_t st) {
#define TLQ_RING_CASE(IT, DD) \
  return launch_gemv_ring<T, IT, DD, MT, LAYOUT>(A, Wp, scales, zeros, C, N, K, group_shift, zero_scalar, out_dtype, p, st)
  if (p.iters == 1) {
    if (p.depth == 1) TLQ_RING_CASE(1, 1);
    if (p.depth == 2 || MT > 1) TLQ_RING_CASE(1, 2);
    if constexpr (MT == 1) TLQ_RING_CASE(1, 3);
  }
  if (p.depth == 1) TLQ_RING_CASE(2, 1);
  if (p.depth == 2 || MT > 1) TLQ_RING_CASE(2, 2);
  if constexpr (MT == 1) TLQ_RING_CASE(2, 3);
#undef TLQ_RING_CASE
  return 1;
}

// whether the ring kernel takes this problem (the automatic kernel choice of tlq_gemm_w4a16 asks)
bool gemv_ring_applies(int64_t M, int64_t N, int64_t K, int64_t group, int in_dtype, const void* scales, const void* zeros) {
  if (!g_gemv_ring || g_gemv_rows < 0 || group < 32 || (group & (group - 1)) != 0) return false;
  if ((((uintptr_t)scales | (uintptr_t)zeros) & 15) != 0) return false;
  if (in_dtype != TLQ_F16 && !(in_dtype == TLQ_BF16 && M == 1)) return false;
  int shift = 0;
  while (((int64_t)1 << shift) < group) ++shift;
  return plan_gemv_ring(1, M, N, K, shift, cu_count()).ok;
}

// The ring kernel on weights whose 32-bit words went through interleave_weight (fp16 target).  -1: the kernel does not take
// the problem (nothing launched).  The sums pair other elements than with plain words (the nibble masks pick neighbours in
// k), so results agree with the plain layout to the last bits of the fp32 sums, not bit for bit.
int gemv_w4a16_ring_interleaved(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t N,
                                int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, hipStream_t st) {
  if (!gemv_ring_applies(M, N, K, group, in_dtype, scales, zeros)) return -1;
  int shift = 0;
  while (((int64_t)1 << shift) < group) ++shift;
  const RingPlan rp = plan_gemv_ring(1, M, N, K, shift, cu_count());
  if (!rp.ok) return -1;
  if (in_dtype == TLQ_F16) {
    if (M == 1) return dispatch_gemv_ring<half_t, 1, 1>(A, Wp, scales, zeros, C, (int)N, (int)K, shift, zero_scalar, out_dtype, rp, st);
    return dispatch_gemv_ring<half_t, 2, 1>(A, Wp, scales, zeros, C, (int)N, (int)K, shift, zero_scalar, out_dtype, rp, st);
  }
  return dispatch_gemv_ring<bf16_t, 1, 1>(A, Wp, scales, zeros, C, (int)N, (int)K, shift, zero_scalar, out_dtype, rp, st);
}

// wavefronts per work-group and work-groups per CU of the rows kernel for this K
static void rows_kernel_shape(int64_t K, int& wpb_rows, int& bpc_rows) {
  bpc_rows = g_gemv_unroll ? g_gemv_unroll : 1;
  const bool long_rows = K > 4096;  // 8 wavefronts per work-group (see the kernel)
  wpb_rows = g_gemv_waves16 ? g_gemv_waves16 : 16;
  if (long_rows && wpb_rows > 8) wpb_rows = 8;
  if (wpb_rows * 64 < K / 32) wpb_rows = (int)ceil_div(K / 32, (int64_t)64);  // one staging thread per chunk
}
static bool rows_kernel_fits(int64_t batch, int64_t N, int64_t K, int shift) {
  int wpb_rows, bpc_rows;
  rows_kernel_shape(K, wpb_rows, bpc_rows);
  return plan_gemv_rows((int)batch, (int)N, (int)K, shift, wpb_rows, bpc_rows, cu_count()).fits;
}

// M = 1, rows of up to 16384 values: the register-resident kernel (see gemv_rows_body)
template <typename T>
static int dispatch_gemv_rows(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t batch,
                              int64_t N, int64_t K, int shift, float zero_scalar, int out_dtype, hipStream_t st) {
  const int depth_req = g_gemv_depth;
  int wpb_rows, bpc_rows;
  rows_kernel_shape(K, wpb_rows, bpc_rows);
  // one problem of a few tens of MB: one row in flight per wavefront (deeper queues delay the staging
  // loads behind the weights and measured slower); many problems per launch stream with two
  const int d = depth_req ? depth_req : (batch * N * (K / 2) > ((int64_t)64 << 20) ? 2 : 1);
#define TLQ_ROWS_CASE(IT, DD, MAXT)                                                                                \
  launch_gemv_rows<T, IT, DD, MAXT>(A, Wp, scales, zeros, C, (int)batch, (int)N, (int)K, shift, zero_scalar, out_dtype, \
                             wpb_rows, bpc_rows, st)
  if (K <= 2048) {
    if (d <= 2) TLQ_ROWS_CASE(1, 2, 1024);
    else if (d <= 4) TLQ_ROWS_CASE(1, 4, 1024);
    else TLQ_ROWS_CASE(1, 8, 1024);
  } else if (K <= 4096) {
    if (d <= 1) TLQ_ROWS_CASE(2, 1, 1024);
    else if (d == 2) TLQ_ROWS_CASE(2, 2, 1024);
    else if (d == 3) TLQ_ROWS_CASE(2, 3, 1024);
    else if (d == 4) TLQ_ROWS_CASE(2, 4, 1024);
    else TLQ_ROWS_CASE(2, 6, 1024);
  } else {
    const int iters = (int)ceil_div(K, (int64_t)2048);  // 3 .. 8
#define TLQ_LONG_CASE(IT)                    \
  case IT:                                   \
    if (d <= 1) TLQ_ROWS_CASE(IT, 1, 512);   \
    else TLQ_ROWS_CASE(IT, 2, 512);          \
    break;
    switch (iters) {
      TLQ_LONG_CASE(3)
      TLQ_LONG_CASE(4)
      TLQ_LONG_CASE(5)
      TLQ_LONG_CASE(6)
      TLQ_LONG_CASE(7)
      default:
        TLQ_LONG_CASE(8)
    }
#undef TLQ_LONG_CASE
  }
#undef TLQ_ROWS_CASE
  return check_launch("tlq_gemm_w4a16(gemv)", std::is_same<T, half_t>::value ? "gemv_w4a16_f16_rows_kernel" : "gemv_w4a16_bf16_rows_kernel") ? 0 : 1;
}

int gemv_w4a16(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t batch, int64_t M,
               int64_t N, int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, hipStream_t st) {
  const int wpb = g_gemv_waves ? g_gemv_waves : 4;
  int rc = 0;
  const bool pow2 = (group & (group - 1)) == 0;
  if (in_dtype == TLQ_F16 && pow2) {
    int shift = 0;
    while (((int64_t)1 << shift) < group) ++shift;
    // One problem of a few tens of MB is latency bound: one row per wavefront and a grid of 8
    // blocks per CU (each wavefront then walks ~3 rows with the next row's loads in flight).
    // Large / batched problems stream: two rows per wavefront, one block per 8 rows.
    const bool streaming = batch * N * (K / 2) > ((int64_t)64 << 20);
    const int R = g_gemv_rows > 0 ? g_gemv_rows : (streaming ? 2 : 1);
    const int bpc = g_gemv_unroll ? g_gemv_unroll : (streaming ? 64 : 8);  // grid size cap, blocks per CU
    const int depth_req = g_gemv_depth;
    if (M <= 2 && g_gemv_ring && g_gemv_rows >= 0 && (((uintptr_t)scales | (uintptr_t)zeros) & 15) == 0) {
      const RingPlan rp = plan_gemv_ring(batch, M, N, K, shift, cu_count());
#define TLQ_RING_M(MM) \
  case MM:             \
    return dispatch_gemv_ring<half_t, MM>(A, Wp, scales, zeros, C, (int)N, (int)K, shift, zero_scalar, out_dtype, rp, st)
      if (rp.ok) switch ((int)M) {
          TLQ_RING_M(1);
          TLQ_RING_M(2);
        }
#undef TLQ_RING_M
    }
    if (M == 1 && K <= 16384 && g_gemv_rows >= 0 && rows_kernel_fits(batch, N, K, shift))
      return dispatch_gemv_rows<half_t>(A, Wp, scales, zeros, C, batch, N, K, shift, zero_scalar, out_dtype, st);
    const bool two_rows = M > 1 && (size_t)2 * (K / 32) * 72 <= 64 * 1024;
#define TLQ_F16_CASE(RR, MTT, DD)                                                                                  \
  rc = launch_gemv_f16<RR, MTT, DD>(A, Wp, scales, zeros, C, (int)batch, (int)M, (int)N, (int)K, shift, zero_scalar, \
                                    out_dtype, wpb, bpc, st)
    // steps in flight per wavefront (each R KB)
    const int depth = g_gemv_depth ? g_gemv_depth : (streaming ? 2 : 6);
    if (two_rows) {
      if (depth <= 1) TLQ_F16_CASE(2, 2, 1);
      else if (depth == 2) TLQ_F16_CASE(2, 2, 2);
      else TLQ_F16_CASE(2, 2, 3);
    } else if (R == 1) {
      if (depth <= 1) TLQ_F16_CASE(1, 1, 1);
      else if (depth == 2) TLQ_F16_CASE(1, 1, 2);
      else if (depth <= 4) TLQ_F16_CASE(1, 1, 4);
      else if (depth <= 6) TLQ_F16_CASE(1, 1, 6);
      else TLQ_F16_CASE(1, 1, 8);
    } else if (R == 4) {
      if (depth <= 1) TLQ_F16_CASE(4, 1, 1);
      else TLQ_F16_CASE(4, 1, 2);
    } else {
      if (depth <= 1) TLQ_F16_CASE(2, 1, 1);
      else if (depth == 2) TLQ_F16_CASE(2, 1, 2);
      else TLQ_F16_CASE(2, 1, 4);
    }
#undef TLQ_F16_CASE
    if (rc) return rc;
  } else if (in_dtype == TLQ_F16) {
    // group size that is not a power of two: generic kernel
    launch_gemv<half_t, 2, 1>(A, Wp, scales, zeros, C, (int)batch, (int)M, (int)N, (int)K, (int)group, zero_scalar,
                              out_dtype, wpb, st);
  } else {
    int shift = 0;
    while (((int64_t)1 << shift) < group) ++shift;
    if (M == 1 && pow2 && g_gemv_ring && g_gemv_rows >= 0 && (((uintptr_t)scales | (uintptr_t)zeros) & 15) == 0) {
      const RingPlan rp = plan_gemv_ring(batch, 1, N, K, shift, cu_count());
      if (rp.ok) return dispatch_gemv_ring<bf16_t, 1>(A, Wp, scales, zeros, C, (int)N, (int)K, shift, zero_scalar, out_dtype, rp, st);
    }
    if (M == 1 && pow2 && K <= 16384 && g_gemv_rows >= 0 && rows_kernel_fits(batch, N, K, shift)) {
      return dispatch_gemv_rows<bf16_t>(A, Wp, scales, zeros, C, batch, N, K, shift, zero_scalar, out_dtype, st);
    }
    // bfloat16 otherwise: element-wise exact dequantisation (generic kernel)
    if (M == 1)
      launch_gemv<bf16_t, 2, 1>(A, Wp, scales, zeros, C, (int)batch, (int)M, (int)N, (int)K, (int)group, zero_scalar,
                                out_dtype, wpb, st);
    else
      launch_gemv<bf16_t, 1, 2>(A, Wp, scales, zeros, C, (int)batch, (int)M, (int)N, (int)K, (int)group, zero_scalar,
                                out_dtype, wpb, st);
  }
  return check_launch("tlq_gemm_w4a16(gemv)") ? 0 : 1;
}

}  // namespace tlq

extern "C" {
int tlq_debug_gemv_rows_plan(int64_t batch, int64_t N, int64_t K, int64_t group, int cus, void* plan_out) {
  int shift = 0;
  while (((int64_t)1 << shift) < group) ++shift;
  if (batch < 1 || N < 1 || K < 64 || K > 16384 || K % 64 || ((int64_t)1 << shift) != group || K % group || cus < 1) {
    tlq::set_error("tlq_debug_gemv_rows_plan: bad arguments");
    return -1;
  }
  int wpb, bpc;
  tlq::rows_kernel_shape(K, wpb, bpc);
  const tlq::RowsPlan p = tlq::plan_gemv_rows((int)batch, (int)N, (int)K, shift, wpb, bpc, cus);
  if (plan_out) {
    int64_t* out = (int64_t*)plan_out;
    out[0] = p.rows_per_block, out[1] = p.blocks, out[2] = (int64_t)p.lds_bytes, out[3] = wpb;
  }
  return p.fits ? 1 : 0;
}

// Tuning hook used by the benchmark sweeps: rows per wavefront (1, 2, 4) and wavefronts per
// block (1..4) of the GEMV kernel; 0 restores the automatic choice.
void tlq_tune_gemv(int rows_per_wave, int waves_per_block) {
  tlq::g_gemv_rows = rows_per_wave;  // negative: never use the register-resident rows kernel
  tlq::g_gemv_waves = (waves_per_block < 0 || waves_per_block > 4) ? 0 : waves_per_block;
  tlq::g_gemv_waves16 = (waves_per_block < 0 || waves_per_block > 16) ? 0 : waves_per_block;  // register-resident kernel
}
void tlq_tune_gemv_ring(int on) { tlq::g_gemv_ring = on != 0; }

int tlq_debug_gemv_ring_plan(int64_t M, int64_t N, int64_t K, int64_t group, int cus, void* plan_out) {
  int shift = 0;
  while (((int64_t)1 << shift) < group) ++shift;
  if (group < 1 || ((int64_t)1 << shift) != group) {
    tlq::set_error("tlq_debug_gemv_ring_plan: the group size must be a power of two");
    return -1;
  }
  const tlq::RingPlan p = tlq::plan_gemv_ring(1, M, N, K, shift, cus);
  if (plan_out) {
    int64_t* o = (int64_t*)plan_out;
    o[0] = p.iters, o[1] = p.depth, o[2] = p.waves, o[3] = p.rows_per_block, o[4] = p.blocks, o[5] = p.lds_bytes;
  }
  return p.ok ? 1 : 0;
}

void tlq_tune_gemv_unroll(int blocks_per_cu) { tlq::g_gemv_unroll = blocks_per_cu; }
void tlq_tune_gemv_depth(int steps_in_flight) { tlq::g_gemv_depth = steps_in_flight < 0 ? 0 : steps_in_flight; }
}
