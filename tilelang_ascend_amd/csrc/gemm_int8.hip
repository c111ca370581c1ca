// int8 MFMA GEMMs (v_mfma_i32_16x16x64_i8, int32 accumulate, bit exact):
//   * W8A8 with the fused rescale epilogue  C = rn_out(f32(acc) * scale_a[m] * scale_b[n])
//   * raw int32 output
//   * W4A8: packed int4 weights expanded to int8 on the way into LDS
// The second operand may be stored [K, N] (transposed on the fly) or [N, K].
#include "gemm_core.h"
#include "gemm_slots.h"

namespace tlq {

// Packed int4 [N, K/2] -> int8 LDS tile.  One stage is 128 values of K = 64 packed bytes per
// row; a thread expands 16 packed bytes into two 16-byte chunks.
template <int ROWS, int NT>
struct W4I8Loader {
  typedef RowFrag Frag;
  static constexpr bool DIRECT = false;
  static constexpr bool PREFETCH2 = false;
  static constexpr int SLOTS = ROWS * 4;
  static constexpr int PASSES = (SLOTS + NT - 1) / NT;
  static constexpr bool PARTIAL = SLOTS % NT != 0;
  static constexpr int UNITS = PASSES;
  static_assert(PASSES == 1 || (NT / 4) % 8 == 0, "pass stride must keep the swizzle phase");
  struct Params {
    const uint8_t* wp;
    int64_t row_bytes;  // K / 2
    int sign_mode;
    int64_t batch_stride;  // bytes between the "batches" (K slices: a slice's packed bytes per row)
  };
  struct Regs {
    uint4_t v[PASSES];
  };
  const uint8_t* base;    // uniform
  uint32_t voff[PASSES];  // per lane: row * row_bytes + quarter * 16
  uint32_t loff[2];       // per lane: LDS offsets of the two chunks this lane writes (pass 0)
  int kb_lane, row_bytes, sign_mode;
  bool active;

  __device__ __forceinline__ W4I8Loader(const Params& p, int batch, int row0, int rows_total, int tid)
      : base(p.wp + batch * p.batch_stride + (int64_t)row0 * p.row_bytes), row_bytes((int)p.row_bytes), sign_mode(p.sign_mode) {
    const int rows_valid = rows_total - row0;
    const int quarter = tid & 3;
    kb_lane = quarter * 16;
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      int row = (ps * NT + tid) >> 2;
      row = row < rows_valid ? row : rows_valid - 1;
      voff[ps] = (uint32_t)row * (uint32_t)p.row_bytes + (uint32_t)kb_lane;
    }
    loff[0] = (uint32_t)lds_off(tid >> 2, quarter * 2 + 0);
    loff[1] = (uint32_t)lds_off(tid >> 2, quarter * 2 + 1);
    active = !PARTIAL || ((PASSES - 1) * NT + tid) < SLOTS;
  }

  template <bool TAIL>
  __device__ __forceinline__ void gload(Regs& r, int kt, uint8_t* /*lds_next*/ = nullptr) const {
    const uint8_t* sb = base + (int64_t)kt * 64;
    if (!TAIL) {
#pragma unroll
      for (int ps = 0; ps < PASSES; ++ps) r.v[ps] = *(const uint4_t*)(sb + voff[ps]);
    } else {
      const bool ok = kt * 64 + kb_lane < row_bytes;
#pragma unroll
      for (int ps = 0; ps < PASSES; ++ps) {
        uint4_t v = *(const uint4_t*)(ok ? sb + voff[ps] : base + (voff[ps] - kb_lane));
        if (!ok) v = uint4_t{0u, 0u, 0u, 0u};
        r.v[ps] = v;
      }
    }
  }
  // four nibbles held one per byte (0..15) -> four int8 under the sign convention
  __device__ __forceinline__ uint32_t sign4(uint32_t x) const {
    if (sign_mode == TLQ_U4) return x;
    if (sign_mode == TLQ_S4_TWOS) x ^= 0x08080808u;  // two's complement == offset-8 of (u ^ 8)
    const uint32_t c = (sign_mode == TLQ_S4_OFFSET7) ? 0x07070707u : 0x08080808u;
    // per-byte u - c without borrows between bytes: bias by 128, subtract, remove the bias
    return ((x | 0x80808080u) - c) ^ 0x80808080u;
  }
  __device__ __forceinline__ void expand(uint32_t v, uint32_t& d0, uint32_t& d1) const {
    const uint32_t lo = sign4(v & 0x0f0f0f0fu);         // k0 k2 k4 k6
    const uint32_t hi = sign4((v >> 4) & 0x0f0f0f0fu);  // k1 k3 k5 k7
    d0 = __builtin_amdgcn_perm(hi, lo, 0x05010400u);    // k0 k1 k2 k3
    d1 = __builtin_amdgcn_perm(hi, lo, 0x07030602u);    // k4 k5 k6 k7
  }
  __device__ __forceinline__ void lstore_piece(const Regs& r, uint8_t* lds, int pc, int np) const {
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      if (ps * np / UNITS != pc) continue;
      if (PARTIAL && ps == PASSES - 1 && !active) continue;
      uint32_t d[8];
      expand(r.v[ps].x, d[0], d[1]);
      expand(r.v[ps].y, d[2], d[3]);
      expand(r.v[ps].z, d[4], d[5]);
      expand(r.v[ps].w, d[6], d[7]);
      uint8_t* dst = lds + ps * (NT / 4) * kStageBytes;
      *(uint4_t*)(dst + loff[0]) = uint4_t{d[0], d[1], d[2], d[3]};
      *(uint4_t*)(dst + loff[1]) = uint4_t{d[4], d[5], d[6], d[7]};
    }
  }
  __device__ __forceinline__ void lstore(const Regs& r, uint8_t* lds) const { lstore_piece(r, lds, 0, 1); }
};

// ---- launch helpers -----------------------------------------------------------------------
template <class WL, class Epi, int BM, int BN, int WM, int WN>
static int run_i8(const void* A, const typename WL::Params& pw, const typename Epi::Params& pe, int64_t batch,
                  int64_t M, int64_t N, int64_t K, hipStream_t st, const char* what) {
  constexpr int NT = WM * WN * 64;
  typedef RowLoaderDirect<BM, NT> AL;  // activations travel global -> LDS without passing through registers
  typename AL::Params pa{(const uint8_t*)A, K, M * K, K};
  return launch_gemm<MmaI8, AL, WL, Epi, BM, BN, WM, WN>(pa, pw, pe, batch, M, N, K, st, what, 2);
}

static thread_local int g_i8_tile = 0;

static int pick_tile(int64_t batch, int64_t M, int64_t N) {
  if (g_i8_tile) return g_i8_tile;
  if (M <= 32) return 32;
  return prefer_small_tiles(batch, M, N) ? 128 : 256;  // by machine fill (the rule holds for int8 as measured: twelve shapes, both weight layouts)
}

template <class Epi>
static int dispatch_i8(const void* A, const void* B, const typename Epi::Params& pe, int64_t batch, int64_t M,
                       int64_t N, int64_t K, int b_layout, hipStream_t st, const char* what) {
  const int tile = pick_tile(batch, M, N);
  // The five-slot kernel where it measured ahead of the two-stage loop in alternating runs: several batches of up to
  // 2048 rows (1 - 3 %); with one batch or longer matrices the two-stage loop is 2 - 14 % ahead.
  const bool slots = g_gemm_slots == 2 || (g_gemm_slots == 1 && batch > 1 && M <= 2048);
  if (b_layout == TLQ_B_KN) {
    if (slots && tile == 256 && K % 128 == 0) {  // whole 128-byte stages
      typedef I8KNLoaderDirect<256, 512> WL;
      typename RowLoaderDirect<256, 512>::Params pa{(const uint8_t*)A, K, M * K, K};
      typename WL::Params pw{(const uint8_t*)B, N, K * N, K};
      return launch_gemm_slots<MmaI8, WL, Epi>(pa, pw, pe, batch, M, N, K, st, what, 2);
    }
#define TLQ_RUN(BM, BN, WM, WN)                                               \
  {                                                                           \
    typedef I8KNLoaderDirect<BN, WM * WN * 64> WL;                            \
    typename WL::Params pw{(const uint8_t*)B, N, K * N, K};                   \
    return run_i8<WL, Epi, BM, BN, WM, WN>(A, pw, pe, batch, M, N, K, st, what); \
  }
    switch (tile) {
      case 32:
        TLQ_RUN(32, 128, 1, 4)
      case 128:
        TLQ_RUN(128, 128, 2, 2)
      default:
        TLQ_RUN(256, 256, 2, 4)
    }
#undef TLQ_RUN
  } else {
    if (slots && tile == 256 && K % 128 == 0) {  // whole 128-byte stages
      typename RowLoaderDirect<256, 512>::Params pa{(const uint8_t*)A, K, M * K, K}, pw{(const uint8_t*)B, K, N * K, K};
      return launch_gemm_slots<MmaI8, RowLoaderDirect<256, 512>, Epi>(pa, pw, pe, batch, M, N, K, st, what, 2);
    }
#define TLQ_RUN(BM, BN, WM, WN)                                               \
  {                                                                           \
    typedef RowLoaderDirect<BN, WM * WN * 64> WL;                             \
    typename WL::Params pw{(const uint8_t*)B, K, N * K, K};                   \
    return run_i8<WL, Epi, BM, BN, WM, WN>(A, pw, pe, batch, M, N, K, st, what); \
  }
    switch (tile) {
      case 32:
        TLQ_RUN(32, 128, 1, 4)
      case 128:
        TLQ_RUN(128, 128, 2, 2)
      default:
        TLQ_RUN(256, 256, 2, 4)
    }
#undef TLQ_RUN
  }
}

int gemm_i8_i32(const void* A, const void* B, void* C, int64_t batch, int64_t M, int64_t N, int64_t K, int b_layout,
                hipStream_t st) {
  EpiInt32::Params pe{(int32_t*)C, N, M * N};
  return dispatch_i8<EpiInt32>(A, B, pe, batch, M, N, K, b_layout, st, "tlq_gemm_i8");
}

int gemm_w8a8_rescale(const void* A, const void* B, const void* scale_a, const void* scale_b, void* C, int64_t batch,
                      int64_t M, int64_t N, int64_t K, int64_t n_scale_b, int b_layout, int out_dtype, hipStream_t st) {
  EpiRescale::Params pe{C, N, M * N, (const float*)scale_a, (const float*)scale_b, n_scale_b, M, out_dtype};
  return dispatch_i8<EpiRescale>(A, B, pe, batch, M, N, K, b_layout, st, "tlq_gemm_w8a8");
}

// ---- split K (one batch, few activation rows) -------------------------------------------------
// With few activation rows the output tiles are too few to fill the machine and the kernel is paced by the weight
// bytes one work-group can pull.  Slice z of K is "batch" z of the loaders (the batch strides step along K) and every
// slice adds its int32 tile into the one accumulator matrix, cleared beforehand: integer adds commute, so the result
// is the exact sum whatever the order.
__global__ __launch_bounds__(256) void i32_clear_kernel(int4_t* __restrict__ p, int64_t n4) {
  for (int64_t i = blockIdx.x * 256 + threadIdx.x; i < n4; i += (int64_t)gridDim.x * 256) p[i] = int4_t{0, 0, 0, 0};
}

// `split` slices of ceil(stages / split) whole stages each, the last one with what is left (at least one stage).
template <class Epi, int BM, int BN, int WM, int WN>
static int run_i8_splitk(const void* A, const void* B, const typename Epi::Params& pe, int64_t M, int64_t N, int64_t K,
                         int64_t split, int b_layout, hipStream_t st) {
  constexpr int NT = WM * WN * 64;
  const int64_t stages = K / kStageBytes;
  const int64_t ks = ceil_div(stages, split) * kStageBytes;
  typedef RowLoaderDirect<BM, NT> AL;
  typename AL::Params pa{(const uint8_t*)A, K, ks, ks};
  if (b_layout == TLQ_B_NK) {
    typedef RowLoaderDirect<BN, NT> WL;
    typename WL::Params pw{(const uint8_t*)B, K, ks, ks};
    return launch_gemm<MmaI8, AL, WL, Epi, BM, BN, WM, WN>(pa, pw, pe, split, M, N, ks, st, "tlq_gemm_i8 (K slices)", 2, (int)stages);
  }
  typedef I8KNLoaderDirect<BN, NT> WL;
  typename WL::Params pw{(const uint8_t*)B, N, ks * N, ks};
  return launch_gemm<MmaI8, AL, WL, Epi, BM, BN, WM, WN>(pa, pw, pe, split, M, N, ks, st, "tlq_gemm_i8 (K slices)", 2, (int)stages);
}

static thread_local int g_i8_split = 0;  // tlq_tune_i8_split: 0 = automatic, 1 = never, n = that many slices where K allows

// Number of K slices for one batch of [M,K] x [N,K] (slice_choice in gemm_core.h): `buffers`: every slice has an int32
// [M,N] matrix of its own, otherwise the slices add into one matrix with atomic adds; `pace`: 2.5 for the loader that
// unpacks int4 on the way into LDS.
int i8_split_choice(int64_t batch, int64_t M, int64_t N, int64_t K, bool buffers, double pace) {
  if (batch != 1 || g_i8_split == 1 || (g_i8_tile && g_i8_split == 0)) return 1;  // a forced tile means: that kernel
  return slice_choice(M, N, K, buffers, pace, g_i8_split);
}

int gemm_i8_i32_splitk(const void* A, const void* B, int32_t* acc, int64_t M, int64_t N, int64_t K, int64_t split,
                       int b_layout, hipStream_t st) {
  split = whole_slices(K / kStageBytes, split);
  const int64_t n4 = M * N / 4;  // N % 16 == 0
  const int64_t want = ceil_div(n4, (int64_t)256);
  i32_clear_kernel<<<(int)(want > 4096 ? 4096 : want), 256, 0, st>>>((int4_t*)acc, n4);
  if (!check_launch("tlq_gemm_i8 (clear)")) return 1;
  if (M <= 32) return run_i8_splitk<EpiAtomicAddI32, 32, 128, 1, 4>(A, B, {acc, N}, M, N, K, split, b_layout, st);
  return run_i8_splitk<EpiAtomicAddI32, 128, 128, 2, 2>(A, B, {acc, N}, M, N, K, split, b_layout, st);
}

// C = rn_out(rn_f32(rn_f32(f32(acc) * scale_a[m]) * scale_b[n])) with acc the sum of the slices' int32 matrices:
// the arithmetic of EpiRescale on the finished sums (four outputs per thread; N % 16 == 0).
__global__ __launch_bounds__(256) void i32_sum_rescale_kernel(const int4_t* __restrict__ partial, int split, void* __restrict__ C,
                                                              const float* __restrict__ scale_a, const float* __restrict__ scale_b,
                                                              int64_t n_scale_b, int64_t n4_total, int n4_row, int out_dtype) {
  for (int64_t i = blockIdx.x * 256 + threadIdx.x; i < n4_total; i += (int64_t)gridDim.x * 256) {
    const int64_t m = i / n4_row;
    const int n = (int)(i - m * n4_row) * 4;
    int4_t a = partial[i];
#pragma unroll 8  // independent loads in flight: with few outputs the pass is paced by their latency
    for (int z = 1; z < split; ++z) a += partial[(int64_t)z * n4_total + i];
    float4_t f;
#pragma unroll
    for (int j = 0; j < 4; ++j) f[j] = (float)a[j];
    if (scale_a) {
      const float sa = scale_a[m];
#pragma unroll
      for (int j = 0; j < 4; ++j) f[j] = f[j] * sa;
    }
    if (scale_b) {
#pragma unroll
      for (int j = 0; j < 4; ++j) f[j] = f[j] * (n_scale_b == 1 ? scale_b[0] : scale_b[n + j]);
    }
    if (out_dtype == TLQ_F32) {
      ((float4_t*)C)[i] = f;
    } else if (out_dtype == TLQ_F16) {
      half_t h[4] = {(half_t)f[0], (half_t)f[1], (half_t)f[2], (half_t)f[3]};
      ((uint2_t*)C)[i] = bitcast<uint2_t>(h);
    } else {
      ((uint2_t*)C)[i] = uint2_t{pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3])};
    }
  }
}

// partial: int32 [split][M][N]
int gemm_w8a8_rescale_splitk(const void* A, const void* B, const void* scale_a, const void* scale_b, void* C, int32_t* partial,
                             int64_t M, int64_t N, int64_t K, int64_t n_scale_b, int64_t split, int b_layout, int out_dtype,
                             hipStream_t st) {
  split = whole_slices(K / kStageBytes, split);
  EpiInt32::Params pe{partial, N, M * N};
  const int rc = M <= 32 ? run_i8_splitk<EpiInt32, 32, 128, 1, 4>(A, B, pe, M, N, K, split, b_layout, st)
                         : run_i8_splitk<EpiInt32, 128, 128, 2, 2>(A, B, pe, M, N, K, split, b_layout, st);
  if (rc) return rc;
  const int64_t n4 = M * N / 4;
  const int64_t want = ceil_div(n4, (int64_t)256);
  i32_sum_rescale_kernel<<<(int)(want > 8192 ? 8192 : want), 256, 0, st>>>((const int4_t*)partial, (int)split, C, (const float*)scale_a,
                                                                            (const float*)scale_b, n_scale_b, n4, (int)(N / 4), out_dtype);
  return check_launch("tlq_gemm_w8a8 (sum and rescale)") ? 0 : 1;
}

int gemm_w4a8_i32(const void* A, const void* Wp, void* C, int64_t M, int64_t N, int64_t K, int sign_mode,
                  hipStream_t st) {
  EpiInt32::Params pe{(int32_t*)C, N, M * N};
  const int tile = pick_tile(1, M, N);
#define TLQ_RUN(BM, BN, WM, WN)                                                                  \
  {                                                                                              \
    typedef W4I8Loader<BN, WM * WN * 64> WL;                                                     \
    typename WL::Params pw{(const uint8_t*)Wp, K / 2, sign_mode, 0};                             \
    return run_i8<WL, EpiInt32, BM, BN, WM, WN>(A, pw, pe, 1, M, N, K, st, "tlq_gemm_w4a8");     \
  }
  switch (tile) {
    case 32:
      TLQ_RUN(32, 128, 1, 4)
    case 128:
      TLQ_RUN(128, 128, 2, 2)
    default:
      TLQ_RUN(256, 256, 2, 4)
  }
#undef TLQ_RUN
}

// C = the sum of the slices' int32 matrices (N % 4 == 0)
__global__ __launch_bounds__(256) void i32_sum_kernel(const int4_t* __restrict__ partial, int split, int4_t* __restrict__ C,
                                                      int64_t n4_total) {
  for (int64_t i = blockIdx.x * 256 + threadIdx.x; i < n4_total; i += (int64_t)gridDim.x * 256) {
    int4_t a = partial[i];
#pragma unroll 8
    for (int z = 1; z < split; ++z) a += partial[(int64_t)z * n4_total + i];
    C[i] = a;
  }
}

// W4A8 over K slices: the unpacking loader is the slowest of the family per work-group (registers, nibble expansion,
// LDS stores), so few output tiles hurt it most.  With `partial` (int32 [split][M][N]) every slice stores its own
// matrix and a second pass sums them; without, the slices add into C (cleared first) with atomic adds.
int gemm_w4a8_i32_splitk(const void* A, const void* Wp, void* C, int64_t M, int64_t N, int64_t K, int sign_mode,
                         int64_t split, int32_t* partial, hipStream_t st) {
  split = whole_slices(K / kStageBytes, split);
  const int64_t n4 = M * N / 4;  // N % 4 == 0
  const int64_t want = ceil_div(n4, (int64_t)256);
  if (!partial) {
    i32_clear_kernel<<<(int)(want > 4096 ? 4096 : want), 256, 0, st>>>((int4_t*)C, n4);
    if (!check_launch("tlq_gemm_w4a8 (clear)")) return 1;
  }
  const int64_t stages = K / kStageBytes;
  const int64_t ks = ceil_div(stages, split) * kStageBytes;
  int rc;
#define TLQ_RUN(Epi, pe, BM, BN, WM, WN)                                                                            \
  {                                                                                                                 \
    constexpr int NT = WM * WN * 64;                                                                                \
    typedef RowLoaderDirect<BM, NT> AL;                                                                             \
    typedef W4I8Loader<BN, NT> WL;                                                                                  \
    typename AL::Params pa{(const uint8_t*)A, K, ks, ks};                                                           \
    typename WL::Params pw{(const uint8_t*)Wp, K / 2, sign_mode, ks / 2};                                           \
    rc = launch_gemm<MmaI8, AL, WL, Epi, BM, BN, WM, WN>(pa, pw, pe, split, M, N, ks, st, "tlq_gemm_w4a8 (K slices)", \
                                                         2, (int)stages);                                           \
  }
  if (partial) {
    EpiInt32::Params pe{partial, N, M * N};
    if (M <= 32) TLQ_RUN(EpiInt32, pe, 32, 128, 1, 4) else TLQ_RUN(EpiInt32, pe, 128, 128, 2, 2)
    if (rc) return rc;
    i32_sum_kernel<<<(int)(want > 8192 ? 8192 : want), 256, 0, st>>>((const int4_t*)partial, (int)split, (int4_t*)C, n4);
    return check_launch("tlq_gemm_w4a8 (sum)") ? 0 : 1;
  }
  EpiAtomicAddI32::Params pe{(int32_t*)C, N};
  if (M <= 32) TLQ_RUN(EpiAtomicAddI32, pe, 32, 128, 1, 4) else TLQ_RUN(EpiAtomicAddI32, pe, 128, 128, 2, 2)
#undef TLQ_RUN
  return rc;
}

}  // namespace tlq

extern "C" {
// Tuning hook used by the benchmark sweeps: forces the activation-tile height (32, 128, 256)
// of the int8 kernels; 0 restores the automatic choice.
void tlq_tune_i8_tile(int block_m) { tlq::g_i8_tile = block_m; }
// Forces the number of K slices of the one-batch int8 kernels: 0 = automatic, 1 = never split, n = up to n slices
// (a power of two, as far as K divides into whole 128-byte stages).
void tlq_tune_i8_split(int slices) { tlq::g_i8_split = slices; }
// The number of K slices the automatic choice (or the forced value) takes for one batch of this shape, with a matrix
// per slice (buffers = 1: tlq_gemm_w8a8_ws) or atomic adds into the one output (0: tlq_gemm_i8).
int tlq_debug_i8_split(int64_t M, int64_t N, int64_t K, int buffers) { return tlq::i8_split_choice(1, M, N, K, buffers != 0, 1.0); }
}
