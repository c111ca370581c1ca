// Plain fp16 / bf16 GEMM with fp32 accumulation: C[b, M, N] = A[b, M, K] . B[b], B[b] stored [K, N]
// (transposed on the fly) or [N, K]; the matrices of a batch follow each other densely.
#include "gemm_core.h"
#include "gemm_slots.h"

namespace tlq {

// 16-bit source stored [K, N] (N contiguous): 4(k) x 8(n) register blocks are transposed with
// v_perm_b32 and written as 8-byte pieces (4 consecutive k of one n) into the [n][k] LDS tile.
template <int ROWS, int NT>
struct H16KNLoader {
  typedef RowFrag Frag;
  static constexpr bool DIRECT = false;
  static constexpr bool PREFETCH2 = false;
  static constexpr int NBLK = ROWS / 8;            // 8-column blocks per tile
  static constexpr int PASSES = (16 * NBLK) / NT;  // 64 k = 16 blocks of 4 rows
  static constexpr int UNITS = PASSES * 4;
  static_assert(PASSES >= 1 && (16 * NBLK) % NT == 0 && NT % NBLK == 0, "bad transposing loader shape");
  struct Params {
    const uint8_t* base;  // B[0, 0]
    int64_t ld;           // bytes per k row (= 2 N)
    int64_t batch_stride;
    int64_t k_total;
  };
  struct Regs {
    uint4_t v[PASSES][4];
  };
  const uint8_t* base;  // uniform
  uint32_t ld;
  uint32_t voff;  // per lane: kblk0 * 4 * ld + col * 2
  int kblk0, nblk;
  int k_total;

  // cols_total must be a multiple of 8 (checked on the host)
  __device__ __forceinline__ H16KNLoader(const Params& p, int batch, int col0, int cols_total, int tid)
      : base(p.base + batch * p.batch_stride + (int64_t)col0 * 2), ld((uint32_t)p.ld), k_total((int)p.k_total) {
    const int cols_valid = cols_total - col0;
    nblk = tid % NBLK;
    kblk0 = tid / NBLK;
    int col = nblk * 8;
    col = col < cols_valid ? col : cols_valid - 8;
    voff = (uint32_t)(kblk0 * 4) * ld + (uint32_t)(col * 2);
  }

  template <bool TAIL>
  __device__ __forceinline__ void gload(Regs& r, int kt, uint8_t* /*lds_next*/ = nullptr) const {
    const uint8_t* sb = base + (int64_t)kt * 64 * ld;
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t o = voff + (uint32_t)(ps * (NT / NBLK) * 4 + i) * ld;
        if (!TAIL) {
          r.v[ps][i] = *(const uint4_t*)(sb + o);
        } else {
          const int k = kt * 64 + (ps * (NT / NBLK) + kblk0) * 4 + i;
          const bool ok = k < k_total;
          uint4_t v = *(const uint4_t*)(ok ? sb + o : base + (voff - (uint32_t)(kblk0 * 4) * ld));
          if (!ok) v = uint4_t{0u, 0u, 0u, 0u};
          r.v[ps][i] = v;
        }
      }
    }
  }
  __device__ __forceinline__ void lstore(const Regs& r, uint8_t* lds) const { lstore_piece(r, lds, 0, 1); }
  __device__ __forceinline__ void lstore_piece(const Regs& r, uint8_t* lds, int pc, int np) const {
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      const int kblk = ps * (NT / NBLK) + kblk0;
      const int chunk = kblk >> 1;
      const int within = (kblk & 1) * 8;
#pragma unroll
      for (int w = 0; w < 4; ++w) {  // word w of each row holds columns 2w, 2w+1
        if ((ps * 4 + w) * np / UNITS != pc) continue;
        const uint32_t a = r.v[ps][0][w], b = r.v[ps][1][w], c = r.v[ps][2][w], d = r.v[ps][3][w];
        uint2_t even, odd;
        even.x = __builtin_amdgcn_perm(b, a, 0x05040100u);  // (a.lo, b.lo)
        even.y = __builtin_amdgcn_perm(d, c, 0x05040100u);  // (c.lo, d.lo)
        odd.x = __builtin_amdgcn_perm(b, a, 0x07060302u);   // (a.hi, b.hi)
        odd.y = __builtin_amdgcn_perm(d, c, 0x07060302u);
        *(uint2_t*)(lds + lds_off(nblk * 8 + 2 * w, chunk) + within) = even;
        *(uint2_t*)(lds + lds_off(nblk * 8 + 2 * w + 1, chunk) + within) = odd;
      }
    }
  }
};

// tlq_tune_gemm_tile: 0 = automatic, 128 / 256 = that square tile
thread_local int g_gemm_f16_tile = 0;

template <class Mma, int BM, int BN, int WM, int WN>
static int run_f16(const void* A, const void* B, void* C, int64_t batch, int64_t M, int64_t N, int64_t K, int out_dtype,
                   int b_layout, hipStream_t st) {
  constexpr int NT = WM * WN * 64;
  typedef RowLoaderDirect<BM, NT> AL;
  typename AL::Params pa{(const uint8_t*)A, K * 2, M * K * 2, K * 2};
  EpiFloat::Params pe{C, N, M * N, out_dtype};
  if (b_layout == TLQ_B_NK) {
    typedef RowLoaderDirect<BN, NT> WL;
    typename WL::Params pw{(const uint8_t*)B, K * 2, N * K * 2, K * 2};
    return launch_gemm<Mma, AL, WL, EpiFloat, BM, BN, WM, WN>(pa, pw, pe, batch, M, N, K * 2, st, "tlq_gemm_f16");
  }
  if (N % 8 == 0) {  // [K, N] rows are whole 16-byte chunks: copied as they are, transposed by the operand read
    typedef H16KNLoaderDirect<BN, NT> WL;
    H16KNParams pw{(const uint8_t*)B, N * 2, K * N * 2, K};
    return launch_gemm<Mma, AL, WL, EpiFloat, BM, BN, WM, WN>(pa, pw, pe, batch, M, N, K * 2, st, "tlq_gemm_f16");
  }
  typedef H16KNLoader<BN, NT> WL;
  typename WL::Params pw{(const uint8_t*)B, N * 2, K * N * 2, K};
  return launch_gemm<Mma, AL, WL, EpiFloat, BM, BN, WM, WN>(pa, pw, pe, batch, M, N, K * 2, st, "tlq_gemm_f16");
}

// Split-K: slice z of K is "batch" z of the loaders (the batch strides step along K), and every slice
// adds its partial tile into the one fp32 C.
template <class Mma, int BM, int BN, int WM, int WN>
static int run_f16_splitk(const void* A, const void* B, float* C, int64_t M, int64_t N, int64_t K, int64_t split_k,
                          int b_layout, hipStream_t st) {
  constexpr int NT = WM * WN * 64;
  const int64_t ks = K / split_k;
  typedef RowLoaderDirect<BM, NT> AL;
  typename AL::Params pa{(const uint8_t*)A, K * 2, ks * 2, ks * 2};
  EpiAtomicAdd::Params pe{C, N};
  if (b_layout == TLQ_B_NK) {
    typedef RowLoaderDirect<BN, NT> WL;
    typename WL::Params pw{(const uint8_t*)B, K * 2, ks * 2, ks * 2};
    return launch_gemm<Mma, AL, WL, EpiAtomicAdd, BM, BN, WM, WN>(pa, pw, pe, split_k, M, N, ks * 2, st, "tlq_gemm_f16_splitk");
  }
  if (N % 8 == 0) {
    typedef H16KNLoaderDirect<BN, NT> WL;
    H16KNParams pw{(const uint8_t*)B, N * 2, ks * N * 2, ks};
    return launch_gemm<Mma, AL, WL, EpiAtomicAdd, BM, BN, WM, WN>(pa, pw, pe, split_k, M, N, ks * 2, st, "tlq_gemm_f16_splitk");
  }
  typedef H16KNLoader<BN, NT> WL;
  typename WL::Params pw{(const uint8_t*)B, N * 2, ks * N * 2, ks};
  return launch_gemm<Mma, AL, WL, EpiAtomicAdd, BM, BN, WM, WN>(pa, pw, pe, split_k, M, N, ks * 2, st, "tlq_gemm_f16_splitk");
}

int gemm_f16_splitk(const void* A, const void* B, float* C, int64_t M, int64_t N, int64_t K, int64_t split_k,
                    int in_dtype, int b_layout, hipStream_t st) {
  const bool small = prefer_small_tiles(split_k, M, N);
  if (in_dtype == TLQ_F16)
    return small ? run_f16_splitk<MmaF16, 128, 128, 2, 2>(A, B, C, M, N, K, split_k, b_layout, st)
                 : run_f16_splitk<MmaF16, 256, 256, 2, 4>(A, B, C, M, N, K, split_k, b_layout, st);
  return small ? run_f16_splitk<MmaBF16, 128, 128, 2, 2>(A, B, C, M, N, K, split_k, b_layout, st)
               : run_f16_splitk<MmaBF16, 256, 256, 2, 4>(A, B, C, M, N, K, split_k, b_layout, st);
}


// ---- K slices with a matrix per slice (one batch, few activation rows) ---------------------------
// With few activation rows the output tiles are too few to fill the machine and a work-group's run of stages is
// latency bound.  Slice z of K is "batch" z of the loaders; slices are whole 128-byte stages, the last one holds what is
// left; every slice stores its fp32 tile into its own [M, N] matrix and a second pass adds them in slice order and
// rounds once (deterministic, unlike the atomic adds of gemm_f16_splitk).
void launch_splitk_reduce(const float* partial, void* C, int64_t M, int64_t N, int split, int out_dtype, hipStream_t st);

thread_local int g_f16_split = 0;  // tlq_tune_f16_split: 0 = automatic, 1 = never, n = up to n slices

// The estimate is slice_choice's (gemm_core.h): a row is K * 2 bytes, every slice has a matrix of its own.
int f16_split_choice(int64_t batch, int64_t M, int64_t N, int64_t K) {
  if (batch != 1 || g_f16_split == 1 || (g_gemm_f16_tile && g_f16_split == 0)) return 1;
  return slice_choice(M, N, K * 2, true, 1.0, g_f16_split);
}

template <class Mma, int BM, int BN, int WM, int WN>
static int run_f16_slices(const void* A, const void* B, float* partial, int64_t M, int64_t N, int64_t K, int64_t split,
                          int b_layout, hipStream_t st) {
  constexpr int NT = WM * WN * 64;
  const int64_t stages = K * 2 / kStageBytes;
  const int64_t ksb = ceil_div(stages, split) * kStageBytes;  // bytes of K per slice
  typedef RowLoaderDirect<BM, NT> AL;
  typename AL::Params pa{(const uint8_t*)A, K * 2, ksb, ksb};
  EpiFloat::Params pe{partial, N, M * N, TLQ_F32};
  if (b_layout == TLQ_B_NK) {
    typedef RowLoaderDirect<BN, NT> WL;
    typename WL::Params pw{(const uint8_t*)B, K * 2, ksb, ksb};
    return launch_gemm<Mma, AL, WL, EpiFloat, BM, BN, WM, WN>(pa, pw, pe, split, M, N, ksb, st, "tlq_gemm_f16 (K slices)", 4, (int)stages);
  }
  typedef H16KNLoaderDirect<BN, NT> WL;  // N % 8 == 0
  H16KNParams pw{(const uint8_t*)B, N * 2, (ksb / 2) * N * 2, ksb / 2};
  return launch_gemm<Mma, AL, WL, EpiFloat, BM, BN, WM, WN>(pa, pw, pe, split, M, N, ksb, st, "tlq_gemm_f16 (K slices)", 4, (int)stages);
}

// partial: fp32 [split][M][N]
int gemm_f16_slices(const void* A, const void* B, void* C, float* partial, int64_t M, int64_t N, int64_t K, int64_t split,
                    int in_dtype, int out_dtype, int b_layout, hipStream_t st) {
  split = whole_slices(K * 2 / kStageBytes, split);  // no empty slice
  int rc;
  if (in_dtype == TLQ_F16)
    rc = M <= 32 ? run_f16_slices<MmaF16, 32, 128, 1, 4>(A, B, partial, M, N, K, split, b_layout, st)
                 : run_f16_slices<MmaF16, 128, 128, 2, 2>(A, B, partial, M, N, K, split, b_layout, st);
  else
    rc = M <= 32 ? run_f16_slices<MmaBF16, 32, 128, 1, 4>(A, B, partial, M, N, K, split, b_layout, st)
                 : run_f16_slices<MmaBF16, 128, 128, 2, 2>(A, B, partial, M, N, K, split, b_layout, st);
  if (rc) return rc;
  launch_splitk_reduce(partial, C, M, N, (int)split, out_dtype, st);
  return check_launch("tlq_gemm_f16 (sum of the slices)") ? 0 : 1;
}

template <class Mma>
static int dispatch_f16(const void* A, const void* B, void* C, int64_t batch, int64_t M, int64_t N, int64_t K, int out_dtype,
                        int b_layout, hipStream_t st) {
  const bool small = g_gemm_f16_tile ? g_gemm_f16_tile == 128 : prefer_small_tiles(batch, M, N);
  if (small)
    return run_f16<Mma, 128, 128, 2, 2>(A, B, C, batch, M, N, K, out_dtype, b_layout, st);
  // (the five-slot kernel only on request: alternating runs on one box have the two-stage loop 3 - 14 % ahead on ten of
  // twelve 16-bit shapes, 2 % behind on the other two)
  if (g_gemm_slots == 2 && b_layout == TLQ_B_NK && K % 64 == 0) {  // whole 128-byte stages
    typename RowLoaderDirect<256, 512>::Params pa{(const uint8_t*)A, K * 2, M * K * 2, K * 2},
        pw{(const uint8_t*)B, K * 2, N * K * 2, K * 2};
    EpiFloat::Params pe{C, N, M * N, out_dtype};
    return launch_gemm_slots<Mma, RowLoaderDirect<256, 512>, EpiFloat>(pa, pw, pe, batch, M, N, K * 2, st, "tlq_gemm_f16", 4);
  }
  if (g_gemm_slots == 2 && b_layout == TLQ_B_KN && K % 64 == 0 && N % 8 == 0) {  // [K, N] weights, transposed in the operand read
    typename RowLoaderDirect<256, 512>::Params pa{(const uint8_t*)A, K * 2, M * K * 2, K * 2};
    H16KNParams pw{(const uint8_t*)B, N * 2, K * N * 2, K};
    EpiFloat::Params pe{C, N, M * N, out_dtype};
    return launch_gemm_slots<Mma, H16KNLoaderDirect<256, 512>, EpiFloat>(pa, pw, pe, batch, M, N, K * 2, st, "tlq_gemm_f16", 4);
  }
  return run_f16<Mma, 256, 256, 2, 4>(A, B, C, batch, M, N, K, out_dtype, b_layout, st);
}

int gemm_f16_plain(const void* A, const void* B, void* C, int64_t batch, int64_t M, int64_t N, int64_t K, int in_dtype,
                   int out_dtype, int b_layout, hipStream_t st) {
  if (in_dtype == TLQ_F16) return dispatch_f16<MmaF16>(A, B, C, batch, M, N, K, out_dtype, b_layout, st);
  return dispatch_f16<MmaBF16>(A, B, C, batch, M, N, K, out_dtype, b_layout, st);
}

}  // namespace tlq
