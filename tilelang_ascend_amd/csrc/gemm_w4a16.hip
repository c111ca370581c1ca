// W4A16 prefill GEMM: packed-int4 weights are dequantised on their way from global memory
// into the LDS weight tile, then fp16 / bf16 MFMA with fp32 accumulation.
//
//   W[n, k] = rn_T( rn_T(T(u) - z) * s ),  C[m, n] = rn_out( sum_k A[m, k] * W[n, k] )
//
// The dequantised tile holds exactly the values of the stand-alone dequantisation kernel
// (one rounding per operation), so the GEMM result equals "dequantise, then fp32-accumulated
// matmul" up to summation order.
//
// One stage is 64 values of K: 32 packed bytes per weight row.  A thread loads 16 packed
// bytes (32 weights of one quantisation group) plus that group's scale / zero, and later
// expands them to four 16-byte LDS chunks.
//
// fp16 expansion, per 32-bit word (8 nibbles k0..k7):
//   (x    & 0x000f000f) | 0x64006400 -> half2 (1024+k0, 1024+k4)     one v_bfi_b32 each
//   (x    & 0x00f000f0) | 0x54005400 -> half2 (  64+k1,   64+k5)
//   (x>>8 & ...) likewise             -> (k2, k6), (k3, k7)
//   packed subtract of the bias (and of an integer zero point folded into it, exact), packed
//   multiply by the scale, then four v_perm_b32 put the halves back into k order.
// bf16 expansion: v_cvt_f32_ubyteN on the masked nibbles, fp32 fma / sub+mul with explicit
// bfloat16 roundings, v_cvt_pk_bf16_f32 to pack pairs in k order.
#include "gemm_core.h"
#include "expand8.h"

namespace tlq {

template <typename T, bool FOLD, int ROWS, int NT>
struct W4Loader {
  typedef RowFrag Frag;
  static constexpr bool DIRECT = false;
  static constexpr bool PREFETCH2 = true;  // convert from registers loaded one stage earlier
  static constexpr int SLOTS = ROWS * 2;  // 16-byte packed loads per stage
  static constexpr int PASSES = (SLOTS + NT - 1) / NT;
  static constexpr bool PARTIAL = SLOTS % NT != 0;
  static constexpr int UNITS = PASSES * 4;  // one unit = one 32-bit word -> one 16-byte LDS chunk
  static_assert(PASSES == 1 || (NT / 2) % 8 == 0, "pass stride must keep the swizzle phase");
  struct Params {
    const uint8_t* wp;
    const T* scales;  // never null: the host passes a dummy readable pointer when there are no scales
    const T* zeros;
    int64_t row_bytes;  // K / 2
    int groups;         // K / group
    int group_shift;    // log2(group); group is a power of two here
    float zero_scalar;
    int has_scales, has_zeros;
    int64_t slice_bytes;  // split-K: packed bytes of one K slice within a row (0 without a split) ...
    int slice_groups;     // ... and its number of quantisation groups; slice z is the kernel's "batch" z
  };
  struct Regs {
    uint4_t v[PASSES];
    uint32_t sz[PASSES];  // scale in the low half, zero point in the high half: 16-bit members of a struct that crosses
                          // a stage boundary are passed through scratch memory by the compiler (a round trip per stage)
  };
  const uint8_t* base;  // uniform: first packed row of the tile
  const T* sbase;       // uniform: scales / zeros row of the tile's first row
  const T* zbase;
  uint32_t voff[PASSES];  // per lane: row * row_bytes + half * 16
  uint32_t goff[PASSES];  // per lane: row * groups + (lane-fixed part of the group index)
  uint32_t loff[4];       // per lane: LDS offsets of the four chunks this lane writes (pass 0)
  int group_shift;
  bool has_s, has_z, active;
  T one, zs;
  NibbleMagic mg;

  __device__ __forceinline__ W4Loader(const Params& p, int batch, int row0, int rows_total, int tid)
      : base(p.wp + (int64_t)row0 * p.row_bytes + batch * p.slice_bytes), group_shift(p.group_shift),
        has_s(p.has_scales != 0), has_z(p.has_zeros != 0), one(from_float<T>(1.0f)), zs(from_float<T>(p.zero_scalar)),
        mg(make_nibble_magic()) {
    const int rows_valid = rows_total - row0;
    sbase = p.scales + (has_s ? (int64_t)row0 * p.groups + batch * p.slice_groups : 0);
    zbase = p.zeros + (has_z ? (int64_t)row0 * p.groups + batch * p.slice_groups : 0);
    const int half = tid & 1;
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      int row = (ps * NT + tid) >> 1;
      row = row < rows_valid ? row : rows_valid - 1;  // clamp: loads stay in bounds, results are masked later
      voff[ps] = (uint32_t)row * (uint32_t)p.row_bytes + (uint32_t)(half * 16);
      goff[ps] = (uint32_t)row * (uint32_t)p.groups + (uint32_t)((half * 32) >> group_shift);
    }
    const int r0 = tid >> 1;
#pragma unroll
    for (int j = 0; j < 4; ++j) loff[j] = (uint32_t)lds_off(r0, half * 4 + j);
    active = !PARTIAL || ((PASSES - 1) * NT + tid) < SLOTS;
  }

  // K is a multiple of 64 on this path, so every stage is complete (TAIL is never needed).
  // Group index of element (kt*64 + half*32) = ((kt*64) >> shift) + ((half*32) >> shift) for every
  // power-of-two group >= 32.
  template <bool TAIL>
  __device__ __forceinline__ void gload(Regs& r, int kt, uint8_t* /*lds_next*/ = nullptr) const {
    const uint8_t* sb = base + (int64_t)kt * 32;
    const uint32_t gk = (uint32_t)((kt * 64) >> group_shift);
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      r.v[ps] = *(const uint4_t*)(sb + voff[ps]);
      const T sv = sbase[has_s ? goff[ps] + gk : 0u];
      const T zv = zbase[has_z ? goff[ps] + gk : 0u];
      r.sz[ps] = (uint32_t)bitcast<uint16_t>(has_s ? sv : one) | ((uint32_t)bitcast<uint16_t>(has_z ? zv : zs) << 16);
    }
  }
  __device__ __forceinline__ void lstore_piece(const Regs& r, uint8_t* lds, int pc, int np) const {
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      if (PARTIAL && ps == PASSES - 1 && !active) continue;
      const Expand8<T, FOLD> ex(bitcast<T>((uint16_t)(r.sz[ps] & 0xffffu)), bitcast<T>((uint16_t)(r.sz[ps] >> 16)), mg);
      const uint32_t w[4] = {r.v[ps].x, r.v[ps].y, r.v[ps].z, r.v[ps].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if ((ps * 4 + j) * np / UNITS != pc) continue;
        *(uint4_t*)(lds + loff[j] + ps * (NT / 2) * kStageBytes) = ex(w[j]);
      }
    }
  }
  __device__ __forceinline__ void lstore(const Regs& r, uint8_t* lds) const { lstore_piece(r, lds, 0, 1); }
};

template <typename T>
struct MmaOf;
template <>
struct MmaOf<half_t> {
  typedef MmaF16 type;
};
template <>
struct MmaOf<bf16_t> {
  typedef MmaBF16 type;
};

template <int ROWS, int NT>
using W4LoaderF16Fold = W4Loader<half_t, true, ROWS, NT>;
template <int ROWS, int NT>
using W4LoaderF16Gen = W4Loader<half_t, false, ROWS, NT>;
template <int ROWS, int NT>
using W4LoaderBF16Fold = W4Loader<bf16_t, true, ROWS, NT>;
template <int ROWS, int NT>
using W4LoaderBF16Gen = W4Loader<bf16_t, false, ROWS, NT>;

struct W4Args {
  const void *A, *Wp, *scales, *zeros;
  void* C;
  int64_t M, N, K, group;
  float zero_scalar;
  int out_dtype;
  hipStream_t st;
  int64_t split = 1;         // K slices handled by different work-groups (the MFMA tile kernel only)
  float* partial = nullptr;  // [split][M][N] fp32 partial sums when split > 1
};

template <typename T, bool FOLD, int ROWS, int NT>
static typename W4Loader<T, FOLD, ROWS, NT>::Params w4_params(const W4Args& a) {
  int shift = 0;
  while (((int64_t)1 << shift) < a.group) ++shift;
  const T* dummy = (const T*)a.A;  // readable placeholder for absent scale / zero tensors
  return {(const uint8_t*)a.Wp,
          a.scales ? (const T*)a.scales : dummy,
          a.zeros ? (const T*)a.zeros : dummy,
          a.K / 2,
          (int)(a.K / a.group),
          shift,
          a.zero_scalar,
          a.scales ? 1 : 0,
          a.zeros ? 1 : 0,
          a.split > 1 ? a.K / a.split / 2 : 0,
          a.split > 1 ? (int)(a.K / a.split / a.group) : 0};
}

template <typename T, bool FOLD, int BM, int BN, int WM, int WN>
static int run_w4a16(const W4Args& a) {
  constexpr int NT = WM * WN * 64;
  // activations travel global -> LDS directly whenever the tile splits into whole wavefront loads
  constexpr bool DIRECT = BM % 8 == 0 && (BM / 8) % (NT / 64) == 0;
  typedef typename std::conditional<DIRECT, RowLoaderDirect<DIRECT ? BM : 8 * (NT / 64), NT>, RowLoader<BM, NT>>::type AL;
  typedef W4Loader<T, FOLD, BN, NT> WL;
  auto pw = w4_params<T, FOLD, BN, NT>(a);
  if (a.split > 1) {
    // slice z of K is "batch" z of the loaders; every slice writes its own fp32 partial matrix
    const int64_t ks = a.K / a.split;
    typename AL::Params pa{(const uint8_t*)a.A, a.K * 2, ks * 2, ks * 2};
    EpiFloat::Params pe{a.partial, a.N, a.M * a.N, TLQ_F32};
    return launch_gemm<typename MmaOf<T>::type, AL, WL, EpiFloat, BM, BN, WM, WN>(pa, pw, pe, a.split, a.M, a.N, ks * 2, a.st,
                                                                                 "tlq_gemm_w4a16(mfma, split K)", 8);
  }
  typename AL::Params pa{(const uint8_t*)a.A, a.K * 2, 0, a.K * 2};
  EpiFloat::Params pe{a.C, a.N, 0, a.out_dtype};
  return launch_gemm<typename MmaOf<T>::type, AL, WL, EpiFloat, BM, BN, WM, WN>(pa, pw, pe, 1, a.M, a.N, a.K * 2, a.st,
                                                                               "tlq_gemm_w4a16(mfma)", 8);
}

// tile override for tuning runs (0 = automatic)
static thread_local int g_w4a16_tile = 0;

template <typename T, bool FOLD>
static int dispatch_w4a16(const W4Args& a) {
  int tile = g_w4a16_tile;
  const int64_t M = a.M, N = a.N;
  if (tile == 0) {
    if (M <= 16)
      tile = 16;
    else if (M <= 32)
      tile = 32;
    else if (M <= 64)
      tile = 64;
    else if (M <= 128 || (a.split <= 1 && prefer_small_tiles(1, M, N, 0.65)))
      tile = 128;  // few large tiles: smaller ones fill more CUs, unless K is being cut for that purpose
    else
      tile = 256;
  }
  switch (tile) {
    case 16:
      return run_w4a16<T, FOLD, 16, 64, 1, 4>(a);
    case 32:
      return run_w4a16<T, FOLD, 32, 128, 1, 4>(a);
    case 64:
      return run_w4a16<T, FOLD, 64, 256, 1, 4>(a);
    case 128:
      return run_w4a16<T, FOLD, 128, 128, 2, 2>(a);
    default:
      return run_w4a16<T, FOLD, 256, 256, 2, 4>(a);
  }
}

// ---- skinny kernel: a few activation rows (M <= 64) against a large weight matrix ---------------
// HBM bound: every packed weight is read once and goes straight from global memory through the
// dequantiser into an MFMA operand register; there is no LDS tile.  A wavefront owns RT tiles of 16
// weight rows and a slice of K; per 128 values of K ("k-block") lane (row r = lane % 16, k-group
// q = lane / 16) loads the 16 packed bytes of k = 128*kb + 32*q .. +31 of its row (one quantisation
// group, so one scale / zero per lane and k-block), expands them into four 8-value operands, and
// feeds four MFMAs whose activation operand holds A[m = lane % 16][the same 8 k] (the MFMA does not
// care which k a k-group holds as long as both operands agree).  The wavefronts of a work-group
// split K between them and add their partial tiles through LDS, so no global reduction is needed.
template <typename T, bool FOLD, int RT, int MT>
__global__ __launch_bounds__(MT >= 4 ? 512 : 1024) void w4a16_skinny_kernel(const T* __restrict__ A, const uint8_t* __restrict__ Wp,
                                                            const T* __restrict__ scales, const T* __restrict__ zeros,
                                                            void* __restrict__ C, int M, int N, int K, int group,
                                                            float zero_scalar, int out_dtype) {
  typedef typename MmaOf<T>::type Mma;
  extern __shared__ __align__(16) uint8_t smem[];
  float4_t* const red = (float4_t*)smem;  // [waves][RT * MT][64 lanes]
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int waves = blockDim.x >> 6;
  const int r16 = lane & 15, q = lane >> 4;
  const int n_base = blockIdx.x * (16 * RT);
  const int groups = K / group;
  const int KB = K >> 7;
  const int kb0 = (int)(((int64_t)wave * KB) / waves), kb1 = (int)(((int64_t)(wave + 1) * KB) / waves);
  const bool has_s = scales != nullptr, has_z = zeros != nullptr;
  const T one = from_float<T>(1.0f), zs = from_float<T>(zero_scalar);
  const NibbleMagic mg = make_nibble_magic();

  uint32_t woff[RT], goff[RT], aoff[MT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    int n = n_base + rt * 16 + r16;
    n = n < N ? n : N - 1;  // clamp: loads stay in bounds, the rows are masked at the store
    woff[rt] = (uint32_t)n * (uint32_t)(K >> 1) + (uint32_t)(q * 16);
    goff[rt] = (uint32_t)n * (uint32_t)groups;
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int m = mt * 16 + r16;
    m = m < M ? m : M - 1;
    aoff[mt] = ((uint32_t)m * (uint32_t)K + (uint32_t)(q * 32)) * 2u;
  }
  const T* const sp = has_s ? scales : A;  // absent tensors: read a valid dummy location, discard the value
  const T* const zp = has_z ? zeros : A;

  struct Block {
    uint4_t w[RT];
    uint32_t sz[RT];  // scale | zero point << 16 (16-bit struct members would travel through scratch memory)
    uint4_t a[MT][4];
  };
  auto load = [&](Block& b, int kb) {
    const uint32_t gi = (uint32_t)((kb * 128 + q * 32) / group);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      b.w[rt] = *(const uint4_t*)(Wp + woff[rt] + (uint32_t)kb * 64u);
      const T sv = sp[has_s ? goff[rt] + gi : 0u];
      const T zv = zp[has_z ? goff[rt] + gi : 0u];
      b.sz[rt] = (uint32_t)bitcast<uint16_t>(has_s ? sv : one) | ((uint32_t)bitcast<uint16_t>(has_z ? zv : zs) << 16);
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < 4; ++j) b.a[mt][j] = *(const uint4_t*)((const uint8_t*)A + aoff[mt] + (uint32_t)kb * 256u + j * 16);
  };

  typename Mma::acc_t acc[RT][MT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = typename Mma::acc_t{0, 0, 0, 0};
  auto compute = [&](const Block& b) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const Expand8<T, FOLD> ex(bitcast<T>((uint16_t)(b.sz[rt] & 0xffffu)), bitcast<T>((uint16_t)(b.sz[rt] >> 16)), mg);
      const uint32_t w[4] = {b.w[rt].x, b.w[rt].y, b.w[rt].z, b.w[rt].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint4_t wf = ex(w[j]);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = Mma::mma(wf, b.a[mt][j], acc[rt][mt]);
      }
    }
  };

  // A wavefront's slice of K is only a few k-blocks long, and one k-block of arithmetic is far
  // shorter than a trip to memory: issue the loads of DEPTH k-blocks at once, then compute them.
  // (Other wavefronts of the CU cover the time between chunks.)
  constexpr int DEPTH = MT == 1 ? 4 : (MT == 2 ? 2 : 1);
  Block b[DEPTH];
  for (int kb = kb0; kb < kb1; kb += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int k = kb + d < kb1 ? kb + d : kb1 - 1;  // past the slice: reload the last block, skip its arithmetic
      load(b[d], k);
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
      if (kb + d < kb1) compute(b[d]);
  }

  // add the partial tiles of the wavefronts (they hold different slices of K)
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) red[(wave * (RT * MT) + rt * MT + mt) * 64 + lane] = acc[rt][mt];
  __syncthreads();
  for (int item = threadIdx.x; item < RT * MT * 64; item += blockDim.x) {
    float4_t sum = red[item];
    for (int w = 1; w < waves; ++w) {
      const float4_t v = red[w * (RT * MT * 64) + item];
      sum[0] += v[0];
      sum[1] += v[1];
      sum[2] += v[2];
      sum[3] += v[3];
    }
    // lane l of a tile holds D[n = 4 * (l / 16) + i][m = l % 16]
    const int tile = item >> 6, l = item & 63;
    const int rt = tile / MT, mt = tile - rt * MT;
    const int m = mt * 16 + (l & 15);
    const int n = n_base + rt * 16 + 4 * (l >> 4);
    if (m >= M || n >= N) continue;
    const int64_t idx = (int64_t)m * N + n;
    if (n + 3 < N && (N & 3) == 0) {
      if (out_dtype == TLQ_F32) {
        *(float4_t*)((float*)C + idx) = sum;
      } else if (out_dtype == TLQ_F16) {
        half_t h[4] = {(half_t)sum[0], (half_t)sum[1], (half_t)sum[2], (half_t)sum[3]};
        *(uint2_t*)((half_t*)C + idx) = bitcast<uint2_t>(h);
      } else {
        uint2_t o;
        o.x = pack_bf16x2(sum[0], sum[1]);
        o.y = pack_bf16x2(sum[2], sum[3]);
        *(uint2_t*)((uint16_t*)C + idx) = o;
      }
    } else {
      for (int i = 0; i < 4 && n + i < N; ++i) store_out(C, idx + i, sum[i], out_dtype);
    }
  }
}

// ---- skinny kernel for M <= 16, operands staged through wavefront-private LDS -------------------
// The direct form above asks every lane for 16 bytes of a different row, which the memory pipeline
// serves one lane per cycle.  Here every global access is a full-width direct global -> LDS load
// (1 KB per wavefront instruction, adjacent lanes adjacent addresses): per k-block RT loads of a
// [16 rows][64 B] packed-weight tile and four loads of the [16 rows][256 B] activation tile, into one
// of two slots of LDS that only this wavefront uses (so there is no barrier, only counters).  The
// MFMA-shaped fragments are then read back with ds_read_b128; 16-byte pieces are XOR-swizzled on the
// global side so that those reads are conflict free.  Scales / zeros come in as dword gathers that
// cover four consecutive groups of the 16 rows at once, i.e. once per four k-blocks at group 128.
// While k-block i is dequantised and multiplied, the loads of i+1 and i+2 are in flight.
template <typename T, bool FOLD, int RT>
__global__ __launch_bounds__(1024) void w4a16_skinny_lds_kernel(const T* __restrict__ A, const uint8_t* __restrict__ Wp,
                                                                const T* __restrict__ scales, const T* __restrict__ zeros,
                                                                void* __restrict__ C, int M, int N, int K, int gshift,
                                                                float zero_scalar, int out_dtype) {
  typedef typename MmaOf<T>::type Mma;
  typedef __attribute__((address_space(3))) uint8_t* lptr_t;
  constexpr int SLOT = RT * 1024 + 4096;  // RT weight tiles + one activation tile
  constexpr int SC = RT * 2 * 256;        // [rt][scale | zero][64 dwords]
  constexpr int WAVE_LDS = 2 * SLOT + 2 * SC;
  constexpr int NI = RT + 4;              // direct loads per k-block
  extern __shared__ __align__(16) uint8_t smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int waves = blockDim.x >> 6;
  const int r16 = lane & 15, q = lane >> 4;
  uint8_t* const mine = smem + wave * WAVE_LDS;
  const uint32_t mine_lds = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lptr_t)mine);
  const int n_base = blockIdx.x * (16 * RT);
  const int groups = K >> gshift;
  const int KB = K >> 7;
  const int kb0 = (int)(((int64_t)wave * KB) / waves), kb1 = (int)(((int64_t)(wave + 1) * KB) / waves);
  const int nkb = kb1 - kb0;
  const bool has_s = scales != nullptr, has_z = zeros != nullptr;
  const int NS = RT * ((has_s ? 1 : 0) + (has_z ? 1 : 0));  // gathers per scale period (uniform)
  const T one = from_float<T>(1.0f), zs = from_float<T>(zero_scalar);
  const NibbleMagic mg = make_nibble_magic();

  // ---- per-lane source offsets of the direct loads ----
  uint32_t voff_w[RT], voff_a[4], row_g[RT];
  {
    const int rho = lane >> 2, piece = (lane & 3) ^ ((rho >> 1) & 3);  // lands on row lane/4, physical piece lane%4
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      int n = n_base + rt * 16 + rho;
      n = n < N ? n : N - 1;
      voff_w[rt] = (uint32_t)n * (uint32_t)(K >> 1) + (uint32_t)(piece * 16);
      int ng = n_base + rt * 16 + r16;  // the row this lane gathers scales for / dequantises
      ng = ng < N ? ng : N - 1;
      row_g[rt] = (uint32_t)ng * (uint32_t)groups;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = i * 4 + (lane >> 4);
      const int lp = (lane & 15) ^ (row & 7);  // physical piece lane%16 holds logical piece lp
      const int m = row < M ? row : M - 1;
      voff_a[i] = ((uint32_t)m * (uint32_t)K) * 2u + (uint32_t)(lp * 16);
    }
  }
  // ---- per-lane LDS offsets of the fragment reads ----
  const uint32_t fo_w = (uint32_t)(r16 * 64 + ((q ^ ((r16 >> 1) & 3)) << 4));
  uint32_t fo_a[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) fo_a[j] = (uint32_t)(RT * 1024 + r16 * 256 + (((q * 4 + j) ^ (r16 & 7)) << 4));

  auto dma16 = [&](uint32_t lds_addr, uint32_t voff, const uint8_t* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
  };
  auto issue_kb = [&](int kb, int slot) {
    const uint8_t* wsb = uniform_ptr(Wp + (int64_t)kb * 64);
    const uint8_t* asb = uniform_ptr((const uint8_t*)A + (int64_t)kb * 256);
    const uint32_t l0 = mine_lds + (uint32_t)(slot * SLOT);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) dma16(l0 + rt * 1024, voff_w[rt], wsb);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma16(l0 + RT * 1024 + i * 1024, voff_a[i], asb);
  };
  // four consecutive groups (base .. base+3) of the 16 rows of every tile: lane (row r16, group q)
  auto issue_sc = [&](int base, int buf) {
    int g = base + q;
    g = g < groups ? g : groups - 1;
    const uint32_t l0 = mine_lds + (uint32_t)(2 * SLOT + buf * SC);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const uint64_t e2 = ((uint64_t)row_g[rt] + (uint64_t)g) * 2u;
      if (has_s) {
        const uint64_t a = ((uint64_t)(uintptr_t)scales + e2) & ~(uint64_t)3;
        asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, off" ::"s"(l0 + (rt * 2 + 0) * 256), "v"(a) : "memory");
      }
      if (has_z) {
        const uint64_t a = ((uint64_t)(uintptr_t)zeros + e2) & ~(uint64_t)3;
        asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, off" ::"s"(l0 + (rt * 2 + 1) * 256), "v"(a) : "memory");
      }
    }
  };
  auto sc_base = [&](int kb) { return ((kb << 7) >> gshift) & ~3; };
  auto new_period = [&](int kb) { return NS > 0 && (kb == kb0 || sc_base(kb) != sc_base(kb - 1)); };
  auto sc_buf = [&](int kb) { return (sc_base(kb) >> 2) & 1; };

  typename Mma::acc_t acc[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) acc[rt] = typename Mma::acc_t{0, 0, 0, 0};

  if (nkb > 0) {
    if (new_period(kb0)) issue_sc(sc_base(kb0), sc_buf(kb0));
    issue_kb(kb0, 0);
    if (nkb > 1) {
      if (new_period(kb0 + 1)) issue_sc(sc_base(kb0 + 1), sc_buf(kb0 + 1));
      issue_kb(kb0 + 1, 1);
    }
  }
  for (int i = 0; i < nkb; ++i) {
    const int kb = kb0 + i;
    // everything issued for this k-block has landed once only the next k-block's loads are outstanding
    if (i + 1 < nkb) {
      if (new_period(kb + 1)) {
        if (NS == 1 * RT) {
          if (RT == 1) asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        } else {
          if (RT == 1) asm volatile("s_waitcnt vmcnt(7)" ::: "memory"); else asm volatile("s_waitcnt vmcnt(10)" ::: "memory");
        }
      } else {
        if (RT == 1) asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); else asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
      }
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    const uint8_t* slot = mine + (i & 1) * SLOT;
    uint4_t wf[RT], af[4];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) wf[rt] = *(const uint4_t*)(slot + rt * 1024 + fo_w);
#pragma unroll
    for (int j = 0; j < 4; ++j) af[j] = *(const uint4_t*)(slot + fo_a[j]);
    T sv[RT], zv[RT];
    {
      const int g = ((kb << 7) + (q << 5)) >> gshift;
      const int rel = g - sc_base(kb);
      const uint8_t* sc = mine + 2 * SLOT + sc_buf(kb) * SC + (r16 + 16 * rel) * 4;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const uint32_t sh = (((uint32_t)row_g[rt] + (uint32_t)g) & 1u) * 16u;
        const uint32_t sa = (uint32_t)(((uintptr_t)scales >> 1) & 1), za = (uint32_t)(((uintptr_t)zeros >> 1) & 1);
        sv[rt] = one;
        zv[rt] = zs;
        if (has_s) {
          const uint32_t dw = *(const uint32_t*)(sc + (rt * 2 + 0) * 256);
          sv[rt] = bitcast<T>((uint16_t)(dw >> (sh ^ (sa * 16u))));
        }
        if (has_z) {
          const uint32_t dw = *(const uint32_t*)(sc + (rt * 2 + 1) * 256);
          zv[rt] = bitcast<T>((uint16_t)(dw >> (sh ^ (za * 16u))));
        }
      }
    }
    // the slot may be overwritten once its contents are in registers
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (i + 2 < nkb) {
      if (new_period(kb + 2)) issue_sc(sc_base(kb + 2), sc_buf(kb + 2));
      issue_kb(kb + 2, i & 1);
    }
    // Zero points that are small integers in every lane (the usual case) fold exactly into the unpack
    // bias, which saves a quarter of the conversion arithmetic; decided per wavefront and k-block.
    bool fold = FOLD;
    if (!FOLD) {
      bool ok = true;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const float zf = to_float(zv[rt]);
        ok = ok && zf == __builtin_rintf(zf) && zf >= -256.0f && zf <= 256.0f;
      }
      fold = __builtin_amdgcn_ballot_w64(ok) == ~0ull;
    }
    if (fold) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const Expand8<T, true> ex(sv[rt], zv[rt], mg);
        const uint32_t w[4] = {wf[rt].x, wf[rt].y, wf[rt].z, wf[rt].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[rt] = Mma::mma(ex(w[j]), af[j], acc[rt]);
      }
    } else {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const Expand8<T, false> ex(sv[rt], zv[rt], mg);
        const uint32_t w[4] = {wf[rt].x, wf[rt].y, wf[rt].z, wf[rt].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[rt] = Mma::mma(ex(w[j]), af[j], acc[rt]);
      }
    }
  }

  // add the partial tiles of the wavefronts (the private regions are dead now)
  __syncthreads();
  float4_t* const red = (float4_t*)smem;  // [waves][RT][64 lanes]
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) red[(wave * RT + rt) * 64 + lane] = acc[rt];
  __syncthreads();
  for (int item = threadIdx.x; item < RT * 64; item += blockDim.x) {
    float4_t sum = red[item];
    for (int w = 1; w < waves; ++w) {
      const float4_t v = red[w * (RT * 64) + item];
      sum[0] += v[0];
      sum[1] += v[1];
      sum[2] += v[2];
      sum[3] += v[3];
    }
    const int rt = item >> 6, l = item & 63;
    const int m = l & 15;
    const int n = n_base + rt * 16 + 4 * (l >> 4);
    if (m >= M || n >= N) continue;
    const int64_t idx = (int64_t)m * N + n;
    if (n + 3 < N && (N & 3) == 0) {
      if (out_dtype == TLQ_F32) {
        *(float4_t*)((float*)C + idx) = sum;
      } else if (out_dtype == TLQ_F16) {
        half_t h[4] = {(half_t)sum[0], (half_t)sum[1], (half_t)sum[2], (half_t)sum[3]};
        *(uint2_t*)((half_t*)C + idx) = bitcast<uint2_t>(h);
      } else {
        uint2_t o;
        o.x = pack_bf16x2(sum[0], sum[1]);
        o.y = pack_bf16x2(sum[2], sum[3]);
        *(uint2_t*)((uint16_t*)C + idx) = o;
      }
    } else {
      for (int i = 0; i < 4 && n + i < N; ++i) store_out(C, idx + i, sum[i], out_dtype);
    }
  }
}

static thread_local int g_skinny_waves = 0, g_skinny_rt = 0;  // tuning overrides (0 = automatic)

template <typename T, bool FOLD, int RT, int MT>
static int launch_skinny(const W4Args& a, int waves) {
  auto kern = w4a16_skinny_kernel<T, FOLD, RT, MT>;
  const int blocks = (int)ceil_div(a.N, 16 * RT);
  const size_t lds = (size_t)waves * RT * MT * 64 * sizeof(float4_t);
  kern<<<blocks, waves * 64, lds, a.st>>>((const T*)a.A, (const uint8_t*)a.Wp, (const T*)a.scales, (const T*)a.zeros, a.C,
                                          (int)a.M, (int)a.N, (int)a.K, (int)a.group, a.zero_scalar, a.out_dtype);
  return check_launch("tlq_gemm_w4a16(skinny)", "w4a16_skinny_kernel") ? 0 : 1;
}

template <typename T, bool FOLD, int RT>
static int launch_skinny_lds(const W4Args& a, int waves, int gshift) {
  auto kern = w4a16_skinny_lds_kernel<T, FOLD, RT>;
  constexpr int WAVE_LDS = 2 * (RT * 1024 + 4096) + 2 * (RT * 2 * 256);
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) {
      set_error("tlq_gemm_w4a16(skinny): cannot reserve LDS: %s", hipGetErrorString(e));
      return 1;
    }
    attr_set = true;
  }
  const int blocks = (int)ceil_div(a.N, 16 * RT);
  kern<<<blocks, waves * 64, (size_t)waves * WAVE_LDS, a.st>>>((const T*)a.A, (const uint8_t*)a.Wp, (const T*)a.scales,
                                                                (const T*)a.zeros, a.C, (int)a.M, (int)a.N, (int)a.K,
                                                                gshift, a.zero_scalar, a.out_dtype);
  return check_launch("tlq_gemm_w4a16(skinny)", "w4a16_skinny_lds_kernel") ? 0 : 1;
}

static thread_local int g_skinny_lds = -1;  // tuning override: 0 = never, 1 = whenever possible, -1 = automatic

template <typename T, bool FOLD>
static int dispatch_skinny(const W4Args& a) {
  const int64_t row_tiles = ceil_div(a.N, 16);
  const int KB = (int)(a.K / 128);
  // M <= 16 and a power-of-two group: operands staged through wavefront-private LDS
  const bool pow2 = (a.group & (a.group - 1)) == 0;
  // (the scale / zero gathers read aligned dwords: the tensors must start and end on a dword boundary)
  const bool sz_ok = (((uintptr_t)a.scales | (uintptr_t)a.zeros) & 3) == 0 && ((a.N * (a.K / a.group)) & 1) == 0;
  if (a.M <= 16 && pow2 && sz_ok && g_skinny_lds != 0) {
    int gshift = 0;
    while (((int64_t)1 << gshift) < a.group) ++gshift;
    const int rt = g_skinny_rt ? g_skinny_rt : (row_tiles >= 512 ? 2 : 1);
    // small work-groups while there are plenty of them (two or more fit on a CU), larger ones to split K further
    int waves = g_skinny_waves ? g_skinny_waves : (row_tiles / rt >= 400 ? 4 : 8);
    const int max_waves = rt == 2 ? 11 : 14;  // 160 KB of LDS
    if (waves > max_waves) waves = max_waves;
    if (waves > KB) waves = KB;
    if (rt == 2) return launch_skinny_lds<T, FOLD, 2>(a, waves, gshift);
    return launch_skinny_lds<T, FOLD, 1>(a, waves, gshift);
  }
  // enough wavefronts to keep every CU streaming: about 24 per CU over the whole grid, at least two k-blocks each
  // two row tiles per wavefront halve the activation loads per weight; worth it once there are plenty of rows
  int rt = g_skinny_rt ? g_skinny_rt : (row_tiles >= 512 ? 2 : 1);
  int waves = g_skinny_waves;
  if (!waves) {
    static int cus = 0;  // cached: one attribute query per process
    if (cus == 0) {
      int dev = 0;
      if (hipGetDevice(&dev) != hipSuccess ||
          hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        cus = 256;
    }
    const int64_t want = (int64_t)cus * 24;
    waves = 1;
    while (waves < 16 && row_tiles / rt * waves < want && KB / (waves * 2) >= 2) waves *= 2;
  }
  if (waves > KB) waves = KB < 1 ? 1 : KB;
  const int mt = a.M <= 16 ? 1 : (a.M <= 32 ? 2 : 4);
  const int max_waves = mt >= 4 ? 8 : 16;  // four activation tiles need 256 registers per lane
  if (waves > max_waves) waves = max_waves;
#define TLQ_SK(RTT, MTT) return launch_skinny<T, FOLD, RTT, MTT>(a, waves)
  if (rt == 2) {
    if (mt == 1) TLQ_SK(2, 1);
    if (mt == 2) TLQ_SK(2, 2);
    TLQ_SK(2, 4);
  }
  if (mt == 1) TLQ_SK(1, 1);
  if (mt == 2) TLQ_SK(1, 2);
  TLQ_SK(1, 4);
#undef TLQ_SK
}

int gemm_w4a16_skinny(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t N,
                      int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, hipStream_t st) {
  const bool fold = zeros == nullptr && zero_scalar == (float)(int)zero_scalar && zero_scalar >= -256.0f &&
                    zero_scalar <= 256.0f;
  const W4Args a{A, Wp, scales, zeros, C, M, N, K, group, zero_scalar, out_dtype, st};
  if (in_dtype == TLQ_F16) return fold ? dispatch_skinny<half_t, true>(a) : dispatch_skinny<half_t, false>(a);
  return fold ? dispatch_skinny<bf16_t, true>(a) : dispatch_skinny<bf16_t, false>(a);
}

// C[i] = round(sum over the K slices of partial[z][i]), slices added in index order (so the result does not
// depend on which work-group finished first)
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float4_t* __restrict__ partial, void* __restrict__ C,
                                                           int64_t n4, int split, int out_dtype) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
    float4_t v = partial[i];
#pragma unroll 8  // loads of eight slices in flight (with few outputs the pass is paced by their latency); same order of adds
    for (int z = 1; z < split; ++z) v += partial[(int64_t)z * n4 + i];
    if (out_dtype == TLQ_F16) {
      half_t h[4] = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
      ((uint2_t*)C)[i] = bitcast<uint2_t>(h);
    } else if (out_dtype == TLQ_BF16) {
      ((uint2_t*)C)[i] = uint2_t{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
    } else {
      ((float4_t*)C)[i] = v;
    }
  }
}

// K slices for the tile kernel at small M, where the output tiles alone leave most of the chip idle and a
// work-group's run of stages is latency bound: aim at one to two work-groups per CU (measured best on the
// MLP shapes), slices of at least 512 values that are whole stages and whole quantisation groups.  1 = no split.
static thread_local int g_w4a16_split = 0;  // forced number of K slices for tuning runs (0 = automatic)

// fraction of the work-group places (256, or 512 for the smaller tiles) that the tile kernel fills with the K cut it would take
double w4a16_mid_fill(int64_t M, int64_t N, int64_t K, int64_t group);

int f16_split_choice(int64_t batch, int64_t M, int64_t N, int64_t K);  // gemm_f16.hip

int64_t w4a16_mid_split(int64_t M, int64_t N, int64_t K, int64_t group) {
  // Where cutting K pays (measured against the two passes on the MLP shapes): up to M = 512 always, up to
  // M = 2048 while the 256 x 256 output tiles would fill at most a quarter of the chip.
  const bool region = M > 16 && (M <= 512 || (M < 2048 && ceil_div(M, (int64_t)256) * ceil_div(N, (int64_t)256) <= 64));
  if (!region || (group & (group - 1)) != 0 || N % 4 != 0) return 1;
  // Above 512 rows the two passes are the alternative, and where their plain GEMM cuts K itself (few output tiles) they
  // are ahead of this kernel: M = 768, N = K = 5120: 66 against 89 us.
  // (Not where that GEMM would only halve rows of 13312 values or more: this kernel over four slices is 7 - 16 % ahead
  // there -- N = 4096, K = 14336, M = 1024: 146 against 163 us; N = 5120, K = 13824, M = 768: 136 against 159 us.)
  if (M > 512 && g_w4a16_split == 0) {
    const int plain_slices = f16_split_choice(1, M, N, K);
    if (plain_slices > 2 || (plain_slices == 2 && K < 13312)) return 1;
  }
  if (g_w4a16_split > 0) {
    const int64_t s = g_w4a16_split, unit0 = group > 64 ? group : 64;
    return (s <= 16 && K % s == 0 && (K / s) % unit0 == 0) ? s : 1;
  }
  const int64_t bm = M <= 32 ? 32 : (M <= 64 ? 64 : (M <= 128 ? 128 : 256)), bn = (M <= 32 || (M > 64 && M <= 128)) ? 128 : 256;
  const int64_t tiles = ceil_div(M, bm) * ceil_div(N, bn);
  const int64_t want = ceil_div((int64_t)(bm == 256 ? 256 : 512), tiles);  // one 256-row work-group fills a CU, two smaller ones do
  const int64_t unit = group > 64 ? group : 64;
  // a cut that leaves more than a third of the work-groups' places empty is not worth the partial sums (M = 1024,
  // N = 4096, K = 11008 = 2 x 43 x 128 can only be halved: 128 work-groups, 173 us against 147 us for the two passes)
  const int64_t places = bm == 256 ? 256 : 512;
  for (int64_t s = want < 16 ? want : 16; s >= 2; --s)
    if (K % s == 0 && (K / s) % unit == 0 && K / s >= 512) return (M > 256 && tiles * s * 3 < places * 2) ? 1 : s;
  return 1;
}

double w4a16_mid_fill(int64_t M, int64_t N, int64_t K, int64_t group) {
  const int64_t bm = M <= 32 ? 32 : (M <= 64 ? 64 : (M <= 128 ? 128 : 256)), bn = (M <= 32 || (M > 64 && M <= 128)) ? 128 : 256;
  const int64_t tiles = ceil_div(M, bm) * ceil_div(N, bn), places = bm == 256 ? 256 : 512;
  const double f = (double)(tiles * w4a16_mid_split(M, N, K, group)) / (double)places;
  return f > 1.0 ? 1.0 : f;
}

void launch_splitk_reduce(const float* partial, void* C, int64_t M, int64_t N, int split, int out_dtype, hipStream_t st) {
  const int64_t n4 = M * N / 4, want = ceil_div(n4, (int64_t)256);
  splitk_reduce_kernel<<<(int)(want > 65536 ? 65536 : want), 256, 0, st>>>((const float4_t*)partial, C, n4, split, out_dtype);
}

int gemm_w4a16_mfma_splitk(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M,
                           int64_t N, int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype,
                           int64_t split, float* partial, hipStream_t st) {
  const bool fold = zeros == nullptr && zero_scalar == (float)(int)zero_scalar && zero_scalar >= -256.0f &&
                    zero_scalar <= 256.0f;
  W4Args a{A, Wp, scales, zeros, C, M, N, K, group, zero_scalar, out_dtype, st};
  a.split = split;
  a.partial = partial;
  int rc;
  if (in_dtype == TLQ_F16)
    rc = fold ? dispatch_w4a16<half_t, true>(a) : dispatch_w4a16<half_t, false>(a);
  else
    rc = fold ? dispatch_w4a16<bf16_t, true>(a) : dispatch_w4a16<bf16_t, false>(a);
  if (rc) return rc;
  const int64_t n4 = M * N / 4, want = ceil_div(n4, (int64_t)256);
  splitk_reduce_kernel<<<(int)(want > 65536 ? 65536 : want), 256, 0, st>>>((const float4_t*)partial, C, n4, (int)split, out_dtype);
  return check_launch("tlq_gemm_w4a16(split-K reduce)") ? 0 : 1;
}

int gemm_w4a16_mfma(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t N,
                    int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, hipStream_t st) {
  if ((group & (group - 1)) != 0) {
    set_error("tlq_gemm_w4a16(mfma): group=%lld must be a power of two", (long long)group);
    return 1;
  }
  // An integer zero point shared by the whole matrix folds exactly into the unpack bias.
  const bool fold = zeros == nullptr && zero_scalar == (float)(int)zero_scalar && zero_scalar >= -256.0f &&
                    zero_scalar <= 256.0f;
  const W4Args a{A, Wp, scales, zeros, C, M, N, K, group, zero_scalar, out_dtype, st};
  if (in_dtype == TLQ_F16) return fold ? dispatch_w4a16<half_t, true>(a) : dispatch_w4a16<half_t, false>(a);
  return fold ? dispatch_w4a16<bf16_t, true>(a) : dispatch_w4a16<bf16_t, false>(a);
}

}  // namespace tlq

extern "C" {
// Tuning hook used by the benchmark sweeps: forces the activation-tile height (16, 32, 64,
// 128, 256) of the W4A16 MFMA kernel; 0 restores the automatic choice.
void tlq_tune_w4a16_tile(int block_m) { tlq::g_w4a16_tile = block_m; }
// K slices of the tile kernel for 16 < M < 256 when a workspace is given (2..16, must divide K into whole
// stages and groups); 0 restores the automatic choice.
void tlq_tune_w4a16_split(int slices) { tlq::g_w4a16_split = slices < 0 ? 0 : slices; }
// Wavefronts per work-group (1..16, the in-group split of K) and 16-row weight tiles per wavefront
// (1 | 2) of the skinny W4A16 kernel; 0 restores the automatic choice.
void tlq_tune_w4a16_skinny(int waves, int row_tiles) {
  tlq::g_skinny_waves = (waves < 0 || waves > 16) ? 0 : waves;
  tlq::g_skinny_rt = (row_tiles % 10 == 2) ? 2 : (row_tiles % 10 == 1 ? 1 : 0);
  tlq::g_skinny_lds = row_tiles >= 20 ? 1 : (row_tiles >= 10 ? 0 : -1);  // +10: registers only, +20: LDS staged
}
}
