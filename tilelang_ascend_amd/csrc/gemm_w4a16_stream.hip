// W4A16 for small and middle M (17 .. 512 activation rows): the weights are streamed from HBM once per block of up
// to 128 activation rows, and every global access is a full-width direct global -> LDS load into a ring deep enough
// to keep the memory pipeline busy.
//
// The tile kernel (gemm_w4a16.hip) is built for large M: it dequantises a 256-row weight tile into LDS so that many
// activation rows can share it, keeps two 128-byte stages, and with few activation rows its work-groups run a handful of
// stages each, at the pace of one memory round trip per stage (M = 64, N = 14336, K = 4096: 36 us for 29 MB of
// weights).  Here
//   * a work-group of 8 wavefronts owns 256 weight rows, 16 TM activation rows (TM = 2, 4, 6, 8) and a slice of K;
//     wavefront w owns weight rows 32 w .. 32 w + 31 (two MFMA tiles) against all activation rows, so no wavefront
//     needs another one's weights: packed weights stay private to the wavefront, are read from LDS as packed words
//     and dequantised in registers right into MFMA operands (no dequantised tile in LDS, nothing dequantised twice);
//   * a step is 128 values of K: per wavefront two 1 KB loads of packed weights (16 rows x 64 B each) and TM / 2
//     loads of the shared activation tile (16 TM rows x 256 B); steps live in a ring of D slots (D = 5, 4, 3 for
//     TM = 2, 4, 6 | 8), D - 1 steps are in flight while one is multiplied;
//   * the scales and zero points of a wavefront's rows are fetched 16 groups at a time into a private 2 KB of LDS:
//     a slice longer than 16 groups runs in windows, each of which fetches its scales and restarts the ring;
//   * one barrier per step publishes the shared activation tile and frees the slot that the next loads overwrite.
// K slices write fp32 partial tiles into a workspace, added up in slice order by splitk_reduce_kernel.
//
// k assignment inside a step: lane (row r16, k-group q) holds, at MFMA k-step ks, the eight values of packed word
// 4 q + ks of its row, i.e. k = 32 q + 8 ks .. + 7; its four words are 16 contiguous bytes (one LDS read), all in one
// quantisation group (groups are >= 32 values), and the activation operand reads the matching 16-byte chunk 4 q + ks.
// Weights whose 32-bit words went through interleave_weight (tilelang/quantize/utils.py:73-101, fp16 target) are taken
// as they are (LAYOUT 1): the word is still the same eight consecutive k, only the decode differs.
#include "expand8.h"
#include "gemm_core.h"

namespace tlq {

void launch_splitk_reduce(const float* partial, void* C, int64_t M, int64_t N, int split, int out_dtype, hipStream_t st);

namespace {

template <typename T>
struct StreamMma;
template <>
struct StreamMma<half_t> {
  typedef MmaF16 type;
};
template <>
struct StreamMma<bf16_t> {
  typedef MmaBF16 type;
};

template <int TM>
struct StreamCfg {
  static_assert(TM == 2 || TM == 4 || TM == 6 || TM == 8, "16-row activation tiles per work-group");
  // ring depth, one work-group per CU (two per CU on rings of two slots were measured no faster, and need twice
  // the K slices, i.e. twice the partial sums)
  static constexpr int D = TM == 2 ? 5 : (TM == 4 ? 4 : 3);  // (TM = 6: four slots would need 176 KB)
  static constexpr int PER_CU = 1;
  static constexpr int A_TILE = TM * 16 * 256;                // bytes of activations per step
  static constexpr int W_TILE = 8 * 2 * 1024;                 // packed weights per step: 8 wavefronts x 2 tiles x 1 KB
  static constexpr int SLOT = A_TILE + W_TILE;
  static constexpr int SZ_WAVE = 2048;                        // scales [32 rows][16 groups] + zero points [32 rows][16 groups], 2 bytes each
  static constexpr int LDS = D * SLOT + 8 * SZ_WAVE;
  static constexpr int LA = TM / 2;                           // activation load instructions per wavefront and step (4 TM / 8)
  static constexpr int L = LA + 2;                            // load instructions per wavefront and step
  static_assert(LDS * PER_CU <= 160 * 1024, "rings do not fit the CU's LDS");
  static_assert((D - 2) * L <= 63, "vmcnt range");
};
constexpr int kStreamMaxGroups = 16;
static_assert(kStreamMaxGroups * 2 == 32, "a row of the scale area is two 16-byte pieces");  // quantisation groups per window of a K slice: what the private LDS area holds

// MANY: the slice is longer than one window of the scale area (the common single-window case keeps the simpler control
// flow, which the compiler schedules 3 - 5 % better)
template <typename T, int TM, int LAYOUT, bool MANY>
__global__ __launch_bounds__(512, 2) void w4a16_stream_kernel(const T* __restrict__ A, const uint8_t* __restrict__ Wp,
                                                             const T* __restrict__ scales, const T* __restrict__ zeros,
                                                             void* __restrict__ C, float* __restrict__ partial, int M, int N, int K,
                                                             int gshift, float zero_scalar, int out_dtype, int slice_steps) {
  typedef StreamCfg<TM> Cfg;
  typedef typename StreamMma<T>::type Mma;
  typedef __attribute__((address_space(3))) uint8_t* lptr_t;
  constexpr int D = Cfg::D, LA = Cfg::LA;
  extern __shared__ __align__(16) uint8_t smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, q = lane >> 4;
  const int n0 = blockIdx.x * 256, m0 = blockIdx.z * (16 * TM);
  const int steps_total = K >> 7;
  const int step0 = blockIdx.y * slice_steps;
  const int steps = steps_total - step0 < slice_steps ? steps_total - step0 : slice_steps;
  const int groups = K >> gshift;
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lptr_t)smem);

  // ---- per-lane source offsets of the direct loads (rows past the matrices are clamped; masked at the store) ----
  uint32_t voff_w[2], voff_a[LA];
#pragma unroll
  for (int tn = 0; tn < 2; ++tn) {
    int n = n0 + wave * 32 + tn * 16 + addr::sw_row(lane);
    n = n < N ? n : N - 1;
    voff_w[tn] = (uint32_t)n * (uint32_t)(K >> 1) + (uint32_t)(addr::sw_piece(lane) * 16);
  }
#pragma unroll
  for (int j = 0; j < LA; ++j) {
    const int I = j * 8 + wave;
    int m = m0 + addr::sa_row(lane, I);
    m = m < M ? m : M - 1;
    voff_a[j] = ((uint32_t)m * (uint32_t)K) * 2u + (uint32_t)(addr::sa_chunk(lane, I) * 16);
  }
  const uint8_t* const w_base = Wp + (int64_t)step0 * 64;
  const uint8_t* const a_base = (const uint8_t*)A + (int64_t)step0 * 256;
  auto dma16 = [&](uint32_t lds_addr, uint32_t voff, const uint8_t* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
  };
  auto issue = [&](int s, int slot) {  // the loads of step s of this slice into ring slot `slot`
    const uint8_t* wsb = uniform_ptr(w_base + (int64_t)s * 64);
    const uint8_t* asb = uniform_ptr(a_base + (int64_t)s * 256);
    const uint32_t l0 = lds0 + (uint32_t)(slot * Cfg::SLOT);
#pragma unroll
    for (int j = 0; j < LA; ++j) dma16(l0 + (uint32_t)((j * 8 + wave) * 1024), voff_a[j], asb);
#pragma unroll
    for (int tn = 0; tn < 2; ++tn) dma16(l0 + (uint32_t)(Cfg::A_TILE + wave * 2048 + tn * 1024), voff_w[tn], wsb);
  };

  typename Mma::acc_t acc[2][TM];
  auto clear = [&]() {
#pragma unroll
    for (int tn = 0; tn < 2; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = typename Mma::acc_t{0, 0, 0, 0};
  };
  const NibbleMagic mg = make_nibble_magic();
  const uint32_t fo_w = (uint32_t)(Cfg::A_TILE + wave * 2048) + addr::sw_frag_off(lane);
  uint32_t fo_a[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) fo_a[ks] = addr::sa_frag_off(lane, 0, ks);
  const bool has_s = scales != nullptr, has_z = zeros != nullptr;
  const T one = from_float<T>(1.0f), zs = from_float<T>(zero_scalar);
  uint8_t* const sz = smem + D * Cfg::SLOT + wave * Cfg::SZ_WAVE;

  auto wait_step = [&](int younger) {  // this wavefront's loads of all but the `younger` most recent steps have landed
    static_assert(D <= 5, "cases below");
    if (younger >= 3)
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * Cfg::L) : "memory");
    else if (younger == 2)
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * Cfg::L) : "memory");
    else if (younger == 1)
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(1 * Cfg::L) : "memory");
    else
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  };
  auto compute = [&](int s, const uint8_t* slot, auto fold_tag) {  // s: step within the window
    constexpr bool FOLD = decltype(fold_tag)::value;
    uint4_t wq[2], af[TM][4];
#pragma unroll
    for (int tn = 0; tn < 2; ++tn) wq[tn] = *(const uint4_t*)(slot + fo_w + tn * 1024);
    const int gl = ((s << 7) + (q << 5)) >> gshift;  // group of this lane's 32 values, relative to the window
    T sv[2], zv[2];
#pragma unroll
    for (int tn = 0; tn < 2; ++tn) {
      sv[tn] = *(const T*)(sz + ((tn * 16 + r16) * kStreamMaxGroups + gl) * 2);
      zv[tn] = *(const T*)(sz + Cfg::SZ_WAVE / 2 + ((tn * 16 + r16) * kStreamMaxGroups + gl) * 2);
    }
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) af[tm][ks] = *(const uint4_t*)(slot + fo_a[ks] + tm * 16 * 256);
#pragma unroll
    for (int tn = 0; tn < 2; ++tn) {
      const Expand8<T, FOLD, LAYOUT> ex(sv[tn], zv[tn], mg);
      const uint32_t w[4] = {wq[tn].x, wq[tn].y, wq[tn].z, wq[tn].w};
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const uint4_t wop = ex(w[ks]);
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = Mma::mma(wop, af[tm][ks], acc[tn][tm]);
      }
    }
  };

  // The slice runs in windows of as many steps as the scale area holds groups for (16 groups: 4, 8, 16 steps for groups
  // of 32, 64, 128 values, more for larger groups).  Every window fetches its scales and restarts the ring: a memory
  // round trip without multiplications per window, which costs less than a further K slice (a partial tile to write
  // and add, and more work-groups than CUs).
  const int window = __builtin_amdgcn_readfirstlane(gshift >= 7 ? kStreamMaxGroups << (gshift - 7) : kStreamMaxGroups >> (7 - gshift));
  // fetch: the window's scales and zero points and its first D - 1 steps; returns whether the zero points are small integers
  auto fetch = [&](int w0, int wsteps) -> bool {
    if (w0 > 0) __syncthreads();  // every wavefront has multiplied the previous window's last steps: the slots are free

    // ---- scales / zero points of this wavefront's 32 rows for the window, and the first D - 1 steps ----
    // Area of the wavefront: [s | z][32 rows][16 groups], 2 bytes each.  A row's groups of the window are contiguous in
    // memory (32 bytes): when they are 16-byte aligned and wholly inside the row, ONE direct load per tensor fetches all
    // of them (lane l: row l / 2, half l % 2), issued ahead of the ring so that the first step's wait covers it.
    // Otherwise 2-byte gathers, four groups per instruction (they keep the address unit busy for about a cycle per lane,
    // so they go behind the weight loads, whose trip to HBM they overlap).
    // groups in this window: a slice is a whole number of groups, or a part of ONE group (large groups, K cut below the group
    // size: the plan takes slice lengths that divide the group, so the slice lies inside the group of its first step)
    const int G = ((wsteps << 7) >> gshift) > 0 ? ((wsteps << 7) >> gshift) : 1;
    const int g0 = ((step0 + w0) << 7) >> gshift;
    const bool wide = (groups & 7) == 0 && (g0 & 7) == 0 && g0 + kStreamMaxGroups <= groups &&
                      (((uintptr_t)scales | (uintptr_t)zeros) & 15) == 0;  // uniform
    bool integral = true;
    if (wide) {
      int n = n0 + wave * 32 + (lane >> 1);
      n = n < N ? n : N - 1;
      const uint32_t voff = ((uint32_t)n * (uint32_t)groups + (uint32_t)g0) * 2u + (uint32_t)((lane & 1) * 16);
      const uint32_t l0 = lds0 + (uint32_t)(D * Cfg::SLOT + wave * Cfg::SZ_WAVE);
      if (has_s) asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(l0), "v"(voff), "s"(scales) : "memory");
      if (has_z) asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(l0 + 1024u), "v"(voff), "s"(zeros) : "memory");
    }
#pragma unroll
    for (int s = 0; s < D - 1; ++s)
      if (s < wsteps) issue(w0 + s, s);
    __builtin_amdgcn_sched_barrier(0);
    if (wide) {
      // loads return in issue order: with the ring's loads still in flight the two above have landed
      if (wsteps >= D - 1)
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((D - 1) * Cfg::L) : "memory");
      else
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if (!has_s || !has_z) {  // an absent tensor is the constant 1 / the scalar zero point
        const uint32_t ws = (uint32_t)bitcast<uint16_t>(one) * 0x10001u, wz = (uint32_t)bitcast<uint16_t>(zs) * 0x10001u;
        const uint4_t cs{ws, ws, ws, ws}, cz{wz, wz, wz, wz};
        if (!has_s) *(uint4_t*)(sz + lane * 16) = cs;
        if (!has_z) *(uint4_t*)(sz + 1024 + lane * 16) = cz;
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int tn = 0; tn < 2; ++tn)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const uint4_t v = *(const uint4_t*)(sz + 1024 + ((tn * 16 + r16) * 2 + h) * 16);
          const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
          for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int e = 0; e < 2; ++e) {
              const float zf = to_float(bitcast<T>((uint16_t)(w[i] >> (16 * e))));
              integral = integral && zf == __builtin_rintf(zf) && zf >= -256.0f && zf <= 256.0f;
            }
        }
    } else {
      T pre_s[2][kStreamMaxGroups / 4], pre_z[2][kStreamMaxGroups / 4];
#pragma unroll
      for (int tn = 0; tn < 2; ++tn) {
        int n = n0 + wave * 32 + tn * 16 + r16;
        n = n < N ? n : N - 1;
#pragma unroll
        for (int i = 0; i < kStreamMaxGroups / 4; ++i) {
          pre_s[tn][i] = one;
          pre_z[tn][i] = zs;
          if (4 * i < G) {  // uniform
            int g = q + 4 * i;
            g = g < G ? g : G - 1;
            const int64_t at = (int64_t)n * groups + g0 + g;
            if (has_s) pre_s[tn][i] = scales[at];
            if (has_z) pre_z[tn][i] = zeros[at];
          }
        }
      }
#pragma unroll
      for (int tn = 0; tn < 2; ++tn)
#pragma unroll
        for (int i = 0; i < kStreamMaxGroups / 4; ++i) {
          const int g = q + 4 * i;
          const float zf = to_float(pre_z[tn][i]);
          integral = integral && zf == __builtin_rintf(zf) && zf >= -256.0f && zf <= 256.0f;
          if (g < kStreamMaxGroups) {
            *(T*)(sz + ((tn * 16 + r16) * kStreamMaxGroups + g) * 2) = pre_s[tn][i];
            *(T*)(sz + Cfg::SZ_WAVE / 2 + ((tn * 16 + r16) * kStreamMaxGroups + g) * 2) = pre_z[tn][i];
          }
        }
    }
    // small integer zero points fold exactly into the unpack bias (a quarter of the conversion arithmetic less); decided
    // once per wavefront and window
    return __builtin_amdgcn_ballot_w64(integral) == ~0ull;
  };
  auto multiply = [&](int w0, int wsteps, auto fold_tag) {
    int slot = 0;  // ring slot of step s
    for (int s = 0; s < wsteps; ++s) {
      wait_step(addr::stream_younger_steps(s, wsteps, D));
      __syncthreads();  // step s is complete for every wavefront, and everyone has multiplied step s - 1
      const int refill = slot == 0 ? D - 1 : slot - 1;  // the slot of step s - 1
      if (s + D - 1 < wsteps) issue(w0 + s + D - 1, refill);
      compute(s, smem + slot * Cfg::SLOT, fold_tag);
      slot = slot + 1 == D ? 0 : slot + 1;
    }
  };
  // One copy of the loops per dequantiser: a choice inside a loop would make the two paths meet with the accumulators
  // in different registers.
  if constexpr (!MANY) {
    const bool fold = fetch(0, steps);
    clear();
    if (fold)
      multiply(0, steps, std::true_type{});
    else
      multiply(0, steps, std::false_type{});
  } else {
    // Windows run folded while their zero points allow it; from the first window that does not, the rest of the slice
    // runs unfolded (the two give the same bits).
    clear();
    int w0 = 0;
    bool fetched = false;
    for (; w0 < steps; w0 += window) {
      const int wsteps = steps - w0 < window ? steps - w0 : window;
      fetched = true;
      if (!fetch(w0, wsteps)) break;
      fetched = false;
      multiply(w0, wsteps, std::true_type{});
    }
    for (; w0 < steps; w0 += window) {
      const int wsteps = steps - w0 < window ? steps - w0 : window;
      if (!fetched) fetch(w0, wsteps);
      fetched = false;
      multiply(w0, wsteps, std::false_type{});
    }
  }

  // lane (r16, q) holds C[m = m0 + 16 tm + r16][n = n0 + 32 wave + 16 tn + 4 q + 0..3]
  const bool split = gridDim.y > 1;
  EpiFloat::Params pe{split ? (void*)partial : C, N, (int64_t)M * N, split ? TLQ_F32 : out_dtype};
  const EpiFloat epi(pe, split ? (int)blockIdx.y : 0);
  // A wavefront's 32 fp32 outputs of a row are one 128-byte line: staged through LDS (the ring is no longer needed once
  // everyone is past the last step) they leave as whole lines; stored from the accumulators' own layout, 16 bytes per
  // lane and two instructions per line, the partial tiles of 128 rows cost 1.47 times their bytes in write traffic.
  static_assert(8 * TM * 16 * kStageBytes <= D * Cfg::SLOT, "the staging areas of the wavefronts fit the ring");
  __syncthreads();
  write_tile<EpiFloat, TM, 2>(epi, acc, smem + wave * (TM * 16 * kStageBytes), lane, m0, n0 + wave * 32, M, N);
}

}  // namespace

thread_local int g_stream_slice_steps = 0;  // tuning and tests: steps of 128 values of K per slice (0: the estimate below)

// Launch geometry: activation rows per work-group, K slices, steps per slice.  ok = the kernel applies.
struct StreamPlan {
  bool ok;
  int tm, m_blocks, n_blocks, split, slice_steps;
};
StreamPlan w4a16_stream_plan(int64_t M, int64_t N, int64_t K, int64_t group, int cus) {
  StreamPlan p{false, 0, 0, 0, 0, 0};
  if (M < 17 || M > 512 || N < 1 || K < 128 || K % 128 != 0 || group < 32 || (group & (group - 1)) != 0 || K % group != 0) return p;
  if (N % 4 != 0) return p;
  // activation rows per work-group: 32, 64, 96 or 128 -- from 65 rows on whichever needs less time for a step of all its
  // blocks (2.1 us per block of 96 rows, 2.6 us per block of 128: M = 96, 160, 192, 288 take blocks of 96)
  p.tm = M > 64 ? 8 : (M > 32 ? 4 : 2);
  if (M > 64 && (double)ceil_div(M, (int64_t)96) * 2.1 < (double)ceil_div(M, (int64_t)128) * 2.6) p.tm = 6;
  p.m_blocks = (int)ceil_div(M, (int64_t)16 * p.tm);
  p.n_blocks = (int)ceil_div(N, (int64_t)256);
  const int steps_total = (int)(K / 128);
  // a slice is a whole number of groups, or -- groups of more than 128 values, e.g. one scale per weight row -- a power-of-two
  // part of one group (K % group == 0: such slices tile K, each inside one group, whose scale every step of the slice uses)
  const int unit = group > 128 ? (int)(group / 128) : 1;
  const int window = (int)(kStreamMaxGroups * group / 128);  // steps whose groups the scale area holds; the ring restarts per window
  // K slices: the cut with the lowest estimate of rounds of work-groups (one work-group per CU) x steps per slice, plus the
  // cost of writing and adding the slices' partial tiles.  (Filling the chip once is usually that cut; but 43 x 3 blocks on
  // 256 CUs, say -- N = 11008, M = 384 -- are 258 work-groups with two slices and run a second round for two of them,
  // where three slices take two rounds of two thirds the length.)
  const double t_step = p.tm == 8 ? 2.6 : (p.tm == 6 ? 2.1 : (p.tm == 4 ? 1.65 : 1.0));  // us per step of 128 values of K
  const double t_window = 2.0;                                        // us per further window of a slice: one round trip to memory
  const double t_gather = 2.5;                                        // us per window whose scales are gathered (measured 2.5 - 3)
  const double t_slice = (double)M * (double)N * 4.0 / 3e6;           // us per slice for its partial tile, written and read back
  const int64_t blocks = (int64_t)p.n_blocks * p.m_blocks;
  double best = 0;
  int64_t best_ss = 0;
  if (g_stream_slice_steps > 0) {
    best_ss = ceil_div((int64_t)g_stream_slice_steps, (int64_t)unit) * unit;
    if (g_stream_slice_steps < unit && unit % g_stream_slice_steps == 0) best_ss = g_stream_slice_steps;  // a part of one group
    if (best_ss > steps_total) best_ss = steps_total;
  }
  for (int64_t want = 1; want <= 16 && g_stream_slice_steps <= 0; ++want) {
    int64_t ss = ceil_div((int64_t)steps_total, want);
    if (ss >= unit) {
      ss = ceil_div(ss, (int64_t)unit) * unit;
    } else {
      int64_t part = 1;
      while (part < ss) part *= 2;
      ss = part;  // (unit is a power of two: part divides it)
    }
    if (ss < 4 && steps_total >= 4) continue;  // at least four steps per work-group
    if (ss > steps_total) ss = steps_total;
    const int64_t sl = ceil_div((int64_t)steps_total, ss);
    if (sl > 16) continue;
    const int64_t rounds = ceil_div(blocks * sl, (int64_t)(cus > 0 ? cus : 256));
    const int64_t windows = ceil_div(ss, (int64_t)window);
    // slices that do not start at a multiple of eight groups gather their scales two bytes at a time
    const bool gathers = sl > 1 && (ss * 128 < group || (ss * 128 / group) % 8 != 0);
    const double t = (double)rounds * ((double)(ss + 2) * t_step + (double)(windows - 1) * t_window + (gathers ? t_gather : 0.0)) +
                     (sl > 1 ? (double)sl * t_slice : 0.0);
    if (best_ss == 0 || t < best * 0.97) best = t, best_ss = ss;
  }
  if (best_ss == 0) return p;
  p.slice_steps = (int)best_ss;
  p.split = (int)ceil_div((int64_t)steps_total, best_ss);
  if (p.split > 16) return p;  // too many partial tiles to add up: the tile kernel with longer slices takes it
  p.ok = true;
  return p;
}

template <typename T, int TM, int LAYOUT, bool MANY>
static int launch_stream(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, float* partial,
                         int64_t M, int64_t N, int64_t K, int gshift, float zero_scalar, int out_dtype, const StreamPlan& p,
                         hipStream_t st) {
  auto kern = w4a16_stream_kernel<T, TM, LAYOUT, MANY>;
  constexpr int lds_bytes = StreamCfg<TM>::LDS;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) {
      set_error("tlq_gemm_w4a16(stream): cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
      return 1;
    }
    attr_set = true;
  }
  kern<<<dim3(p.n_blocks, p.split, p.m_blocks), 512, lds_bytes, st>>>((const T*)A, (const uint8_t*)Wp, (const T*)scales,
                                                                     (const T*)zeros, C, partial, (int)M, (int)N, (int)K, gshift,
                                                                     zero_scalar, out_dtype, p.slice_steps);
  char detail[64];
  snprintf(detail, sizeof(detail), "w4a16_stream_kernel, %d activation rows per work-group", 16 * TM);
  return check_launch("tlq_gemm_w4a16(stream)", detail) ? 0 : 1;
}

// partial: fp32 [split][M][N] workspace, needed when the plan has more than one K slice
int gemm_w4a16_stream(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t N,
                      int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, int w_layout, const StreamPlan& p,
                      float* partial, hipStream_t st) {
  int gshift = 0;
  while (((int64_t)1 << gshift) < group) ++gshift;
  const bool many = (int64_t)p.slice_steps * 128 > kStreamMaxGroups * group;  // the slice holds more groups than one window of the scale area
  int rc;
#define TLQ_STREAM4(T, TM, LAY, MANY) launch_stream<T, TM, LAY, MANY>(A, Wp, scales, zeros, C, partial, M, N, K, gshift, zero_scalar, out_dtype, p, st)
#define TLQ_STREAM3(T, TM, LAY) (many ? TLQ_STREAM4(T, TM, LAY, true) : TLQ_STREAM4(T, TM, LAY, false))
#define TLQ_STREAM(T, TM) (w_layout == TLQ_W_INTERLEAVED_F16 ? TLQ_STREAM3(T, TM, 1) : TLQ_STREAM3(T, TM, 0))
  if (in_dtype == TLQ_F16)
    rc = p.tm == 2 ? TLQ_STREAM(half_t, 2) : (p.tm == 4 ? TLQ_STREAM(half_t, 4) : (p.tm == 6 ? TLQ_STREAM(half_t, 6) : TLQ_STREAM(half_t, 8)));
  else
    rc = p.tm == 2 ? TLQ_STREAM(bf16_t, 2) : (p.tm == 4 ? TLQ_STREAM(bf16_t, 4) : (p.tm == 6 ? TLQ_STREAM(bf16_t, 6) : TLQ_STREAM(bf16_t, 8)));
#undef TLQ_STREAM3
#undef TLQ_STREAM4
#undef TLQ_STREAM
  if (rc) return rc;
  if (p.split == 1) return 0;
  launch_splitk_reduce(partial, C, M, N, p.split, out_dtype, st);
  return check_launch("tlq_gemm_w4a16(stream, reduce)", "splitk_reduce_kernel") ? 0 : 1;
}

}  // namespace tlq
