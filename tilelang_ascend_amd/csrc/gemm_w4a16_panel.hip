// W4A16 for large M (prefill): one launch, packed weights copied global -> LDS as they are and dequantised on the
// operand read, no dequantised matrix in memory and no dequantised tile in LDS.
//
// The reference's large-M form is unpack-then-GEMM (examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:176-223:
// the whole weight matrix is unpacked into a workspace, then T.gemm_v0 runs on it).  Fused here:
//   * a work-group of 8 wavefronts owns 128 activation rows x 512 weight rows; wavefront w owns weight rows
//     64 w .. 64 w + 63 (four MFMA tiles) against all 128 activation rows (eight MFMA tiles): nobody else needs its
//     weights, so they stay private to the wavefront and every weight is dequantised exactly once per 128 activation
//     rows.  Per 128 values of K the work-group pulls 32 KB of activations and 32 KB of packed weights through the
//     L2 -> LDS path, half of what a 256 x 256 tile of 16-bit operands needs, and the operand reads move 18 KB per
//     wavefront and 128 MFMAs (the 16-bit kernel: 24 KB);
//   * a step is 128 values of K, two ring slots of 64 KB; every global access is a full-width direct global -> LDS load
//     (eight per wavefront and step), one barrier per step publishes the shared activation tile; the wavefront's own
//     weights are requested two steps ahead, so that the expansion of a step's first words can run under the MFMAs of
//     the step before (the step loop is software-pipelined inside the wavefront, see below);
//   * scales and zero points travel in windows of eight quantisation groups (one 16-byte piece per weight row and
//     tensor) into a private, double-buffered 4 KB per wavefront: the next window is requested at the first step of the
//     current one, so the ring never stops;
//   * work-groups are numbered so that the 32 resident on one XCD form a block of tiles that share activation and weight
//     panels in that XCD's L2; K slices (few tiles, long rows) write fp32 partial tiles that splitk_reduce_kernel adds.
// The k assignment inside a step, the LDS layouts of both tiles and their swizzles are the streaming kernel's
// (gemm_addr.h: sw_*, sa_*).
#include <atomic>

#include "expand8.h"
#include "gemm_core.h"


namespace tlq {

void launch_splitk_reduce(const float* partial, void* C, int64_t M, int64_t N, int split, int out_dtype, hipStream_t st);

namespace {

// The MFMA as an instruction of its own with the accumulator as an in-out operand: the accumulators then stay in the
// registers they were given for the whole launch.  (With the builtin, whose result is a new value, the register
// allocator lets them wander through the file and spills lane constants inside the step loop.)  The hazards the
// compiler would otherwise cover: the operands come from vector instructions and waited-for LDS reads (none
// needed), an accumulator is written once per k-step (32 MFMAs apart), and the epilogue reads them only after a
// barrier.
template <typename T>
struct PanelMma;
template <>
struct PanelMma<half_t> {
  struct type {
    typedef float4_t acc_t;
    static __device__ __forceinline__ void mma(const uint4_t& a, const uint4_t& b, acc_t& c) {
      asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
    }
  };
};
template <>
struct PanelMma<bf16_t> {
  struct type {
    typedef float4_t acc_t;
    static __device__ __forceinline__ void mma(const uint4_t& a, const uint4_t& b, acc_t& c) {
      asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
    }
  };
};

struct PanelCfg {
  static constexpr int TM = addr::kPanelTM, TN = addr::kPanelTN;
  static constexpr int BM = 16 * TM, BN = 8 * 16 * TN;
  static constexpr int A_TILE = BM * 256;             // activations per step
  static constexpr int W_WAVE = TN * 1024;            // packed weights per wavefront and step
  static constexpr int SLOT = A_TILE + 8 * W_WAVE;
  static constexpr int SC_BUF = 2048;                 // one window: scales [64 rows][8 groups] | zero points [64 rows][8 groups]
  static constexpr int SC_WAVE = 2 * SC_BUF;
  static constexpr int LDS = 2 * SLOT + 8 * SC_WAVE;
  static constexpr int LA = A_TILE / 1024 / 8;        // activation load instructions per wavefront and step
  static_assert(LDS <= 160 * 1024, "ring and scale windows do not fit the CU's LDS");
  static_assert(SLOT == (int)addr::kPanelSlot && SC_BUF == (int)addr::kPanelScBuf, "layout shared with the host walker");
};

// Small integer zero points fold exactly into the unpack bias, which halves the dequantiser's arithmetic; other zero points
// take the two roundings of rn(rn(u - z) s) one after the other.  Which of the two applies to a zero-point TENSOR is only
// known on the device, and a kernel with two step loops (one per dequantiser) pays for the second with spills of lane
// constants inside the first.  So there is one step loop per kernel:
//   ZM 1 = no tensor, integer zero point (folded)          ZM 2 = no tensor, any zero point (unfolded)
//   ZM 0 = tensor, folded; every wavefront checks the windows of zero points it meets, and one that is not integral
//          writes `epoch` to *flag (the launch's output is then discarded)
//   ZM 3 = tensor, unfolded; launched behind ZM 0, returns at once unless *flag == epoch
// (epoch: a number the host draws per call, so the flag never needs clearing; a stale equal value only makes ZM 3 run, and
// both dequantisers give the same bits.)
template <typename T, int LAYOUT, int ZM>
__global__ __launch_bounds__(512, 1) void w4a16_panel_kernel(const T* __restrict__ A, const uint8_t* __restrict__ Wp,
                                                            const T* __restrict__ scales, const T* __restrict__ zeros,
                                                            void* __restrict__ C, float* __restrict__ partial, int M, int N, int K,
                                                            int gshift, float zero_scalar, int out_dtype, int slice_steps,
                                                            int tiles_m, int tiles_n, int band_rows, uint32_t* __restrict__ flag,
                                                            uint32_t epoch) {
  typedef PanelCfg Cfg;
  if constexpr (ZM == 3) {
    if (__builtin_nontemporal_load(flag) != epoch) return;  // (uniform: every wavefront of the launch takes the same way)
  }
  typedef typename PanelMma<T>::type Mma;
  typedef __attribute__((address_space(3))) uint8_t* lptr_t;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, LA = Cfg::LA;
  extern __shared__ __align__(16) uint8_t smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, q = lane >> 4;
  const TileCoord tc = tile_of_block<Cfg::BM, Cfg::BN>(tiles_m, tiles_n, band_rows);  // batch = K slice
  const int m0 = tc.m0, n0 = tc.n0, slice = tc.batch;
  const int steps_total = K >> 7;
  const int step0 = slice * slice_steps;
  const int steps = steps_total - step0 < slice_steps ? steps_total - step0 : slice_steps;
  const int groups = K >> gshift;
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lptr_t)smem);

  // ---- source addresses of the direct loads: one lane offset per operand, the row block of an instruction in the
  // scalar base.  An instruction covers 16 weight rows or 4 activation rows; N is a multiple of 16 and M of 4, so an
  // instruction lies wholly inside the matrix or wholly outside, and the outside ones repeat the last block (their
  // outputs are masked at the store).
  const uint32_t voff_w = addr::panel_w_lane(lane, K), voff_a = addr::panel_a_lane(lane, K) + addr::panel_a_chunk(lane, wave);
  const uint32_t voff_sc = addr::panel_sc_voff(lane, wave, n0, N, groups);
  const uint8_t* const w_base = Wp + (int64_t)step0 * 64;
  const uint8_t* const a_base = (const uint8_t*)A + (int64_t)step0 * 256;
  auto dma16 = [&](uint32_t lds_addr, uint32_t voff, const uint8_t* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
  };
  // the loads of step s of this slice into ring slot s % 2: the shared activation tile one step ahead of its use, the
  // wavefront's own packed weights two steps ahead (their slot is free once the words of step s - 2 have been read)
  auto issue_a = [&](int s) {
    const uint32_t l0 = lds0 + (uint32_t)((s & 1) * Cfg::SLOT);
#pragma unroll
    for (int j = 0; j < LA; ++j)
      dma16(l0 + addr::panel_a_lds(wave, j), voff_a, uniform_ptr(a_base + (int64_t)s * 256 + addr::panel_a_block(wave, j, m0, M, K)));
  };
  auto issue_w = [&](int s) {
    const uint32_t l0 = lds0 + (uint32_t)((s & 1) * Cfg::SLOT);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
      dma16(l0 + addr::panel_w_lds(wave, tn), voff_w, uniform_ptr(w_base + (int64_t)s * 64 + addr::panel_w_block(wave, tn, n0, N, K)));
  };
  const bool has_s = scales != nullptr, has_z = zeros != nullptr;
  // window w of this slice: groups g0 + 8 w .. + 7 of every row of the wavefront, into buffer w % 2
  const int g0 = (step0 << 7) >> gshift;
  auto issue_scales = [&](int w) {
    const uint32_t l0 = lds0 + addr::panel_sc_lds(wave, w & 1);
    if (has_s) dma16(l0, voff_sc, uniform_ptr((const uint8_t*)scales + (int64_t)(g0 + 8 * w) * 2));
    if (has_z) dma16(l0 + 1024u, voff_sc, uniform_ptr((const uint8_t*)zeros + (int64_t)(g0 + 8 * w) * 2));
  };

  typename Mma::acc_t acc[TN][TM];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn)
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = typename Mma::acc_t{0, 0, 0, 0};
  const NibbleMagic mg = make_nibble_magic();
  const uint32_t fo_w = addr::panel_w_lds(wave, 0) + addr::sw_frag_off(lane);
  // operand read of k-step ks: logical chunk 4 q + ks = 4 q ^ ks, so the swizzled offset is that of k-step 0 ^ (16 ks)
  const uint32_t fo_a0 = addr::sa_frag_off(lane, 0, 0);
  auto fo_a = [&](int ks) -> uint32_t { return fo_a0 ^ (uint32_t)(ks << 4); };
  const T one = from_float<T>(1.0f), zs = from_float<T>(zero_scalar);
  uint8_t* const sc = smem + addr::panel_sc_lds(wave, 0);

  // an absent tensor is the constant 1 / the scalar zero point: both windows are filled once and never loaded
  if (!has_s || !has_z) {
    const uint32_t ws = (uint32_t)bitcast<uint16_t>(one) * 0x10001u, wz = (uint32_t)bitcast<uint16_t>(zs) * 0x10001u;
    const uint4_t cs{ws, ws, ws, ws}, cz{wz, wz, wz, wz};
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      if (!has_s) *(uint4_t*)(sc + b * Cfg::SC_BUF + lane * 16) = cs;
      if (!has_z) *(uint4_t*)(sc + b * Cfg::SC_BUF + 1024 + lane * 16) = cz;
    }
  }

  // steps per window of eight groups
  const int window = __builtin_amdgcn_readfirstlane(gshift >= 7 ? 8 << (gshift - 7) : 8 >> (7 - gshift));
  const int nwin = (steps + window - 1) / window;

  // ---- the step loop, software-pipelined inside the wavefront --------------------------------------------------
  // A step is four k-steps (phases) of 32 MFMAs: activation tile tm outermost, the four weight operands of the k-step
  // stay in registers.  While the MFMAs of phase ks run, the wavefront
  //   (a) reads the activation operands four tiles ahead into a ring of four (slot by slot),
  //   (b) expands the packed words of the NEXT k-step into the other operand set, one half word per slot,
  //   (c) reads the packed words of the k-step after that (one dword per weight tile, two rotating sets).
  // Packed words and scales are private to the wavefront and their loads run two steps ahead, so the pipeline runs
  // straight through the step boundary: phase 2 reads the first words and the scales of step s + 1, phase 3 expands
  // them.  Only the first four activation operands of a step wait for the barrier that publishes the shared tile.
  // A slot is written as "MFMA, a piece of two or three vector instructions" four times, then its LDS reads, each quarter
  // closed by a scheduling barrier: the expansion issues in the shadow of the matrix pipeline instead of ahead of it
  // (an in-order wavefront overlaps nothing with four MFMAs issued back to back), and the compiler cannot pull the
  // reads of later slots forward (registers: 128 accumulators + 32 operands + 16 operands in flight + 8 words + 12
  // dequantiser constants + addresses: about 220 of 256).
  uint4_t wop[2][TN];   // expanded weight operands: [k-step parity][tn]
  uint32_t ww[2][TN];   // packed words: [k-step parity][tn]
  auto read_words = [&](int s, int ks) {  // word ks of step s of every weight tile, into set ks % 2
    const uint8_t* slot = smem + (s & 1) * Cfg::SLOT;
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) ww[ks & 1][tn] = *(const uint32_t*)(slot + fo_w + tn * 1024 + ks * 4);
  };
  T sv_raw[TN], zv_raw[TN];
  auto read_scales = [&](int s) {
    const int w = s / window, sw = s - w * window;
    const uint8_t* scb = sc + (w & 1) * Cfg::SC_BUF;
    const int gl = ((sw << 7) + (q << 5)) >> gshift;  // group of this lane's 32 values, relative to the window
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      sv_raw[tn] = *(const T*)(scb + addr::panel_sc_off(tn * 16 + r16, gl));
      zv_raw[tn] = *(const T*)(scb + 1024 + addr::panel_sc_off(tn * 16 + r16, gl));
    }
  };
  auto make_expanders = [&](auto& exs) {
    typedef std::remove_reference_t<decltype(exs[0])> Ex;
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) exs[tn] = Ex(sv_raw[tn], zv_raw[tn], mg);
  };
  // expansion work comes in eight parts per k-step, one per slot: part 2 tn + p is half p of the word of weight tile tn,
  // itself cut into four pieces that the slot places behind its four MFMAs (dequantisers that do not split a word do
  // all of it in piece 0 of part 2 tn)
  // (The statements of a piece have no side effects and would drift: the compiler likes to issue the four MFMAs of a
  // slot back to back and the slot's expansion behind them, where an in-order wavefront cannot overlap the two.  Each
  // piece is therefore pinned between the MFMA statement it follows and the next one, see Pieces::pin.)
  auto expand_piece = [&](int part, int ks, int i, auto& exs, auto& st) {
    typedef std::remove_reference_t<decltype(exs[0])> Ex;
    const int tn = part >> 1, p = part & 1;
    uint4_t& o = wop[ks & 1][tn];
    uint32_t& w = ww[ks & 1][tn];
    if constexpr (Ex::SPLITS) {
      if (i == 0) asm volatile("" : "+v"(w)); else st.pin(i - 1);
      exs[tn].piece(st, w, p, i);
      if (i == 3) {
        st.pin(3);
        Ex::place(o, uint2_t{st.a, st.b}, p);
      }
    } else {
      if (p == 0 && i == 0) o = exs[tn](w);
    }
  };
  auto expand_part = [&](int part, int ks, auto& exs) {
    typedef std::remove_reference_t<decltype(exs[0])> Ex;
    typename Ex::Pieces st;
#pragma unroll
    for (int i = 0; i < 4; ++i) expand_piece(part, ks, i, exs, st);
  };
  // are the zero points of window w (all 64 rows of the wavefront) small integers?
  auto window_integral = [&](int w) -> bool {
    const uint4_t v = *(const uint4_t*)(sc + (w & 1) * Cfg::SC_BUF + 1024 + lane * 16);
    const uint32_t x[4] = {v.x, v.y, v.z, v.w};
    bool integral = true;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const float zf = to_float(bitcast<T>((uint16_t)(x[i] >> (16 * e))));
        integral = integral && zf == __builtin_rintf(zf) && zf >= -256.0f && zf <= 256.0f;
      }
    return __builtin_amdgcn_ballot_w64(integral) == ~0ull;
  };

  bool all_integral = true;
  // steps [s_begin, s_end) of the slice with one dequantiser.  primed: the caller's previous run (same dequantiser)
  // ended at s_begin and has left the words, scales and first operands of step s_begin in place.
  auto run_steps = [&](int s_begin, int s_end, bool primed, auto& exs) {
    if (!primed) {
      read_words(s_begin, 0);
      read_words(s_begin, 1);
      read_scales(s_begin);
      make_expanders(exs);
#pragma unroll
      for (int part = 0; part < 2 * TN; ++part) expand_part(part, 0, exs);
    }
    for (int s = s_begin; s < s_end; ++s) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();  // the activations of step s are complete for every wavefront, and everyone has multiplied step s - 1
      {
        const int w = s / window;
        if (s == w * window) {
          if (w + 1 < nwin) issue_scales(w + 1);  // buffer (w + 1) % 2 was last read in window w - 1
          if constexpr (ZM == 0) all_integral = all_integral && window_integral(w);  // (landed a window ago; window 0: before the loop)
        }
      }
      if (s + 1 < steps) issue_a(s + 1);
      const int s_w = s + 2 < steps ? s + 2 : steps - 1;  // (past the end: any step, into a slot nobody reads again)
      const uint8_t* slot = smem + (s & 1) * Cfg::SLOT;
      constexpr int AR = 4;  // activation operands in flight
      uint4_t af[AR];
#pragma unroll
      for (int j = 0; j < AR; ++j) af[j] = *(const uint4_t*)(slot + fo_a(0) + j * 16 * 256);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
          const int j = (ks * TM + tm) % AR;
          typename std::remove_reference_t<decltype(exs[0])>::Pieces st;
          if (ks == 3 && tm == 0) make_expanders(exs);
#pragma unroll
          for (int tn = 0; tn < TN; ++tn) {
            Mma::mma(wop[ks & 1][tn], af[j], acc[tn][tm]);
            expand_piece(tm, ks + 1, tn, exs, st);  // (k-step 4 = k-step 0 of step s + 1)
            if (tn == TN - 1) {
              const int ks2 = tm + AR < TM ? ks : ks + 1, tm2 = tm + AR < TM ? tm + AR : tm + AR - TM;
              if (ks2 < 4) af[j] = *(const uint4_t*)(slot + fo_a(ks2) + tm2 * 16 * 256);
              if (ks == 2 && tm == 2) read_scales(s + 1);  // (used at the start of phase 3)
              if (tm == 0) {
                // the words two k-steps on (phases 2 and 3: of step s + 1)
                if (ks < 2) read_words(s, ks + 2); else read_words(s + 1, ks - 2);
                if (ks == 2) issue_w(s_w);  // the last word of step s left its slot in phase 1
              }
            }
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      }
    }
  };
  issue_scales(0);
  issue_w(0);
  issue_a(0);
  if (steps > 1) issue_w(1);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (window w + 1 lands during window w)
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  if constexpr (ZM == 0 || ZM == 1) {
    Expand8<T, true, LAYOUT> exs_fold[TN];
    run_steps(0, steps, false, exs_fold);
    if constexpr (ZM == 0) {
      if (!all_integral && lane == 0) __hip_atomic_store(flag, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  } else {
    Expand8<T, false, LAYOUT> exs_plain[TN];
    run_steps(0, steps, false, exs_plain);
  }

  // lane (r16, q) holds C[m = m0 + 16 tm + r16][n = n0 + 64 wave + 16 tn + 4 q + 0..3]
  const bool split = slice_steps < steps_total;
  EpiFloat::Params pe{split ? (void*)partial : C, N, (int64_t)M * N, split ? TLQ_F32 : out_dtype};
  const EpiFloat epi(pe, split ? slice : 0);
  static_assert(8 * TM * 16 * kStageBytes <= 2 * Cfg::SLOT, "the staging areas of the wavefronts fit the ring");
  // (the loads issued past the last step; and the wait states between the last MFMAs, which the compiler does not know
  // for what they are, and the first vector instruction that reads an accumulator)
  asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  __syncthreads();  // everyone is past the last step: the ring becomes the output staging area
  write_tile<EpiFloat, TM, TN>(epi, acc, smem + wave * (TM * 16 * kStageBytes), lane, m0, n0 + wave * (16 * TN), M, N);
}

}  // namespace

thread_local int g_panel_slice_steps = 0;  // tuning and tests: steps of 128 values of K per slice (0: the plan's own)

// Launch geometry.  ok = the kernel applies.
struct PanelPlan {
  bool ok;
  int tiles_m, tiles_n, split, slice_steps;
};
PanelPlan w4a16_panel_plan(int64_t M, int64_t N, int64_t K, int64_t group, int cus) {
  PanelPlan p{false, 0, 0, 0, 0};
  if (M < 1 || N < 1 || K < 128 || K % 128 != 0 || group < 32 || (group & (group - 1)) != 0 || K % group != 0) return p;
  if ((K / group) % 8 != 0) return p;  // scale windows are whole 16-byte pieces of a row of the scale tensor
  if (N % 16 != 0 || M % 4 != 0) return p;  // a direct load (16 weight rows, 4 activation rows) lies inside a matrix or outside
  if (M >= ((int64_t)1 << 30) || N >= ((int64_t)1 << 30)) return p;
  p.tiles_m = (int)ceil_div(M, (int64_t)PanelCfg::BM);
  p.tiles_n = (int)ceil_div(N, (int64_t)PanelCfg::BN);
  const int steps_total = (int)(K / 128);
  const int window = (int)(group >= 128 ? 8 * (group / 128) : 8 / (128 / group));  // steps per window of eight groups
  const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
  if (cus <= 0) cus = 256;
  // K slices (whole windows): only where the tiles leave most of the machine idle; the cut that fills it best with
  // slices of at least 16 steps
  int64_t ss = steps_total;
  if (g_panel_slice_steps > 0) {
    ss = ceil_div((int64_t)g_panel_slice_steps, (int64_t)window) * window;
  } else if (tiles * 2 <= cus) {
    double best = (double)ceil_div(tiles, (int64_t)cus) * (steps_total + 8);
    for (int64_t want = 2; want <= 16; ++want) {
      int64_t cand = ceil_div(ceil_div((int64_t)steps_total, want), (int64_t)window) * window;
      if (cand < 16 || cand >= steps_total) continue;
      const int64_t sl = ceil_div((int64_t)steps_total, cand);
      const double t = (double)ceil_div(tiles * sl, (int64_t)cus) * (double)(cand + 8) + (double)sl * (double)M * (double)N * 4.0 / 3e6 / 1.5;
      if (t < best * 0.95) best = t, ss = cand;
    }
  }
  if (ss > steps_total) ss = steps_total;
  if (ss < 1) return p;
  p.slice_steps = (int)ss;
  p.split = (int)ceil_div((int64_t)steps_total, ss);
  if ((int64_t)p.split * tiles > 0x7fffffff) return p;
  p.ok = true;
  return p;
}

template <typename T, int LAYOUT, int ZM>
static int launch_panel(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, float* partial, int64_t M,
                        int64_t N, int64_t K, int gshift, float zero_scalar, int out_dtype, const PanelPlan& p, int band_rows,
                        uint32_t* flag, uint32_t epoch, hipStream_t st) {
  auto kern = w4a16_panel_kernel<T, LAYOUT, ZM>;
  constexpr int lds_bytes = PanelCfg::LDS;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) {
      set_error("tlq_gemm_w4a16(panel): cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
      return 1;
    }
    attr_set = true;
  }
  const unsigned blocks = (unsigned)((int64_t)p.tiles_m * p.tiles_n * p.split);
  kern<<<blocks, 512, lds_bytes, st>>>((const T*)A, (const uint8_t*)Wp, (const T*)scales, (const T*)zeros, C, partial, (int)M, (int)N,
                                       (int)K, gshift, zero_scalar, out_dtype, p.slice_steps, p.tiles_m, p.tiles_n, band_rows, flag, epoch);
  return check_launch("tlq_gemm_w4a16(panel)", ZM == 0 ? "w4a16_panel_kernel, zero-point tensor folded" : (ZM == 3 ? "w4a16_panel_kernel, unfolded behind the flag" : "w4a16_panel_kernel")) ? 0 : 1;
}

// partial: fp32 [split][M][N] workspace, needed when the plan has more than one K slice
// flag: one 32-bit word of device memory of the caller's (any contents), needed with a zero-point tensor
int gemm_w4a16_panel(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t N, int64_t K,
                     int64_t group, float zero_scalar, int in_dtype, int out_dtype, int w_layout, const PanelPlan& p, float* partial,
                     uint32_t* flag, hipStream_t st) {
  int gshift = 0;
  while (((int64_t)1 << gshift) < group) ++gshift;
  const int band = g_gemm_band_rows > 0 ? g_gemm_band_rows : 4;
  const bool fold_scalar = zero_scalar == (float)(int)zero_scalar && zero_scalar >= -256.0f && zero_scalar <= 256.0f;
  static std::atomic<uint32_t> epochs{0x5eed0001u};
  const uint32_t epoch = zeros != nullptr ? epochs.fetch_add(1, std::memory_order_relaxed) : 0u;
  int rc;
#define TLQ_PANEL3(T, LAY, ZM) launch_panel<T, LAY, ZM>(A, Wp, scales, zeros, C, partial, M, N, K, gshift, zero_scalar, out_dtype, p, band, flag, epoch, st)
#define TLQ_PANEL2(T, ZM) (w_layout == TLQ_W_INTERLEAVED_F16 ? TLQ_PANEL3(T, 1, ZM) : TLQ_PANEL3(T, 0, ZM))
#define TLQ_PANEL(ZM) (in_dtype == TLQ_F16 ? TLQ_PANEL2(half_t, ZM) : TLQ_PANEL2(bf16_t, ZM))
  if (zeros != nullptr) {
    rc = TLQ_PANEL(0);
    if (!rc) rc = TLQ_PANEL(3);
  } else {
    rc = fold_scalar ? TLQ_PANEL(1) : TLQ_PANEL(2);
  }
#undef TLQ_PANEL
#undef TLQ_PANEL2
#undef TLQ_PANEL3
  if (rc) return rc;
  if (p.split > 1) {
    launch_splitk_reduce(partial, C, M, N, p.split, out_dtype, st);
    return check_launch("tlq_gemm_w4a16(panel, reduce)", "splitk_reduce_kernel") ? 0 : 1;
  }
  return 0;
}

}  // namespace tlq
