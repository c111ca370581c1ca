// W4A16 for middle M (about 48 to 512 activation rows): the 256-row panel kernel's structure (gemm_w4a16_panel256.hip: four
// wavefronts, one per SIMD, each with 64 weight rows against all activation rows of the tile; packed weights copied
// global -> LDS as they are and dequantised on the MFMA operand read; loads, LDS reads and the pieces of the dequantiser
// placed one by one between the MFMAs of a step) on tiles of 64 or 128 activation rows x 256 weight rows.
//
// What differs from the 256-row kernel, and why:
//   * a step of 128 values of K is short here (64 or 128 MFMAs per wavefront), shorter than a trip to memory: the ring has
//     four (64 rows) or three (128 rows) slots, the activation tile is loaded D - 1 steps ahead and the packed weights D;
//   * nothing may force a wait for ALL outstanding loads inside a step, which register gathers of the scales would (the
//     compiler's own wait for them): scales and zero points come through LDS in windows of eight groups per row, loaded a
//     window ahead by two direct loads (the 128-row kernel's scheme, gemm_w4a16_panel.hip); the two waits of a step count
//     loads exactly (addr::panelm_wait_w / panelm_wait_a, played through on the host by the address walker);
//   * a second launch for fractional zero points would cost a fifth of such a short kernel: the kernel with a zero-point
//     tensor holds both step loops (accumulators sit in the accumulation registers either way) and runs folded while
//     the windows' zero points are small integers; from the first window that is not, the rest runs unfolded (the two
//     dequantisers give the same bits on integral zero points, so the switch does not show in the result).
// K is cut into slices of whole windows; partial tiles go to the workspace as fp32 and splitk_reduce adds them in slice
// order (deterministic).
#include <type_traits>

#include "expand8.h"
#include "gemm_core.h"

namespace tlq {

void launch_splitk_reduce(const float* partial, void* C, int64_t M, int64_t N, int split, int out_dtype, hipStream_t st);

namespace {

template <int I, int N, typename F>
__device__ __forceinline__ void static_for_m(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for_m<I + 1, N>(f);
  }
}

// The MFMA as an instruction of its own, accumulator in-out in the accumulation registers (see the 128-row kernel for why,
// and for the hazards the compiler would otherwise cover).
template <typename T>
struct PanelMMma;
template <>
struct PanelMMma<half_t> {
  typedef float4_t acc_t;
  static __device__ __forceinline__ void mma(const uint4_t& a, const uint4_t& b, acc_t& c) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};
template <>
struct PanelMMma<bf16_t> {
  typedef float4_t acc_t;
  static __device__ __forceinline__ void mma(const uint4_t& a, const uint4_t& b, acc_t& c) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};

template <int TM_>
struct PanelMCfg {
  static_assert(TM_ == 4 || TM_ == 8, "16-row activation tiles per work-group");
  static constexpr int TM = TM_, TN = addr::kPanel2TN, WAVES = 4;
  static constexpr int BM = 16 * TM, BN = WAVES * 16 * TN;
  static constexpr int D = addr::panelm_depth(TM), AR = addr::panelm_ahead(TM);
  static constexpr int SLOTS = addr::panelm_slots(TM), BARRIER = addr::panelm_barrier_slot(TM), WSLOT = addr::panelm_w_slot(TM);
  static constexpr int SLOT = (int)addr::panelm_slot_bytes(TM);
  static constexpr int SC_BUF = (int)addr::kPanelScBuf;
  static constexpr int LDS = (int)addr::panelm_lds_bytes(TM);
  static constexpr int WORD_SLOT = TM >= 8 ? TM / 2 : 0;  // slot of a phase in which the first packed word is read
  static_assert(SLOTS % AR == 0, "the operand ring closes over a step");
  static_assert(WAVES * TM * 16 * kStageBytes <= D * SLOT, "the staging areas of the wavefronts fit the ring");
};

// ZM: 0 = zero-point tensor (folded while the windows allow it, then unfolded); 1 = no tensor, integer zero point (folded);
// 2 = no tensor (unfolded)
template <typename T, int TM, int ZM>
__global__ __launch_bounds__(256, 1) void w4a16_panelm_kernel(const T* __restrict__ A, const uint8_t* __restrict__ Wp,
                                                             const T* __restrict__ scales, const T* __restrict__ zeros,
                                                             void* __restrict__ C, float* __restrict__ partial, int M, int N, int K,
                                                             int gshift, float zero_scalar, int out_dtype, int slice_steps,
                                                             int tiles_m, int tiles_n, int band_rows) {
  typedef PanelMCfg<TM> Cfg;
  typedef PanelMMma<T> Mma;
  typedef __attribute__((address_space(3))) uint8_t* lptr_t;
  typedef __attribute__((address_space(3))) const uint4_t* lds16_t;
  typedef __attribute__((address_space(3))) const uint32_t* lds4_t;
  typedef __attribute__((address_space(3))) const uint16_t* lds2_t;
  constexpr int TN = Cfg::TN, D = Cfg::D, AR = Cfg::AR, LAYOUT = 0;
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

  // ---- sources of the direct loads: the row block of every load instruction sits in the lane offset (16 weight rows or 4
  // activation rows per instruction; N % 16 == 0 and M % 4 == 0, blocks past a matrix repeat its last; a matrix spans less
  // than 4 GiB), so that a step's loads share one scalar base.
  uint32_t voff_a[TM], voff_w[TN];
#pragma unroll
  for (int j = 0; j < TM; ++j)
    voff_a[j] = (uint32_t)addr::panel2_a_block(wave, j, m0, M, K) + addr::panel_a_lane(lane, K) + addr::panel_a_chunk(lane, wave);
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) voff_w[tn] = (uint32_t)addr::panel_w_block(wave, tn, n0, N, K) + addr::panel_w_lane(lane, K);
  const uint32_t voff_sc = addr::panel_sc_voff(lane, wave, n0, N, groups);
  const uint8_t* const w_base = Wp + (int64_t)step0 * 64;
  const uint8_t* const a_base = (const uint8_t*)A + (int64_t)step0 * 256;
  auto dma16 = [&](uint32_t lds_addr, uint32_t voff, const uint8_t* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
  };
  auto clamp_step = [&](int s) { return s < steps ? s : steps - 1; };  // past the end: the last step again, into a slot nobody reads
  auto a_src = [&](int s) { return uniform_ptr(a_base + (int64_t)clamp_step(s) * 256); };
  auto w_src = [&](int s) { return uniform_ptr(w_base + (int64_t)clamp_step(s) * 64); };
  // ring_off: byte offset of the ring slot the load goes to (uniform)
  auto issue_a1 = [&](uint32_t ring_off, int j, const uint8_t* src) { dma16(lds0 + ring_off + addr::panel2_a_lds(wave, j), voff_a[j], src); };
  auto issue_w1 = [&](uint32_t ring_off, int tn, const uint8_t* src) { dma16(lds0 + ring_off + addr::panelm_w_lds(TM, wave, tn), voff_w[tn], src); };
  const bool has_s = scales != nullptr;
  constexpr bool HAS_Z = ZM == 0;
  // window w of this slice: groups g0 + 8 w .. + 7 of every row of the wavefront, into buffer w % 2
  const int g0 = (step0 << 7) >> gshift;
  auto issue_scales = [&](int w) {
    const uint32_t l0 = lds0 + addr::panelm_sc_lds(TM, wave, w & 1);
    if (has_s) dma16(l0, voff_sc, uniform_ptr((const uint8_t*)scales + (int64_t)(g0 + 8 * w) * 2));
    if (HAS_Z) dma16(l0 + 1024u, voff_sc, uniform_ptr((const uint8_t*)zeros + (int64_t)(g0 + 8 * w) * 2));
  };

  typename Mma::acc_t acc[TN][TM];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn)
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = typename Mma::acc_t{0, 0, 0, 0};
  const NibbleMagic mg = make_nibble_magic();
  const uint32_t fo_w = addr::panelm_w_lds(TM, wave, 0) + addr::sw_frag_off(lane);
  // operand read of k-step ks: logical chunk 4 q + ks = 4 q ^ ks, so the swizzled offset is that of k-step 0 ^ (16 ks)
  const uint32_t fo_a0 = addr::sa_frag_off(lane, 0, 0);
  const T one = from_float<T>(1.0f), zs = from_float<T>(zero_scalar);
  uint8_t* const sc = smem + addr::panelm_sc_lds(TM, wave, 0);

  // an absent tensor is the constant 1 / the scalar zero point: both windows are filled once and never loaded
  if (!has_s || !HAS_Z) {
    const uint32_t ws = (uint32_t)bitcast<uint16_t>(one) * 0x10001u, wz = (uint32_t)bitcast<uint16_t>(zs) * 0x10001u;
    const uint4_t cs{ws, ws, ws, ws}, cz{wz, wz, wz, wz};
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      if (!has_s) *(uint4_t*)(sc + b * Cfg::SC_BUF + lane * 16) = cs;
      if (!HAS_Z) *(uint4_t*)(sc + b * Cfg::SC_BUF + 1024 + lane * 16) = cz;
    }
  }
  // steps per window of eight groups
  const int window = __builtin_amdgcn_readfirstlane(gshift >= 7 ? 8 << (gshift - 7) : 8 >> (7 - gshift));
  const int nwin = (steps + window - 1) / window;

  // are the zero points of window w (all 64 rows of the wavefront) small integers?
  auto window_integral = [&](int w) -> bool {
    const uint4_t v = *(const uint4_t*)(sc + (w & 1) * Cfg::SC_BUF + 1024 + lane * 16);
    const uint32_t x[4] = {v.x, v.y, v.z, v.w};
    uint32_t fract_bits = 0;
    float max_abs = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const float zf = to_float(bitcast<T>((uint16_t)(x[i] >> (16 * e))));
        fract_bits |= bitcast<uint32_t>(__builtin_amdgcn_fractf(zf));
        max_abs = __builtin_fmaxf(max_abs, __builtin_fabsf(zf));
      }
    return __builtin_amdgcn_ballot_w64(fract_bits == 0 && max_abs <= 256.0f) == ~0ull;
  };

  // ---- state of the pipeline that runs across steps
  uint4_t wop[2][TN];  // expanded weight operands: [k-step parity][tn]
  uint32_t ww[2][TN];  // packed words: [k-step parity][tn]
  uint4_t af[AR];      // activation operands in flight
  T sv_raw[TN], zv_raw[TN];
  // LDS addresses of this lane's reads in the ring slot of the current step (activation operands per k-step, packed
  // words) and of the next step; scale reads go by the window buffer
  int cur = 0;  // ring slot of step s
  auto ring_off = [&](int slot) -> uint32_t { return (uint32_t)slot * (uint32_t)Cfg::SLOT; };
  auto next_slot = [&](int slot) { return slot + 1 == D ? 0 : slot + 1; };
  auto prev_slot = [&](int slot) { return slot == 0 ? D - 1 : slot - 1; };
  uint32_t a_k[4], a_nxt, w_cur, w_nxt;
  auto set_read_addresses = [&](int slot) {
    const uint32_t o = ring_off(slot), on = ring_off(next_slot(slot));
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) a_k[ks] = lds0 + o + (fo_a0 ^ (uint32_t)(ks << 4));
    a_nxt = lds0 + on + fo_a0;
    w_cur = lds0 + o + fo_w;
    w_nxt = lds0 + on + fo_w;
  };
  // (ordinary LDS loads, so that the compiler counts them in its waits; each takes its address from a register that an
  // empty volatile statement "rewrites" behind the MFMA it follows, which keeps the read there)
  auto lds_read16 = [&](uint32_t& base, uint32_t imm) {
    asm volatile("" : "+v"(base));
    return *(lds16_t)(uintptr_t)(base + imm);
  };
  auto read_word = [&](uint32_t& base, int word, int tn) {
    asm volatile("" : "+v"(base));
    return *(lds4_t)(uintptr_t)(base + (uint32_t)(word * 4 + tn * 1024));
  };
  // scales of step s (of the slice): window s / window, group of this lane's 32 values inside it
  uint32_t sc_lane = lds0 + addr::panelm_sc_lds(TM, wave, 0) + addr::panel_sc_off(r16, 0);
  auto read_scales = [&](int w_buf, int step_in_window) {
    const int gl = ((step_in_window << 7) + (q << 5)) >> gshift;
    uint32_t base = sc_lane + (uint32_t)(w_buf * Cfg::SC_BUF) + (uint32_t)(gl * 2);
    asm volatile("" : "+v"(base));
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      sv_raw[tn] = bitcast<T>(*(lds2_t)(uintptr_t)(base + (uint32_t)(tn * 256)));
      zv_raw[tn] = bitcast<T>(*(lds2_t)(uintptr_t)(base + (uint32_t)(1024 + tn * 256)));
    }
  };

  // One pass over steps [s_begin, s_end) with one dequantiser.  On entry the ring, the loads in flight and the operand
  // ring af are as the previous pass (or the prologue) left them; words, scales and the first k-step's operands of step
  // s_begin are (re)made here, because the previous pass may have made them with the other dequantiser.
  // win / win_pos: window of step s and s's place in it.  Returns at s_end, or earlier (with the step it stopped in front
  // of) when `stop_on_fraction` and the zero points of the NEXT window are not small integers.
  int win = 0, win_pos = 0;
  auto run_steps = [&](int s_begin, int s_end, auto fold_tag, bool stop_on_fraction) -> int {
    constexpr bool FOLD = decltype(fold_tag)::value;
    typedef Expand8<T, FOLD, LAYOUT> Ex;
    Ex exs[TN];
    auto expand_piece = [&](int part, int ks, int i, typename Ex::Pieces& st) {
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
    {
      // words 0 and 1, scales and the expanded first k-step of step s_begin
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) ww[0][tn] = read_word(w_cur, 0, tn), ww[1][tn] = read_word(w_cur, 1, tn);
      read_scales(win & 1, win_pos);
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) exs[tn] = Ex(sv_raw[tn], zv_raw[tn], mg);
      typename Ex::Pieces st;
#pragma unroll
      for (int part = 0; part < 2 * TN; ++part)
#pragma unroll
        for (int i = 0; i < 4; ++i) expand_piece(part, 0, i, st);
    }
    int s = s_begin;
    for (; s < s_end; ++s) {
      const bool win_start = win_pos == 0;
      // step s + 1: its window and place
      int nwin_pos = win_pos + 1, nwin_idx = win;
      if (nwin_pos == window) nwin_pos = 0, nwin_idx = win + 1;
      if constexpr (ZM == 0) {
        // the next window landed during this one: before its first scales are read (phase 2 of this window's last step),
        // know whether the folded dequantiser may go on
        if (stop_on_fraction && nwin_pos == 0 && nwin_idx < nwin && !window_integral(nwin_idx)) break;
      }
      const uint8_t* const asrc = a_src(s + D - 1);
      const uint8_t* const wsrc = w_src(s + D);
      const uint32_t a_ring = ring_off(prev_slot(cur)), w_ring = ring_off(cur);
      typename Ex::Pieces st;
      __builtin_amdgcn_sched_barrier(0);
      // (the slots as separate instantiations: every condition below is a compile-time constant of the slot)
      static_for_m<0, Cfg::SLOTS>([&](auto tc_) {
        constexpr int t = decltype(tc_)::value, ks = t / TM, tm = t % TM, j = t % AR;
        if constexpr (t == 2 * TM) {
          asm volatile("s_waitcnt vmcnt(%0)" ::"n"(addr::panelm_wait_w(TM)) : "memory");  // the packed weights of step s + 1
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
        if constexpr (t == Cfg::BARRIER) {
          asm volatile("s_waitcnt vmcnt(%0)" ::"n"(addr::panelm_wait_a(TM)) : "memory");  // the activation tile of step s + 1
          __syncthreads();
        }
        // the dequantiser constants of weight tile tn for step s + 1: between the last piece that uses the old ones (in
        // phase 2) and the first that uses the new ones (in phase 3)
        if constexpr (TM == 8) {
          if constexpr (t >= 2 * TM + 2 && t < 2 * TM + 2 + 2 * TN && (t - 2 * TM) % 2 == 0) {
            constexpr int tn = (t - 2 * TM - 2) / 2;
            exs[tn] = Ex(sv_raw[tn], zv_raw[tn], mg);
          }
        } else {
          if constexpr (t >= 2 * TM + 1 && t < 2 * TM + 1 + TN) {
            constexpr int tn = t - 2 * TM - 1;
            exs[tn] = Ex(sv_raw[tn], zv_raw[tn], mg);
          }
        }
        static_for_m<0, TN>([&](auto tnc) {
          constexpr int tn = decltype(tnc)::value, m = tm * TN + tn;  // MFMA m of the phase
          Mma::mma(wop[ks & 1][tn], af[j], acc[tn][tm]);
          // the 32 pieces of k-step ks + 1 (k-step 4 = k-step 0 of step s + 1) over the phase's 4 TM MFMAs
          if constexpr (TM == 8) {
            expand_piece(m >> 2, ks + 1, m & 3, st);
          } else {
            expand_piece((2 * m) >> 2, ks + 1, (2 * m) & 3, st);
            expand_piece((2 * m + 1) >> 2, ks + 1, (2 * m + 1) & 3, st);
          }
          if constexpr (tn == 1) {
            if constexpr (t < TM) issue_a1(a_ring, t, asrc);
            if constexpr (t == TM) {
              if (win_start && win + 1 < nwin) issue_scales(win + 1);  // buffer (win + 1) % 2 was last read in window win - 1
            }
            if constexpr (t >= Cfg::WSLOT && t < Cfg::WSLOT + TN) issue_w1(w_ring, t - Cfg::WSLOT, wsrc);
            // the ring entry that the slot before this one consumed takes the operand of slot t + AR - 1: of this step,
            // or one of the first of the next step, behind the barrier
            constexpr int at = t + AR - 1, jn = at % AR;
            if constexpr (at < Cfg::SLOTS)
              af[jn] = lds_read16(a_k[at / TM], (uint32_t)((at % TM) * 16 * 256));
            else
              af[jn] = lds_read16(a_nxt, (uint32_t)((at - Cfg::SLOTS) * 16 * 256));
            // the words two k-steps on (phases 2 and 3: of step s + 1), one per slot
            if constexpr (tm >= Cfg::WORD_SLOT && tm < Cfg::WORD_SLOT + TN)
              ww[ks & 1][tm - Cfg::WORD_SLOT] = read_word(ks < 2 ? w_cur : w_nxt, (ks + 2) & 3, tm - Cfg::WORD_SLOT);
            // the scales of step s + 1 (their window landed at least D - 1 steps ago)
            if constexpr (t == 2 * TM) read_scales(nwin_idx & 1, nwin_pos);
          }
          __builtin_amdgcn_sched_barrier(0);
        });
      });
      cur = next_slot(cur);
      set_read_addresses(cur);
      win = nwin_idx, win_pos = nwin_pos;
    }
    return s;
  };

  // ---- prologue: window 0, then what the steps before step 0 would have issued (the activation tiles of steps
  // 0 .. D - 2 and the packed weights of steps 0 .. D - 1), in the loop's order
  issue_scales(0);
  {
    const uint8_t* wsrc = w_src(0);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) issue_w1(ring_off(0), tn, wsrc);
  }
#pragma unroll
  for (int i = 0; i < D - 1; ++i) {
    const uint8_t *asrc = a_src(i), *wsrc = w_src(i + 1);
#pragma unroll
    for (int j = 0; j < TM; ++j) issue_a1(ring_off(i), j, asrc);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) issue_w1(ring_off(i + 1), tn, wsrc);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  set_read_addresses(0);
#pragma unroll
  for (int jj = 0; jj < AR - 1; ++jj) af[jj] = *(lds16_t)(uintptr_t)(a_k[0] + (uint32_t)(jj * 16 * 256));
  af[AR - 1] = af[0];  // (read in slot 0)

  if constexpr (ZM == 0) {
    int s = 0;
    if (window_integral(0)) s = run_steps(0, steps, std::true_type{}, true);
    if (s < steps) run_steps(s, steps, std::false_type{}, false);
  } else if constexpr (ZM == 1) {
    run_steps(0, steps, std::true_type{}, false);
  } else {
    run_steps(0, steps, std::false_type{}, false);
  }

  // lane (r16, q) holds C[m = m0 + 16 tm + r16][n = n0 + 64 wave + 16 tn + 4 q + 0..3]
  const bool split = slice_steps < steps_total;
  EpiFloat::Params pe{split ? (void*)partial : C, N, (int64_t)M * N, split ? TLQ_F32 : out_dtype};
  const EpiFloat epi(pe, split ? slice : 0);
  // (the loads issued past the last step; and the wait states between the last MFMAs, which the compiler does not know
  // for what they are, and the first instruction that reads an accumulator)
  asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  __syncthreads();  // everyone is past the last step: the ring becomes the output staging area
  write_tile<EpiFloat, TM, TN>(epi, acc, smem + wave * (TM * 16 * kStageBytes), lane, m0, n0 + wave * (16 * TN), M, N);
}

}  // namespace

thread_local int g_panelm_slice_steps = 0;  // tuning and tests: steps of 128 values of K per slice (0: the plan's own)
thread_local int g_panelm_rows = 0;         // tuning and tests: 64 or 128 activation rows per work-group (0: the plan's own)

// Launch geometry.  ok = the kernel applies.
struct PanelMPlan {
  bool ok;
  int tm, tiles_m, tiles_n, split, slice_steps;
};
PanelMPlan w4a16_panelm_plan(int64_t M, int64_t N, int64_t K, int64_t group, int cus) {
  PanelMPlan p{false, 0, 0, 0, 0, 0};
  if (M < 1 || N < 1 || K < 128 || K % 128 != 0 || group < 32 || (group & (group - 1)) != 0 || K % group != 0) return p;
  if (N % 16 != 0 || M % 4 != 0) return p;  // a direct load (16 weight rows, 4 activation rows) lies inside a matrix or outside
  if (M >= ((int64_t)1 << 30) || N >= ((int64_t)1 << 30)) return p;
  const int64_t groups = K / group;
  if (groups % 8 != 0) return p;  // whole windows of eight groups (16-byte pieces of a scale row)
  const int window = group >= 128 ? (int)(8 * (group / 128)) : (int)(8 / (128 / group));  // steps per window
  if (cus <= 0) cus = 256;
  const int steps_total = (int)(K / 128);
  // 64 rows per work-group up to 64 rows and where 128-row tiles would waste more than a quarter of their rows
  int tm = (M <= 64 || (M % 128 != 0 && M % 128 <= 64 && M < 256)) ? 4 : 8;
  if (g_panelm_rows == 64) tm = 4;
  if (g_panelm_rows == 128) tm = 8;
  // a window's loads have landed by the barrier of the (D - 1)-th step after their issue (the host play-through of the
  // schedule shows it); its zero points are looked at at the top of the window's last step: a window spans D steps or more
  if (window < addr::panelm_depth(tm)) {
    if (tm == 4 && window >= addr::panelm_depth(8)) tm = 8; else return p;
  }
  p.tm = tm;
  p.tiles_m = (int)ceil_div(M, (int64_t)(16 * tm));
  p.tiles_n = (int)ceil_div(N, (int64_t)256);
  const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
  // K slices of whole windows: the cut whose rounds of work-groups cost least, a slice priced at its steps plus a fixed
  // part (prologue, partial tile) and a slice's partial tile at its write and read
  int64_t ss = steps_total;
  if (g_panelm_slice_steps > 0) {
    ss = ceil_div((int64_t)g_panelm_slice_steps, (int64_t)window) * window;
  } else {
    const double fixed = tm == 4 ? 10.0 : 6.0;  // in steps
    double best = (double)ceil_div(tiles, (int64_t)cus) * (steps_total + fixed);
    for (int64_t want = 2; want <= 32; ++want) {
      const int64_t cand = ceil_div(ceil_div((int64_t)steps_total, want), (int64_t)window) * window;
      if (cand >= steps_total || cand < 4) continue;
      const int64_t sl = ceil_div((int64_t)steps_total, cand);
      const double step_us = tm == 4 ? 0.8 : 1.4;
      const double t = (double)ceil_div(tiles * sl, (int64_t)cus) * (double)(cand + fixed) +
                       (double)sl * (double)M * (double)N * 8.0 / 4e6 / step_us;  // (4 TB/s for the partial tiles, in steps)
      if (t < best * 0.97) best = t, ss = cand;
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

template <typename T, int TM, int ZM>
static int launch_panelm(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, float* partial, int64_t M,
                         int64_t N, int64_t K, int gshift, float zero_scalar, int out_dtype, const PanelMPlan& p, int band_rows,
                         hipStream_t st) {
  auto kern = w4a16_panelm_kernel<T, TM, ZM>;
  constexpr int lds_bytes = PanelMCfg<TM>::LDS;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) {
      set_error("tlq_gemm_w4a16(panelm): cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
      return 1;
    }
    attr_set = true;
  }
  const unsigned blocks = (unsigned)((int64_t)p.tiles_m * p.tiles_n * p.split);
  kern<<<blocks, 256, lds_bytes, st>>>((const T*)A, (const uint8_t*)Wp, (const T*)scales, (const T*)zeros, C, partial, (int)M, (int)N,
                                       (int)K, gshift, zero_scalar, out_dtype, p.slice_steps, p.tiles_m, p.tiles_n, band_rows);
  return check_launch("tlq_gemm_w4a16(panelm)", TM == 4 ? (ZM == 0 ? "w4a16_panelm_kernel, 64 activation rows per work-group, zero-point tensor"
                                                                   : "w4a16_panelm_kernel, 64 activation rows per work-group")
                                                        : (ZM == 0 ? "w4a16_panelm_kernel, 128 activation rows per work-group, zero-point tensor"
                                                                   : "w4a16_panelm_kernel, 128 activation rows per work-group"))
             ? 0
             : 1;
}

// partial: fp32 [split][M][N] workspace, needed when the plan has more than one K slice
int gemm_w4a16_panelm(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t N, int64_t K,
                      int64_t group, float zero_scalar, int in_dtype, int out_dtype, const PanelMPlan& p, float* partial, hipStream_t st) {
  int gshift = 0;
  while (((int64_t)1 << gshift) < group) ++gshift;
  const int band = g_gemm_band_rows > 0 ? g_gemm_band_rows : 4;
  const bool fold_scalar = zero_scalar == (float)(int)zero_scalar && zero_scalar >= -256.0f && zero_scalar <= 256.0f;
  int rc;
#define TLQ_PANELM3(T, TM, ZM) launch_panelm<T, TM, ZM>(A, Wp, scales, zeros, C, partial, M, N, K, gshift, zero_scalar, out_dtype, p, band, st)
#define TLQ_PANELM2(T, ZM) (p.tm == 4 ? TLQ_PANELM3(T, 4, ZM) : TLQ_PANELM3(T, 8, ZM))
#define TLQ_PANELM(ZM) (in_dtype == TLQ_F16 ? TLQ_PANELM2(half_t, ZM) : TLQ_PANELM2(bf16_t, ZM))
  if (zeros != nullptr)
    rc = TLQ_PANELM(0);
  else
    rc = fold_scalar ? TLQ_PANELM(1) : TLQ_PANELM(2);
#undef TLQ_PANELM
#undef TLQ_PANELM2
#undef TLQ_PANELM3
  if (rc) return rc;
  if (p.split > 1) {
    launch_splitk_reduce(partial, C, M, N, p.split, out_dtype, st);
    return check_launch("tlq_gemm_w4a16(panelm, reduce)", "splitk_reduce_kernel") ? 0 : 1;
  }
  return 0;
}

}  // namespace tlq
