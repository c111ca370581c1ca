// W4A16 for large M, 256 activation rows per work-group: the panel kernel's structure (gemm_w4a16_panel.hip: packed weights
// copied global -> LDS as they are, dequantised on the MFMA operand read, step loop software-pipelined inside the
// wavefront) on FOUR wavefronts, one per SIMD, each with the full register file.
//
// Why a second tile shape: in the 128-row kernel every weight is dequantised once per 128 activation rows and every
// activation operand read from LDS feeds four MFMAs; the dequantiser's vector instructions and the LDS reads cost power,
// and on this part the matrix pipeline's clock is set by power.  Here
//   * a work-group of 4 wavefronts owns 256 activation rows x 256 weight rows; wavefront w owns weight rows 64 w ..
//     64 w + 63 (four MFMA tiles) against all 256 activation rows (sixteen MFMA tiles): 256 accumulator registers, kept
//     in the accumulation half of the register file, and per MFMA half the dequantiser arithmetic and half the LDS
//     operand traffic of the 128-row kernel;
//   * a step is 128 values of K in two ring slots of 80 KB (activation tile [256 rows][256 B] + the four wavefronts'
//     packed weights): all of the CU's LDS.  Scales and zero points therefore do not pass through LDS: every lane
//     gathers the two values of its own weight rows for the next step straight into registers (eight 2-byte loads per
//     wavefront and step, issued ahead of the step's activation loads, waited for half a step later);
//   * one barrier per step; the waits count loads exactly (vmcnt(4) at the top of a step leaves the packed weights
//     of the step after next in flight, vmcnt(16) in the middle leaves the next activation tile), every step issues the
//     same number of loads (past the end: the last step again, into a slot nobody reads).
// The k assignment inside a step, both LDS tile layouts and their swizzles are the streaming kernel's (gemm_addr.h:
// sw_*, sa_* with sixteen activation tiles).  Zero-point tensors: the kernel holds both step loops (the accumulators sit in
// the accumulation registers either way, so two loops do not cost spills) and runs folded while the zero points of the
// step ahead are small integers; from the first step whose zero points are not, the rest runs unfolded (on integral
// zero points the two dequantisers give the same bits, so the switch does not show in the result).
#include <type_traits>

#include "expand8.h"
#include "gemm_core.h"

namespace tlq {

void launch_splitk_reduce(const float* partial, void* C, int64_t M, int64_t N, int split, int out_dtype, hipStream_t st);

namespace {

// The MFMA as an instruction of its own with the accumulator as an in-out operand in the accumulation registers (see
// the 128-row kernel for why, and for the hazards the compiler would otherwise cover).
template <typename T>
struct Panel2Mma;
template <>
struct Panel2Mma<half_t> {
  typedef float4_t acc_t;
  static __device__ __forceinline__ void mma(const uint4_t& a, const uint4_t& b, acc_t& c) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};
template <>
struct Panel2Mma<bf16_t> {
  typedef float4_t acc_t;
  static __device__ __forceinline__ void mma(const uint4_t& a, const uint4_t& b, acc_t& c) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};

template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

struct Panel2Cfg {
  static constexpr int TM = addr::kPanel2TM, TN = addr::kPanel2TN, WAVES = 4;
  static constexpr int BM = 16 * TM, BN = WAVES * 16 * TN;
  static constexpr int A_TILE = BM * 256;       // activations per step
  static constexpr int W_WAVE = TN * 1024;      // packed weights per wavefront and step
  static constexpr int SLOT = A_TILE + WAVES * W_WAVE;
  static constexpr int LDS = 2 * SLOT;
  static constexpr int LA = A_TILE / 1024 / WAVES;  // activation load instructions per wavefront and step
  static_assert(LDS <= 160 * 1024, "the ring does not fit the CU's LDS");
  static_assert(SLOT == (int)addr::kPanel2Slot && LA == 16 && TN == 4, "layout shared with the host walker; the waits below count these loads");
};

// ZM: 0 = zero-point tensor (folded while the zero points allow it, then unfolded); 1 = no tensor, integer zero point
// (folded); 2 = no tensor (unfolded)
template <typename T, int LAYOUT, int ZM>
__global__ __launch_bounds__(256, 1) void w4a16_panel256_kernel(const T* __restrict__ A, const uint8_t* __restrict__ Wp,
                                                               const T* __restrict__ scales, const T* __restrict__ zeros,
                                                               void* __restrict__ C, float* __restrict__ partial, int M, int N, int K,
                                                               int gshift, float zero_scalar, int out_dtype, int slice_steps,
                                                               int tiles_m, int tiles_n, int band_rows) {
  typedef Panel2Cfg Cfg;
  typedef Panel2Mma<T> Mma;
  typedef __attribute__((address_space(3))) uint8_t* lptr_t;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, LA = Cfg::LA;
  constexpr bool HAS_Z = ZM == 0;
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

  // ---- sources of the loads: the row block of every load instruction sits in the lane offset (16 weight rows or 4
  // activation rows per instruction; N % 16 == 0 and M % 4 == 0, blocks past a matrix repeat its last; a matrix spans less
  // than 4 GiB), so that a step's loads share one scalar base and issuing one costs two instructions -- with one
  // wavefront per SIMD nothing else hides address arithmetic.
  uint32_t voff_a[LA], voff_w[TN], voff_sc[TN];
#pragma unroll
  for (int j = 0; j < LA; ++j)
    voff_a[j] = (uint32_t)addr::panel2_a_block(wave, j, m0, M, K) + addr::panel_a_lane(lane, K) + addr::panel_a_chunk(lane, wave);
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) {
    voff_w[tn] = (uint32_t)addr::panel_w_block(wave, tn, n0, N, K) + addr::panel_w_lane(lane, K);
    voff_sc[tn] = (uint32_t)addr::panel2_sc_block(wave, tn, n0, N, groups) + addr::panel2_sc_lane(lane, groups, gshift);
  }
  const uint8_t* const w_base = Wp + (int64_t)step0 * 64;
  const uint8_t* const a_base = (const uint8_t*)A + (int64_t)step0 * 256;
  auto dma16 = [&](uint32_t lds_addr, uint32_t voff, const uint8_t* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
  };
  auto clamp_step = [&](int s) { return s < steps ? s : steps - 1; };  // past the end: the last step again
  auto a_src = [&](int s) { return uniform_ptr(a_base + (int64_t)clamp_step(s) * 256); };
  auto w_src = [&](int s) { return uniform_ptr(w_base + (int64_t)clamp_step(s) * 64); };
  auto issue_a1 = [&](int s, int j, const uint8_t* src) {  // load j (of 16) of the activation tile of step s
    dma16(lds0 + (uint32_t)((s & 1) * Cfg::SLOT) + addr::panel2_a_lds(wave, j), voff_a[j], src);
  };
  auto issue_w1 = [&](int s, int tn, const uint8_t* src) {  // load tn (of 4) of the wavefront's packed weights of step s
    dma16(lds0 + (uint32_t)((s & 1) * Cfg::SLOT) + addr::panel2_w_lds(wave, tn), voff_w[tn], src);
  };
  // Scales and zero points of a step for this lane's four weight rows (tn * 16 + r16) and its k-group: eight 2-byte
  // loads into registers.  They are ordinary loads, not statements of this file's own: a register that a load of our
  // own is still to fill must not be moved by the compiler in the meantime, and nothing can keep it from doing that
  // (seen: wrong scales in the kernels with the most vector registers in use).  The compiler's own wait stands where the
  // values are first touched (pin_scales); it knows nothing of the direct loads and therefore waits for everything
  // issued before that point, which is why no direct load is in flight there.  An absent tensor is read from the
  // packed weights instead (any valid address: the value is replaced), so that every step issues the same number of loads.
  const bool has_s = scales != nullptr;
  const uint8_t* const s_tensor = has_s ? (const uint8_t*)scales : Wp;
  const uint8_t* const z_tensor = HAS_Z ? (const uint8_t*)zeros : Wp;
  auto sc_src = [&](const uint8_t* tensor, bool present, int s) {
    return uniform_ptr(present ? tensor + addr::panel2_sc_step(step0 + clamp_step(s), gshift) : tensor);
  };
  uint32_t sv_step[TN], zv_step[TN];  // of the current step (kept for a change of dequantiser)
  uint32_t sv_raw[TN], zv_raw[TN];    // of the next step: the dequantiser constants made next
  uint32_t sv_load[TN], zv_load[TN];  // in flight
  auto issue_sc1 = [&](int i, const uint8_t* ssrc, const uint8_t* zsrc) {  // gather i (of 8)
    const int tn = i >> 1;
    // (global, not flat: a flat load counts as an LDS access too.  The waits count these loads: every value is touched
    // by pin_scales, so none is dropped, and the stand-in addresses of an absent tensor differ and are not adjacent,
    // so none is merged with another.  A volatile load would be waited for on the spot.)
    typedef __attribute__((address_space(1))) const uint16_t* global16_t;
    const uint32_t stand_in = (uint32_t)tn * 256u;  // (inside the packed weights: N >= 16 rows of K / 2 >= 64 bytes)
    if ((i & 1) == 0)
      sv_load[tn] = *(global16_t)(uintptr_t)(ssrc + (has_s ? voff_sc[tn] : stand_in));
    else
      zv_load[tn] = *(global16_t)(uintptr_t)(zsrc + (HAS_Z ? voff_sc[tn] : stand_in));
  };
  auto pin_scales = [&]() {  // the first touch of the loaded values (also of those that are replaced: their loads stay)
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      asm volatile("" : "+v"(sv_load[tn]), "+v"(zv_load[tn]));
      sv_step[tn] = sv_raw[tn], zv_step[tn] = zv_raw[tn];
      sv_raw[tn] = sv_load[tn], zv_raw[tn] = zv_load[tn];
    }
  };
  const uint32_t one_bits = (uint32_t)bitcast<uint16_t>(from_float<T>(1.0f)), zs_bits = (uint32_t)bitcast<uint16_t>(from_float<T>(zero_scalar));
  const NibbleMagic mg = make_nibble_magic();
  // are these raw zero points (one per weight tile and lane) small integers, for every lane of the wavefront?
  auto integral = [&](const uint32_t (&zb)[TN]) -> bool {
    uint32_t fract_bits = 0;  // not zero for a fraction or a NaN
    float max_abs = 0.0f;
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const float zf = to_float(bitcast<T>((uint16_t)zb[tn]));
      fract_bits |= bitcast<uint32_t>(__builtin_amdgcn_fractf(zf));
      max_abs = __builtin_fmaxf(max_abs, __builtin_fabsf(zf));
    }
    return __builtin_amdgcn_ballot_w64(fract_bits == 0 && max_abs <= 256.0f) == ~0ull;
  };

  typename Mma::acc_t acc[TN][TM];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn)
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = typename Mma::acc_t{0, 0, 0, 0};
  const uint32_t fo_w = addr::panel2_w_lds(wave, 0) + addr::sw_frag_off(lane);
  // operand read of k-step ks: logical chunk 4 q + ks = 4 q ^ ks, so the swizzled offset is that of k-step 0 ^ (16 ks)
  const uint32_t fo_a0 = addr::sa_frag_off(lane, 0, 0);
  auto fo_a = [&](int ks) -> uint32_t { return fo_a0 ^ (uint32_t)(ks << 4); };

  // ---- the step loop (see the 128-row kernel): four k-steps (phases) of 64 MFMAs, activation tile tm outermost; while
  // phase ks runs, the activation operands are read eight tiles ahead, the words of k-step ks + 1 are expanded (one piece of
  // two vector instructions behind every second MFMA), the words of k-step ks + 2 are read.
  uint4_t wop[2][TN];   // expanded weight operands: [k-step parity][tn]
  uint32_t ww[2][TN];   // packed words: [k-step parity][tn]
  // Loads of one step, in issue order (addr::panel2_slot_load): 16 of the activation tile of step s + 1 (phase 0, one per
  // slot), 8 gathers of the scales of step s + 2 (phase 1), 4 of the packed weights of step s + 2 (behind the barrier).
  // Loads retire in order, so "at most n outstanding" means "everything but the youngest n has landed":
  //   slot 32:  the packed weights of step s + 1 (issued a step earlier); younger: this step's 16 + 8      -> vmcnt(24)
  //   slot 57:  the activation tile of step s + 1 and the gathers; nothing younger                          -> vmcnt(0)
  // The step's one barrier stands behind that wait and behind the step's last activation operand read (slot 56 of 64
  // reads the operand of slot 63): past it every wavefront's part of the next activation tile is in LDS, and nobody reads
  // this step's tile any more -- the loads of the tile after next, issued from the next phase 0 on, may overwrite it.
  // The ring of activation operands runs on across the steps: slots 57 .. 63 read the first operands of step s + 1, so
  // that the matrix pipeline never waits behind the barrier for an LDS read.
  // The dequantiser constants of weight tile tn change between the last piece that uses the old ones (phase 2, slot
  // 4 tn + 3) and the first that uses the new ones (phase 3, slot 4 tn).
  constexpr int AR = addr::kPanel2Ahead;  // activation operands in flight (divides the 64 slots of a step)
  static_assert(addr::kPanel2Slots % AR == 0 && addr::kPanel2Slots == 4 * TM, "the operand ring closes over a step");
  uint4_t af[AR];
  // prologue: the scales of steps 0 and 1, everything of step 0, the packed weights of step 1
  {
    const uint8_t *s0 = sc_src(s_tensor, has_s, 0), *z0 = sc_src(z_tensor, HAS_Z, 0);
#pragma unroll
    for (int i = 0; i < 8; ++i) issue_sc1(i, s0, z0);
    const uint8_t *wsrc = w_src(0), *asrc = a_src(0);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) issue_w1(0, tn, wsrc);
#pragma unroll
    for (int j = 0; j < LA; ++j) issue_a1(0, j, asrc);
    pin_scales();  // (the compiler's wait: everything so far)
    const uint8_t *s1 = sc_src(s_tensor, has_s, 1), *z1 = sc_src(z_tensor, HAS_Z, 1);
#pragma unroll
    for (int i = 0; i < 8; ++i) issue_sc1(i, s1, z1);
    wsrc = w_src(1);
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) issue_w1(1, tn, wsrc);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    pin_scales();
  }
  __syncthreads();  // (sv_step / zv_step: step 0, sv_raw / zv_raw: step 1)
#pragma unroll
  for (int j = 0; j < AR - 1; ++j) af[j] = *(const uint4_t*)(smem + fo_a(0) + j * 16 * 256);
  af[AR - 1] = af[0];  // (read in slot 0)
  // Where what stands inside a slot of four MFMAs (measured on this part with one wavefront per SIMD: an MFMA takes
  // 16 cycles of the matrix pipeline and 8 of the wavefront's issue; two vector instructions behind it are free, a third
  // costs 4 cycles; an LDS read is free behind an MFMA that another MFMA follows, and costs 4 cycles when a wait for LDS
  // follows it -- and the compiler puts that wait in front of the slot's first MFMA, which consumes the operand):
  //   MFMA 0, a piece of expansion (2 instructions); MFMA 1, the slot's load if any, the operand read AR slots on, in
  //   four slots per phase a packed word; MFMA 2, a piece (2); MFMA 3, the odd shift of the expansion.
  // The LDS reads are ordinary loads, so that the compiler counts them in its waits; each takes its address from a
  // register that an empty volatile statement "rewrites" behind the MFMA, which keeps the read behind it.
  typedef __attribute__((address_space(3))) const uint4_t* lds16_t;
  typedef __attribute__((address_space(3))) const uint32_t* lds4_t;
  auto lds_read16 = [&](uint32_t& base, uint32_t imm) {  // base: an LDS address in a register of its own
    asm volatile("" : "+v"(base));
    return *(lds16_t)(uintptr_t)(base + imm);
  };
  // LDS addresses of this lane's reads: activation operands of k-step ks of the current ring slot, of k-step 0 of the
  // other; packed words of both
  uint32_t a_k[4], a_nxt = lds0 + fo_a0 + Cfg::SLOT;
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) a_k[ks] = lds0 + fo_a(ks);
  uint32_t w_cur = lds0 + fo_w, w_nxt = lds0 + fo_w + Cfg::SLOT;
  const uint8_t* asrc = a_src(1);
  // One pass over steps [s_begin, s_end) with one dequantiser.  On entry the ring, the loads in flight and the operand ring
  // af are as the previous pass (or the prologue) left them; the words, the dequantiser constants and the expanded first
  // k-step of step s_begin are (re)made here, because the previous pass made them with the other dequantiser.  With
  // stop_on_fraction the pass ends in front of the first step during which constants would be made from zero points that
  // are not small integers, and returns that step.
  auto run_steps = [&](int s_begin, int s_end, auto fold_tag, bool stop_on_fraction) -> int {
    constexpr bool FOLD = decltype(fold_tag)::value;
    typedef Expand8<T, FOLD, LAYOUT> Ex;
    Ex exs[TN];
    auto make_expander = [&](int tn, const uint32_t (&sraw)[TN], const uint32_t (&zraw)[TN]) {  // absent tensors replaced by their constants
      const uint32_t sb = has_s ? sraw[tn] : one_bits, zb = HAS_Z ? zraw[tn] : zs_bits;
      exs[tn] = Ex(bitcast<T>((uint16_t)sb), bitcast<T>((uint16_t)zb), mg);
    };
    auto expand_piece = [&](int part, int ks, int i, typename Ex::Pieces& st, uint32_t shifted) {
      const int tn = part >> 1, p = part & 1;
      uint4_t& o = wop[ks & 1][tn];
      uint32_t& w = ww[ks & 1][tn];
      if constexpr (Ex::SPLITS) {
        if (i == 0) {
          if (p == 0) {
            asm volatile("" : "+v"(w));
            exs[tn].piece(st, w, 0, 0);
          } else {
            exs[tn].piece(st, shifted, 0, 0);  // (shifted = w >> 8: the word's second half, read like a first)
          }
        } else {
          st.pin(i - 1);
          exs[tn].piece(st, w, p, i);
        }
        if (i == 3) {
          st.pin(3);
          Ex::place(o, uint2_t{st.a, st.b}, p);
        }
      } else {
        if (p == 0 && i == 0) o = exs[tn](w);
      }
    };

    {
      const uint8_t* slot = smem + (s_begin & 1) * Cfg::SLOT;
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        ww[0][tn] = *(const uint32_t*)(slot + fo_w + tn * 1024);
        ww[1][tn] = *(const uint32_t*)(slot + fo_w + tn * 1024 + 4);
        make_expander(tn, sv_step, zv_step);
      }
      typename Ex::Pieces st;
#pragma unroll
      for (int part = 0; part < 2 * TN; ++part)
#pragma unroll
        for (int i = 0; i < 4; ++i) expand_piece(part, 0, i, st, ww[0][part >> 1] >> 8);
    }
    int s = s_begin;
    for (; s < s_end; ++s) {
    if constexpr (ZM == 0) {
      if (stop_on_fraction && !integral(zv_raw)) break;  // (zv_raw: the zero points of step s + 1)
    }
    const uint8_t *const ssrc = sc_src(s_tensor, has_s, s + 2), *const zsrc = sc_src(z_tensor, HAS_Z, s + 2);
    const uint8_t* const wsrc = w_src(s + 2);
    uint32_t wsh = 0;
    __builtin_amdgcn_sched_barrier(0);
    typename Ex::Pieces st;
    // (the slots as separate instantiations: every condition below is a compile-time constant of the slot)
    static_for<0, addr::kPanel2Slots>([&](auto tc) {
      constexpr int t = decltype(tc)::value, ks = t / TM, tm = t % TM, j = t % AR;
      if constexpr (t == addr::kPanel2WaitWSlot) {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(addr::kPanel2WaitW) : "memory");  // the packed weights of step s + 1
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      }
      // the dequantiser constants of step s + 1, from the values taken over a step ago
      if constexpr (t >= addr::kPanel2ExpanderSlot && t < addr::kPanel2ExpanderSlot + 4 * TN && (t - addr::kPanel2ExpanderSlot) % 4 == 0)
        make_expander((t - addr::kPanel2ExpanderSlot) / 4, sv_raw, zv_raw);
      if constexpr (t == addr::kPanel2BarrierSlot) {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(addr::kPanel2WaitA) : "memory");
        pin_scales();  // those of step s + 2
        __syncthreads();
      }
      static_for<0, TN>([&](auto tnc) {
        constexpr int tn = decltype(tnc)::value;
        Mma::mma(wop[ks & 1][tn], af[j], acc[tn][tm]);
        // part tm / 2 of k-step ks + 1 (k-step 4 = k-step 0 of step s + 1): two pieces per slot
        if constexpr ((tn & 1) == 0) expand_piece(tm >> 1, ks + 1, 2 * (tm & 1) + (tn >> 1), st, wsh);
        if constexpr (tn == 1) {
          constexpr int kind = addr::panel2_slot_load(t), idx = addr::panel2_slot_load_index(t);
          if constexpr (kind == addr::kPanel2LoadA) issue_a1(s + 1, idx, asrc);
          if constexpr (kind == addr::kPanel2LoadScale) issue_sc1(idx, ssrc, zsrc);
          if constexpr (kind == addr::kPanel2LoadW) issue_w1(s + 2, idx, wsrc);  // (the last word of step s left its ring slot in phase 1)
          // the ring entry that the slot before this one consumed takes the operand of slot t + AR - 1: of this step,
          // or one of the first of the next step, behind the barrier
          constexpr int at = t + AR - 1, jn = at % AR;
          if constexpr (at < 4 * TM)
            af[jn] = lds_read16(a_k[at / TM], (uint32_t)((at % TM) * 16 * 256));
          else
            af[jn] = lds_read16(a_nxt, (uint32_t)((at - 4 * TM) * 16 * 256));
          // the words two k-steps on (phases 2 and 3: of step s + 1), one in each of slots 8 .. 11 of a phase
          if constexpr (tm >= addr::kPanel2WordSlot && tm < addr::kPanel2WordSlot + TN) {
            constexpr int wt = tm - addr::kPanel2WordSlot;
            uint32_t& base = ks < 2 ? w_cur : w_nxt;
            asm volatile("" : "+v"(base));
            ww[ks & 1][wt] = *(lds4_t)(uintptr_t)(base + (uint32_t)(((ks + 2) & 3) * 4 + wt * 1024));
          }
        }
        if constexpr (tn == TN - 1) {
          // the second half of a word goes through a shift: one instruction ahead of the part's first piece
          if constexpr ((tm & 3) == 1) {
            uint32_t& w = ww[(ks + 1) & 1][tm >> 2];
            asm volatile("" : "+v"(w));
            wsh = w >> 8;
            asm volatile("" : "+v"(wsh));
          }
          if constexpr (t == 60) asrc = a_src(s + 2);
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    });
    {
      const uint32_t x = a_k[0];
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) a_k[ks] = a_nxt ^ (uint32_t)(ks << 4);  // (fo_a(ks) = fo_a(0) ^ 16 ks; slots are multiples of 64 bytes apart)
      a_nxt = x;
    }
    { const uint32_t x = w_cur; w_cur = w_nxt; w_nxt = x; }
    }
    return s;
  };
  if constexpr (ZM == 0) {
    int s = 0;
    if (integral(zv_step)) s = run_steps(0, steps, std::true_type{}, true);
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
  static_assert(Cfg::WAVES * TM * 16 * kStageBytes <= Cfg::LDS, "the staging areas of the wavefronts fit the ring");
  // (the loads issued past the last step; and the wait states between the last MFMAs, which the compiler does not know
  // for what they are, and the first instruction that reads an accumulator)
  asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  __syncthreads();  // everyone is past the last step: the ring becomes the output staging area
  write_tile<EpiFloat, TM, TN>(epi, acc, smem + wave * (TM * 16 * kStageBytes), lane, m0, n0 + wave * (16 * TN), M, N);
}

}  // namespace

thread_local int g_panel2_slice_steps = 0;  // tuning and tests: steps of 128 values of K per slice (0: the plan's own)

// Launch geometry.  ok = the kernel applies.
struct Panel2Plan {
  bool ok;
  int tiles_m, tiles_n, split, slice_steps;
};
Panel2Plan w4a16_panel256_plan(int64_t M, int64_t N, int64_t K, int64_t group, int cus) {
  Panel2Plan p{false, 0, 0, 0, 0};
  if (M < 1 || N < 1 || K < 128 || K % 128 != 0 || group < 32 || (group & (group - 1)) != 0 || K % group != 0) return p;
  if (N % 16 != 0 || M % 4 != 0) return p;  // a direct load (16 weight rows, 4 activation rows) lies inside a matrix or outside
  if (M >= ((int64_t)1 << 30) || N >= ((int64_t)1 << 30)) return p;
  p.tiles_m = (int)ceil_div(M, (int64_t)Panel2Cfg::BM);
  p.tiles_n = (int)ceil_div(N, (int64_t)Panel2Cfg::BN);
  const int steps_total = (int)(K / 128);
  // a slice is a whole number of groups or, with groups longer than a slice (one scale per weight row, say), a power-of-two
  // part of one group: the kernel takes every step's group from the step's position in K
  const int unit = group > 128 ? (int)(group / 128) : 1;
  auto whole_or_part = [&](int64_t steps) {
    if (steps >= unit) return ceil_div(steps, (int64_t)unit) * unit;
    int64_t part = 1;
    while (part < steps) part *= 2;
    return part;
  };
  const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
  if (cus <= 0) cus = 256;
  int64_t ss = steps_total;
  if (g_panel2_slice_steps > 0) {
    ss = whole_or_part((int64_t)g_panel2_slice_steps);
  } else if (tiles * 2 <= cus) {
    // K slices only where the tiles leave most of the machine idle: the cut that fills it best with slices of 16 steps or more
    double best = (double)ceil_div(tiles, (int64_t)cus) * (steps_total + 8);
    for (int64_t want = 2; want <= 16; ++want) {
      int64_t cand = whole_or_part(ceil_div((int64_t)steps_total, want));
      if (cand < 16 || cand >= steps_total) continue;
      const int64_t sl = ceil_div((int64_t)steps_total, cand);
      const double t = (double)ceil_div(tiles * sl, (int64_t)cus) * (double)(cand + 8) + (double)sl * (double)M * (double)N * 4.0 / 3e6 / 3.0;
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
static int launch_panel256(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, float* partial, int64_t M,
                           int64_t N, int64_t K, int gshift, float zero_scalar, int out_dtype, const Panel2Plan& p, int band_rows,
                           hipStream_t st) {
  auto kern = w4a16_panel256_kernel<T, LAYOUT, ZM>;
  constexpr int lds_bytes = Panel2Cfg::LDS;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) {
      set_error("tlq_gemm_w4a16(panel256): cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
      return 1;
    }
    attr_set = true;
  }
  const unsigned blocks = (unsigned)((int64_t)p.tiles_m * p.tiles_n * p.split);
  kern<<<blocks, 256, lds_bytes, st>>>((const T*)A, (const uint8_t*)Wp, (const T*)scales, (const T*)zeros, C, partial, (int)M, (int)N,
                                       (int)K, gshift, zero_scalar, out_dtype, p.slice_steps, p.tiles_m, p.tiles_n, band_rows);
  return check_launch("tlq_gemm_w4a16(panel256)", ZM == 0 ? "w4a16_panel256_kernel, zero-point tensor" : "w4a16_panel256_kernel")
             ? 0
             : 1;
}

// partial: fp32 [split][M][N] workspace, needed when the plan has more than one K slice
int gemm_w4a16_panel256(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t N, int64_t K,
                        int64_t group, float zero_scalar, int in_dtype, int out_dtype, int w_layout, const Panel2Plan& p, float* partial,
                        hipStream_t st) {
  int gshift = 0;
  while (((int64_t)1 << gshift) < group) ++gshift;
  const int band = g_gemm_band_rows > 0 ? g_gemm_band_rows : 4;
  const bool fold_scalar = zero_scalar == (float)(int)zero_scalar && zero_scalar >= -256.0f && zero_scalar <= 256.0f;
  int rc;
#define TLQ_PANEL3(T, LAY, ZM) launch_panel256<T, LAY, ZM>(A, Wp, scales, zeros, C, partial, M, N, K, gshift, zero_scalar, out_dtype, p, band, st)
#define TLQ_PANEL2(T, ZM) (w_layout == TLQ_W_INTERLEAVED_F16 ? TLQ_PANEL3(T, 1, ZM) : TLQ_PANEL3(T, 0, ZM))
#define TLQ_PANEL(ZM) (in_dtype == TLQ_F16 ? TLQ_PANEL2(half_t, ZM) : TLQ_PANEL2(bf16_t, ZM))
  if (zeros != nullptr)
    rc = TLQ_PANEL(0);
  else
    rc = fold_scalar ? TLQ_PANEL(1) : TLQ_PANEL(2);
#undef TLQ_PANEL
#undef TLQ_PANEL2
#undef TLQ_PANEL3
  if (rc) return rc;
  if (p.split > 1) {
    launch_splitk_reduce(partial, C, M, N, p.split, out_dtype, st);
    return check_launch("tlq_gemm_w4a16(panel256, reduce)", "splitk_reduce_kernel") ? 0 : 1;
  }
  return 0;
}

}  // namespace tlq
