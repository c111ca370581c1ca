// 256 x 256 tile, both operands copied global -> LDS directly (activations row-major [M, K]; weights [N, K], or int8
// [K, N] read transposed), with the 160 KB of LDS cut into FIVE slots of one operand tile (32 KB: 256 rows x 128 bytes
// of K, or 128 k x 256 bytes of N) instead of two stages of two tiles.
//
// With two stages the loads of stage k + 1 can only be issued when stage k - 1 has been consumed and must have landed
// one stage of MFMA time later; a stage's slowest load takes longer than that, and the loop runs at the pace of the
// loads.  Here tile t (A of stage s is t = 2s, W of stage s is t = 2s + 1) lives in slot t mod 5.  At the start of
// stage k the slots of A(k - 1) and W(k - 1) are free, which is where W(k + 1) and A(k + 2) go: one and a half stages
// of loads are in flight, the A tiles are requested two stages ahead and the W tiles one stage ahead with only half
// a stage's bytes behind them.  The wait at the end of stage k leaves the youngest tile (A(k + 2), four loads per
// wavefront) outstanding.  Everything else -- wave tiling, LDS tile layout, fragment reads, epilogue -- is the
// two-stage kernel's.
//
// Selected by tlq_tune_gemm_slots(1); whole stages only (K bytes a multiple of 128).
#pragma once
#include "gemm_core.h"

namespace tlq {

template <class Mma, class WL, class Epi>
__global__ __launch_bounds__(512, 2) void gemm_slots_kernel(typename RowLoaderDirect<256, 512>::Params pa,
                                                           typename WL::Params pw, typename Epi::Params pe, int M, int N,
                                                           int KT, int tiles_m, int tiles_n, int band_rows) {
  constexpr int BM = 256, BN = 256, WM = 2, WN = 4, TM = 8, TN = 4, SLOTS = 5;
  constexpr int TILE = 256 * kStageBytes;  // one operand, one stage: 32 KB
  typedef RowLoaderDirect<256, 512> Loader;
  static_assert(Loader::PER_WAVE == 4 && WL::PER_WAVE == 4 && WL::DIRECT, "the waits below count four direct loads per wavefront and tile");
  extern __shared__ __align__(16) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m0 = (wave % WM) * (BM / WM), wave_n0 = (wave / WM) * (BN / WN);
  const TileCoord tc = tile_of_block<BM, BN>(tiles_m, tiles_n, band_rows);
  Loader al(pa, tc.batch, tc.m0, M, tid);
  WL wl(pw, tc.batch, tc.n0, N, tid);
  typename Loader::Regs regs;  // unused by full stages (the data never passes through registers)
  typename WL::Regs regs_w;
  const RowFrag fragA(lane, wave_m0);
  const typename WL::Frag fragW(lane, wave_n0);
  typename Mma::acc_t acc[TN][TM];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn)
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = typename Mma::acc_t{0, 0, 0, 0};

  // per-row / per-column output scales travel while the main loop runs (24 registers; this kernel has 256 per lane)
  const Epi epi(pe, tc.batch);
  const auto out_scales = fetch_scales<Epi, TM, TN>(epi, tc.m0 + wave_m0, tc.n0 + wave_n0, lane, M, N);

  auto slot_of = [&](int t) { return smem + addr::slot_of_tile(t) * TILE; };
  struct Ops {
    decltype(slot_of)& slot;
    const Loader& al;
    const WL& wl;
    typename Loader::Regs& regs;
    typename WL::Regs& regs_w;
    const RowFrag& fragA;
    const typename WL::Frag& fragW;
    typename Mma::acc_t (&acc)[TN][TM];
    __device__ __forceinline__ void issue_a(int s) { al.template gload<false>(regs, s, slot(2 * s)); }
    __device__ __forceinline__ void issue_w(int s) { wl.template gload<false>(regs_w, s, slot(2 * s + 1)); }
    // four direct loads per wavefront and tile: vmcnt(4) leaves exactly the youngest tile outstanding
    __device__ __forceinline__ void wait_tiles(bool keep) {
      if (keep)
        asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
      else
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __device__ __forceinline__ void barrier() { __syncthreads(); }
    __device__ __forceinline__ void compute(int k) {
      const uint8_t* la = slot(2 * k);
      const uint8_t* lw = slot(2 * k + 1);
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        uint4_t wf[TN], af[TM];
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) wf[tn] = fragW.read(lw, ks, tn);
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) af[tm] = fragA.read(la, ks, tm);
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
          for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = Mma::mma(wf[tn], af[tm], acc[tn][tm]);
      }
    }
  } ops{slot_of, al, wl, regs, regs_w, fragA, fragW, acc};
  addr::slots_schedule(KT, ops);

  if constexpr (Epi::STAGED) __syncthreads();  // every wavefront is past its last operand read: LDS becomes the output staging area
  write_tile_with<Epi, TM, TN>(epi, out_scales, acc, smem + wave * (TM * 16 * kStageBytes), lane, tc.m0 + wave_m0, tc.n0 + wave_n0, M, N);
}

// tlq_tune_gemm_slots: 0 = the two-stage kernel (default), 1 = this one where it applies
extern thread_local int g_gemm_slots;

// k_bytes (bytes of K per activation row) a positive multiple of 128: whole stages only.
template <class Mma, class WL, class Epi>
int launch_gemm_slots(const typename RowLoaderDirect<256, 512>::Params& pa, const typename WL::Params& pw,
                      const typename Epi::Params& pe, int64_t batch, int64_t M, int64_t N, int64_t k_bytes, hipStream_t st,
                      const char* what, int band_rows) {
  auto kern = gemm_slots_kernel<Mma, WL, Epi>;
  constexpr int lds_bytes = 5 * 256 * kStageBytes;  // all of the CU's LDS
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) {
      set_error("%s: cannot reserve %d bytes of LDS: %s", what, lds_bytes, hipGetErrorString(e));
      return 1;
    }
    attr_set = true;
  }
  const int64_t tiles_m = ceil_div(M, (int64_t)256), tiles_n = ceil_div(N, (int64_t)256);
  const int64_t blocks = batch * tiles_m * tiles_n;
  if (blocks <= 0) return 0;
  if (blocks > 0x7fffffff) {
    set_error("%s: too many tiles", what);
    return 1;
  }
  kern<<<(unsigned)blocks, 512, lds_bytes, st>>>(pa, pw, pe, (int)M, (int)N, (int)(k_bytes / kStageBytes), (int)tiles_m,
                                                 (int)tiles_n, g_gemm_band_rows > 0 ? g_gemm_band_rows : band_rows);
  return check_launch(what, "gemm_slots_kernel 256x256 tiles, five slots") ? 0 : 1;
}

}  // namespace tlq
