// W4A16 for decode batches (1 .. 32 activation rows): every packed weight is read from HBM once, as full-width direct
// global -> LDS loads into wavefront-private rings deep enough to cover the memory latency, dequantised in registers
// straight into MFMA operands, and multiplied with activation operands that stay in registers for the whole launch.
//
//   * A work-group of up to 16 wavefronts covers a chunk of K: wavefront w owns values 256 s .. 256 s + 255
//     (s = chunk * waves + w) and keeps the matching activations A[0 .. 16 MT)[that slice] as MFMA operands in
//     32 MT registers.  With K <= 4096 one chunk covers K and the result is written directly; longer rows take
//     several chunks (grid y), fp32 partial results in a workspace and splitk_reduce_kernel.
//   * Work-groups are persistent: work-group b handles the 16-row weight tiles b, b + grid, ...; a wavefront's tiles
//     form one stream through a ring of three slots, so the loads of the next two tiles are in flight while a tile is
//     multiplied and reduced.  Per tile: two 1 KB loads of packed weights (16 rows x 64 B, the two k-blocks of 128
//     values of the slice) and one dword gather each, by 16 to 64 lanes, for the scales and zero points of the 16 rows.
//     Everything else in the loop is kept to a minimum: the kernel is bound by instruction issue (about 100
//     instructions per 1 KB of packed weights, most of them the dequantisation).
//   * Per tile the wavefronts' partial tiles meet in LDS (two buffers, one barrier per tile) and are added in
//     wavefront order by a wavefront that rotates from tile to tile.
//
// The dequantisation skips the four byte permutes per word that put a plain word's values back into k order (the
// decode of expand8.h for interleaved words, applied to either layout): for plain words the activation operands are
// permuted the same way once, when they are loaded; interleaved words come out in k order by themselves.
//
// k assignment as in the streaming kernel: lane (row r16, k-group q) holds at MFMA k-step j the eight values of packed
// word 4 q + j of its row's 64 bytes, k = 32 q + 8 j .. + 7 inside the k-block; the activation operand of lane
// (m = r16, q) holds the same eight k.  The activations reach their operand lanes through the wavefront's LDS (direct
// loads of whole 256-byte row segments, then 16-byte reads), once per launch.
#include "expand8.h"
#include "gemm_addr.h"
#include "gemm_core.h"

namespace tlq {

void launch_splitk_reduce(const float* partial, void* C, int64_t M, int64_t N, int split, int out_dtype, hipStream_t st);

namespace {

template <typename T>
struct DecodeMma;
template <>
struct DecodeMma<half_t> {
  typedef MmaF16 type;
};
template <>
struct DecodeMma<bf16_t> {
  typedef MmaBF16 type;
};

// s_waitcnt takes an immediate: 4 loads per tile, at most two younger tiles, plus the tile's own second piece
__device__ __forceinline__ void wait_vm(int c) {
  switch (c) {
    case 9: asm volatile("s_waitcnt vmcnt(9)" ::: "memory"); break;
    case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
    case 5: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
    case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
    case 1: asm volatile("s_waitcnt vmcnt(1)" ::: "memory"); break;
    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;  // never too few: waiting for everything is always safe
  }
}

template <typename T, int MT, int LAYOUT>
__global__ __launch_bounds__(1024) void w4a16_decode_kernel(const T* __restrict__ A, const uint8_t* __restrict__ Wp,
                                                            const T* __restrict__ scales, const T* __restrict__ zeros,
                                                            void* __restrict__ C, float* __restrict__ partial, int M, int N,
                                                            int K, int gshift, float zero_scalar, int out_dtype, int tiles,
                                                            int slices) {
  typedef typename DecodeMma<T>::type Mma;
  typedef __attribute__((address_space(3))) uint8_t* lptr_t;
  constexpr int TS = addr::kDecTileSlots;
  constexpr uint32_t SLOT = addr::kDecSlotBytes;
  constexpr int RB = MT == 1 ? 2 : 1;  // buffers of partial sums: with one, a second barrier per tile protects it
  constexpr uint32_t RED = TS * SLOT, WAVE = RED + RB * MT * 1024;
  extern __shared__ __align__(16) uint8_t smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int waves = blockDim.x >> 6;
  const int r16 = lane & 15, q = lane >> 4;
  uint8_t* const mine = smem + wave * WAVE;
  const uint32_t mine_lds = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lptr_t)mine);
  const int chunk = blockIdx.y;
  const int slice = chunk * waves + wave;
  const bool active = slice < slices;  // uniform per wavefront
  int n_active = slices - chunk * waves;
  n_active = n_active < waves ? n_active : waves;
  const int64_t k0 = (int64_t)(active ? slice : 0) * addr::kDecSlice;
  const int groups = K >> gshift;
  const int first = blockIdx.x, stride = gridDim.x;
  const int my_tiles = (tiles - first + stride - 1) / stride;
  const bool has_s = scales != nullptr, has_z = zeros != nullptr;
  const T one = from_float<T>(1.0f), zs = from_float<T>(zero_scalar);
  const NibbleMagic mg = make_nibble_magic();
  const uint32_t fo_w = addr::sw_frag_off(lane);

  // per-lane parts of the load addresses: the same in every tile but the last, whose rows past N repeat row N - 1
  const uint32_t w_lane = addr::dec_w_lane(lane, 0, 16, K), w_lane_last = addr::dec_w_lane(lane, tiles - 1, N, K);
  const bool sc_lane = lane < 16 * addr::dec_sc_dwords(gshift);
  const int64_t sc_e0 = addr::dec_sc_elem(lane, 0, 16, groups, k0, gshift);
  const int64_t sc_e_last = addr::dec_sc_elem(lane, tiles - 1, N, groups, k0, gshift);
  const uint32_t rd_cell[2] = {addr::dec_sc_cell(lane, 0, gshift), addr::dec_sc_cell(lane, 1, gshift)};
  const uint32_t rd_half[2] = {addr::dec_sc_half(lane, 0, groups, k0, gshift), addr::dec_sc_half(lane, 1, groups, k0, gshift)};
  // a tensor that is absent is gathered from the activations instead (never used): the number of loads per tile stays four
  const uint8_t* const s_src = has_s ? (const uint8_t*)scales : (const uint8_t*)A;
  const uint8_t* const z_src = has_z ? (const uint8_t*)zeros : (const uint8_t*)A;

  auto issue_tile = [&](int ts) {
    const int t = first + ts * stride;
    const uint32_t l0 = mine_lds + (uint32_t)(ts % TS) * SLOT;
    const bool last = t == tiles - 1;
    const uint32_t sc_off = addr::dec_sc_off(last ? sc_e_last : sc_e0 + (int64_t)t * 16 * groups);
    const uint32_t so = has_s ? sc_off : 0u, zo = has_z ? sc_off : 0u;
    if (sc_lane) {
      asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, %2" ::"s"(l0 + 2048u), "v"(so), "s"(s_src) : "memory");
      asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, %2" ::"s"(l0 + 2304u), "v"(zo), "s"(z_src) : "memory");
    }
    const uint8_t* wsb = uniform_ptr(Wp + addr::dec_w_base(t, K, k0));
    const uint32_t voff = last ? w_lane_last : w_lane;
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(l0), "v"(voff), "s"(wsb) : "memory");
    // the instruction offset moves the LDS side as well as the global side: M0 is set 64 bytes low to land on l0 + 1024
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2 offset:64" ::"s"(l0 + 1024u - 64u), "v"(voff), "s"(wsb) : "memory");
  };

  // ---- activations of this wavefront's K slice -> MFMA operands in registers ----
  // Direct loads of 1 KB into the wavefront's own LDS, one [16 rows][256 B] block (4 KB) at a time, staged in the third
  // ring slot plus the partial-sum area (both idle yet): direct loads move twice as many bytes per clock as loads into
  // registers, and every work-group has to pull all of A through its CU.  The first two tiles of weights are requested
  // right behind the first block, so that HBM is busy while the activations (L2 hits) are rearranged.
  uint4_t af[2][4][MT];
  if (active) {
    constexpr uint32_t STG = 2 * SLOT;
    static_assert(STG + 4096 <= WAVE, "staging area of the activations");
    auto issue_block = [&](int kb, int mt) {
      const uint8_t* asb = uniform_ptr((const uint8_t*)A + (k0 + kb * 128) * 2);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t voff = (uint32_t)(addr::dec_a_off(lane, mt, kb, i, M, K, k0) - (k0 + kb * 128) * 2);
        // rows past M are not fetched: what the staging area holds for them only reaches output rows that are never stored
        if (mt * 16 + 4 * i + (lane >> 4) < M)
          asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(mine_lds + STG + (uint32_t)(i * 1024)), "v"(voff), "s"(asb)
                       : "memory");
      }
    };
    issue_block(0, 0);
    issue_tile(0);
    if (my_tiles > 1) issue_tile(1);
#pragma unroll
    for (int b = 0; b < 2 * MT; ++b) {
      const int kb = b / MT, mt = b % MT;
      // loads return in issue order: the first block is followed by at most two tiles (eight loads), every later block
      // is the youngest load there is
      if (b == 0) {
        if (my_tiles > 1) asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); else asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
      } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint4_t v = *(const uint4_t*)(mine + STG + addr::dec_a_frag(lane, j));
        if (LAYOUT == 0) {
          // plain words are decoded without the byte permutes that would restore k order, i.e. as values
          // k0, k4, k1, k5, k2, k6, k3, k7 of the word: the activations take the same order, once, here
          af[kb][j][mt] = uint4_t{__builtin_amdgcn_perm(v.z, v.x, 0x05040100u), __builtin_amdgcn_perm(v.z, v.x, 0x07060302u),
                                  __builtin_amdgcn_perm(v.w, v.y, 0x05040100u), __builtin_amdgcn_perm(v.w, v.y, 0x07060302u)};
        } else {
          af[kb][j][mt] = v;
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the staging area is free again: next block, or the third tile
      if (b + 1 < 2 * MT) issue_block((b + 1) / MT, (b + 1) % MT);
    }
    if (my_tiles > 2) issue_tile(2);
  }

  typename Mma::acc_t acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = typename Mma::acc_t{0, 0, 0, 0};

  for (int ts = 0; ts < my_tiles; ++ts) {
    const int t = first + ts * stride;
    if (active) {
      if (ts > 0 && ts + 2 < my_tiles) issue_tile(ts + 2);  // into the slot that tile ts - 1 was read from (tile 2: issued above)
      const uint8_t* const slotp = mine + (ts % TS) * SLOT;
      wait_vm(addr::dec_wait_count(ts, 1, my_tiles));  // one wait per tile: both k-blocks, their scales and zero points
      if constexpr (MT == 1) {
        // one round of LDS reads per tile, and the two k-blocks accumulate separately (two independent MFMA chains)
        uint4_t wf[2];
        uint32_t sdw[2], zdw[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
          wf[kb] = *(const uint4_t*)(slotp + kb * 1024 + fo_w);
          sdw[kb] = *(const uint32_t*)(slotp + 2048 + rd_cell[kb]);
          zdw[kb] = *(const uint32_t*)(slotp + 2304 + rd_cell[kb]);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        T sv[2], zv[2];
        bool ok = true;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
          sv[kb] = has_s ? bitcast<T>((uint16_t)(sdw[kb] >> rd_half[kb])) : one;
          zv[kb] = has_z ? bitcast<T>((uint16_t)(zdw[kb] >> rd_half[kb])) : zs;
          const float zf = to_float(zv[kb]);
          ok = ok && zf == __builtin_rintf(zf) && zf >= -256.0f && zf <= 256.0f;
        }
        typename Mma::acc_t acc2[2] = {typename Mma::acc_t{0, 0, 0, 0}, typename Mma::acc_t{0, 0, 0, 0}};
        if (__builtin_amdgcn_ballot_w64(ok) == ~0ull) {  // integer zero points fold into the unpack bias (exact)
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
              const Expand8<T, true, 1> ex(sv[kb], zv[kb], mg);
              const uint32_t w[4] = {wf[kb].x, wf[kb].y, wf[kb].z, wf[kb].w};
              acc2[kb] = Mma::mma(ex(w[j]), af[kb][j][0], acc2[kb]);
            }
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
              const Expand8<T, false, 1> ex(sv[kb], zv[kb], mg);
              const uint32_t w[4] = {wf[kb].x, wf[kb].y, wf[kb].z, wf[kb].w};
              acc2[kb] = Mma::mma(ex(w[j]), af[kb][j][0], acc2[kb]);
            }
        }
        acc[0] = acc2[0] + acc2[1];
      } else {
        // two activation tiles: the operands fill the register file (128 per lane with 16 wavefronts per CU), so the
        // k-blocks go one after the other into one chain per activation tile
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[mt] = typename Mma::acc_t{0, 0, 0, 0};
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
          const uint4_t wf = *(const uint4_t*)(slotp + kb * 1024 + fo_w);
          const uint32_t sdw = *(const uint32_t*)(slotp + 2048 + rd_cell[kb]);
          const uint32_t zdw = *(const uint32_t*)(slotp + 2304 + rd_cell[kb]);
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          const T sv = has_s ? bitcast<T>((uint16_t)(sdw >> rd_half[kb])) : one;
          const T zv = has_z ? bitcast<T>((uint16_t)(zdw >> rd_half[kb])) : zs;
          const float zf = to_float(zv);
          const bool ok = zf == __builtin_rintf(zf) && zf >= -256.0f && zf <= 256.0f;
          const uint32_t w[4] = {wf.x, wf.y, wf.z, wf.w};
          if (__builtin_amdgcn_ballot_w64(ok) == ~0ull) {
            const Expand8<T, true, 1> ex(sv, zv, mg);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const uint4_t b = ex(w[j]);
#pragma unroll
              for (int mt = 0; mt < MT; ++mt) acc[mt] = Mma::mma(b, af[kb][j][mt], acc[mt]);
            }
          } else {
            const Expand8<T, false, 1> ex(sv, zv, mg);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const uint4_t b = ex(w[j]);
#pragma unroll
              for (int mt = 0; mt < MT; ++mt) acc[mt] = Mma::mma(b, af[kb][j][mt], acc[mt]);
            }
          }
        }
      }
    }
    if (RB == 1 && ts > 0) __syncthreads();  // the single buffer: the wavefronts that added up tile ts - 1 have read it
    if (active) {
      // partial tile of this wavefront -> its slot of buffer ts % RB
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        *(float4_t*)(mine + RED + ((ts % RB) * MT + mt) * 1024 + lane * 16) = acc[mt];
      }
    }
    __syncthreads();  // all partial tiles of tile t are in LDS (two buffers: the other one was read before the previous barrier)
    int rw = wave - (ts * MT) % waves;
    rw = rw < 0 ? rw + waves : rw;
    if (rw < MT) {  // wavefronts (ts MT) % waves .. + MT - 1 add up the MT activation tiles
      const int mt = rw;
      const uint32_t ro = RED + ((ts % RB) * MT + mt) * 1024 + lane * 16;
      float4_t sum = *(const float4_t*)(smem + ro);
      for (int w = 1; w < n_active; ++w) sum += *(const float4_t*)(smem + w * WAVE + ro);
      // lane l holds D[n = 4 (l / 16) + i][m = l % 16]
      const int m = mt * 16 + r16;
      const int n = t * 16 + 4 * q;
      if (m < M && n < N) {
        const int64_t idx = (int64_t)m * N + n;
        if (partial) {
          float* const P = partial + (int64_t)chunk * M * N;
          if (n + 3 < N && (N & 3) == 0) {
            *(float4_t*)(P + idx) = sum;
          } else {
            for (int i = 0; i < 4 && n + i < N; ++i) P[idx + i] = sum[i];
          }
        } else if (n + 3 < N && (N & 3) == 0) {
          if (out_dtype == TLQ_F32) {
            *(float4_t*)((float*)C + idx) = sum;
          } else if (out_dtype == TLQ_F16) {
            half_t h[4] = {(half_t)sum[0], (half_t)sum[1], (half_t)sum[2], (half_t)sum[3]};
            *(uint2_t*)((half_t*)C + idx) = bitcast<uint2_t>(h);
          } else {
            *(uint2_t*)((uint16_t*)C + idx) = uint2_t{pack_bf16x2(sum[0], sum[1]), pack_bf16x2(sum[2], sum[3])};
          }
        } else {
          for (int i = 0; i < 4 && n + i < N; ++i) store_out(C, idx + i, sum[i], out_dtype);
        }
      }
    }
  }
}

}  // namespace

struct DecodePlan {
  bool ok;
  int mt, chunks, waves, grid_x;
  int64_t lds_bytes;
};

// Shapes the kernel takes: 1 <= M <= 32, K a multiple of 256, a power-of-two group >= 32 that divides K; scale and zero
// tensors that start on a dword boundary and hold an even number of values (their gathers read aligned dwords).
DecodePlan w4a16_decode_plan(int64_t M, int64_t N, int64_t K, int64_t group, int cus) {
  DecodePlan p{false, 0, 0, 0, 0, 0};
  if (M < 1 || M > 32 || N < 1 || K < addr::kDecSlice || K % addr::kDecSlice != 0) return p;
  if (group < 32 || (group & (group - 1)) != 0 || K % group != 0) return p;
  if (((N * (K / group)) & 1) != 0) return p;
  if (N * (K / 2) >= ((int64_t)1 << 32) || M * K * 2 >= ((int64_t)1 << 32)) return p;
  if (cus < 1) cus = 256;
  const int64_t slices = K / addr::kDecSlice;
  p.mt = M <= 16 ? 1 : 2;
  p.chunks = (int)((slices + 15) / 16);
  p.waves = (int)((slices + p.chunks - 1) / p.chunks);
  const int64_t tiles = (N + 15) / 16;
  int64_t gx = cus / p.chunks;
  gx = gx < 1 ? 1 : gx;
  p.grid_x = (int)(gx < tiles ? gx : tiles);
  p.lds_bytes = (int64_t)p.waves * addr::dec_wave_bytes(p.mt);
  // every activation tile's partial sums are added up by a wavefront of its own: a row of 256 values (one wavefront)
  // cannot serve two activation tiles
  p.ok = p.lds_bytes <= 160 * 1024 && p.chunks <= 16 && p.waves >= p.mt;
  return p;
}

template <typename T, int MT, int LAYOUT>
static int launch_decode(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, float* partial, int64_t M,
                         int64_t N, int64_t K, int gshift, float zero_scalar, int out_dtype, const DecodePlan& p, hipStream_t st) {
  auto kern = w4a16_decode_kernel<T, MT, LAYOUT>;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) {
      set_error("tlq_gemm_w4a16(decode): cannot reserve LDS: %s", hipGetErrorString(e));
      return 1;
    }
    attr_set = true;
  }
  const int tiles = (int)((N + 15) / 16);
  kern<<<dim3(p.grid_x, p.chunks), p.waves * 64, (size_t)p.lds_bytes, st>>>(
      (const T*)A, (const uint8_t*)Wp, (const T*)scales, (const T*)zeros, C, p.chunks > 1 ? partial : nullptr, (int)M, (int)N, (int)K,
      gshift, zero_scalar, out_dtype, tiles, (int)(K / addr::kDecSlice));
  return check_launch("tlq_gemm_w4a16(decode)", "w4a16_decode_kernel") ? 0 : 1;
}

// partial: fp32 [chunks][M][N] when the plan has more than one chunk (ignored otherwise)
int gemm_w4a16_decode(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t N, int64_t K,
                      int64_t group, float zero_scalar, int in_dtype, int out_dtype, int w_layout, const DecodePlan& p, float* partial,
                      hipStream_t st) {
  int gshift = 0;
  while (((int64_t)1 << gshift) < group) ++gshift;
  int rc;
#define TLQ_DEC(T, MTT, LAY) launch_decode<T, MTT, LAY>(A, Wp, scales, zeros, C, partial, M, N, K, gshift, zero_scalar, out_dtype, p, st)
  if (w_layout == TLQ_W_INTERLEAVED_F16) {
    if (in_dtype == TLQ_F16)
      rc = p.mt == 1 ? TLQ_DEC(half_t, 1, 1) : TLQ_DEC(half_t, 2, 1);
    else
      rc = p.mt == 1 ? TLQ_DEC(bf16_t, 1, 1) : TLQ_DEC(bf16_t, 2, 1);
  } else {
    if (in_dtype == TLQ_F16)
      rc = p.mt == 1 ? TLQ_DEC(half_t, 1, 0) : TLQ_DEC(half_t, 2, 0);
    else
      rc = p.mt == 1 ? TLQ_DEC(bf16_t, 1, 0) : TLQ_DEC(bf16_t, 2, 0);
  }
#undef TLQ_DEC
  if (rc) return rc;
  if (p.chunks == 1) return 0;
  launch_splitk_reduce(partial, C, M, N, p.chunks, out_dtype, st);
  return check_launch("tlq_gemm_w4a16(decode, reduce)", "splitk_reduce_kernel") ? 0 : 1;
}

}  // namespace tlq
