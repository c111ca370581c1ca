// LDS-staged MFMA GEMM main loop for gfx950, shared by the W4A16, fp16/bf16 and int8 paths.
//
//   D[n, m] += sum_k Wt[n, k] * At[m, k]
//
// Everything is expressed in BYTES of K: one stage is 128 bytes of K per row (64 fp16/bf16
// or 128 int8 values).  Both operand tiles live in LDS as [rows][128 B] with the 16-byte
// chunk index XOR-swizzled by (row & 7), and one 16x16 MFMA k-step consumes one 16-byte chunk
// per lane from each operand (v_mfma_f32_16x16x32_{f16,bf16}: 8 values, v_mfma_i32_16x16x64_i8:
// 16 values), so the loop body is identical for all element types.
//
// MFMA operand roles: the WEIGHT tile is the first (row) operand and the ACTIVATION tile
// the second (column) operand.  Lane l then holds D[n = 4*(l/16) + i][m = l%16], i = 0..3,
// i.e. four consecutive output columns of one row of the row-major C[M, N]: the epilogue
// writes 8/16-byte vectors.
//
// Pipeline: global -> registers -> (convert / dequantise / transpose) -> LDS, double
// buffered.  The global loads of stage t+1 are issued at the top of stage t; their conversion
// and LDS stores are cut into pieces that follow every group of MFMAs of stage t; one barrier
// per stage.  Addressing is arranged so that the loop needs almost no address arithmetic:
// global loads use a scalar base that advances per stage plus a loop-invariant 32-bit lane
// offset, LDS accesses use a loop-invariant lane offset plus an immediate (the swizzle depends
// only on row bits 0..2, so rows 8 apart differ by a constant).
#pragma once

#include <type_traits>

#include "gemm_addr.h"
#include "tlq_common.h"

namespace tlq {

constexpr int kStageBytes = 128;

// 16-byte chunk swizzle.  Measured on gfx950 with the LDS bank-conflict counter: conflict free
// for the MFMA operand reads (16 consecutive rows, one logical chunk per 16 lanes), the row-copy
// stores (8 lanes per row) and the dequantising stores (2 lanes per row, 4 chunks each).
static_assert(kStageBytes == addr::kStage, "stage width");
__device__ __forceinline__ int lds_swz(int row) { return addr::row_swz(row); }
__device__ __forceinline__ int lds_off(int row, int chunk) { return addr::row_lds_off(row, chunk); }

// ---- MFMA operand fragments ---------------------------------------------------------------
// A loader names the reader of its LDS tile layout as `Frag`:
//   Frag(lane, wave_row0)     per-lane offsets, computed once
//   read(tile, ks, t)         the 16 bytes lane (row = lane % 16, k-group = lane / 16) feeds to the
//                             MFMA for 16-row tile t of this wavefront and k-step ks (0 | 1)
// [rows][128 B] tiles with the (row & 7) chunk swizzle: one ds_read_b128.  K-step 1 uses logical
// chunk q + 4, i.e. the k-step 0 offset ^ 64; tiles 16 rows apart add 2048.
struct RowFrag {
  uint32_t fo;
  __device__ __forceinline__ RowFrag(int lane, int wave_row0)
      : fo(addr::rowfrag_base(lane, wave_row0)) {}
  __device__ __forceinline__ uint4_t read(const uint8_t* tile, int ks, int t) const {
    return *(const uint4_t*)(tile + addr::rowfrag_off(fo, ks, t));
  }
};

// [128 k][BN bytes] tiles (a [K, N] int8 source copied as it is, n contiguous): the operand needs 16
// consecutive k of one n per lane, which ds_read_b64_tr_b8 delivers straight from this layout.
// Semantics of the instruction (established by probing): each group of 16 lanes supplies 16 row
// addresses R[0..15] (8 bytes each); lane j of the group receives bytes b = 0..7 =
// R[2b + j/8][j % 8].  With lane i supplying the row of k = i/2 at columns n_t + 8*(i%2), lane j
// receives k = 0..7 of column n_t + j: two such reads (k 0..7, 8..15) make one operand.
// 16-byte chunks of a k row are XOR-swizzled so that the 32 rows a wavefront touches per read, and
// the row-wise fill stores, spread over all banks.
template <int BN>
__device__ __forceinline__ int kn_swz(int k) {
  return addr::kn_swz<BN>(k);
}
template <int BN>
struct KNFrag8 {
  typedef int v2i_t __attribute__((ext_vector_type(2)));
  uint32_t off[4];
  __device__ __forceinline__ KNFrag8(int lane, int wave_row0) {
    // the swizzle of a k row is unchanged by the +8 (second read) and +64 (k-step) row offsets
#pragma unroll
    for (int t = 0; t < 4; ++t) off[t] = addr::knfrag_off<BN>(lane, wave_row0, t);
  }
  __device__ __forceinline__ uint4_t read(const uint8_t* tile, int ks, int t) const {
    typedef __attribute__((address_space(3))) v2i_t* lds_ptr;
    const uint8_t* p = tile + off[t] + ks * 64 * BN;
    const v2i_t lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_ptr)(p));
    const v2i_t hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_ptr)(p + 8 * BN));
    return uint4_t{(uint32_t)lo.x, (uint32_t)lo.y, (uint32_t)hi.x, (uint32_t)hi.y};
  }
};

// [64 k][BN columns] tiles of 16-bit values (a [K, N] source copied as it is): ds_read_b64_tr_b16 hands every lane four
// consecutive k of its column, two reads make an operand (addressing and the instruction's semantics: gemm_addr.h).
template <int BN>
struct KNFrag16 {
  typedef short v4s_t __attribute__((ext_vector_type(4)));
  uint32_t off[4];
  __device__ __forceinline__ KNFrag16(int lane, int wave_col0) {
#pragma unroll
    for (int t = 0; t < 4; ++t) off[t] = addr::kn16frag_off<BN>(lane, wave_col0, t);
  }
  __device__ __forceinline__ uint4_t read(const uint8_t* tile, int ks, int t) const {
    typedef __attribute__((address_space(3))) v4s_t* lds_ptr;
    const uint8_t* p = tile + off[t] + ks * 32 * 2 * BN;
    const uint2_t lo = bitcast<uint2_t>(__builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p)));
    const uint2_t hi = bitcast<uint2_t>(__builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 4 * 2 * BN)));
    return uint4_t{lo.x, lo.y, hi.x, hi.y};
  }
};

// ---- MFMA wrappers ----------------------------------------------------------------------
struct MmaF16 {
  typedef float4_t acc_t;
  static __device__ __forceinline__ acc_t mma(const uint4_t& a, const uint4_t& b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(bitcast<half8_t>(a), bitcast<half8_t>(b), c, 0, 0, 0);
  }
};
struct MmaBF16 {
  typedef float4_t acc_t;
  static __device__ __forceinline__ acc_t mma(const uint4_t& a, const uint4_t& b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(bitcast<bf16x8_t>(a), bitcast<bf16x8_t>(b), c, 0, 0, 0);
  }
};
struct MmaI8 {
  typedef int4_t acc_t;
  static __device__ __forceinline__ acc_t mma(const uint4_t& a, const uint4_t& b, acc_t c) {
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(bitcast<int4_t>(a), bitcast<int4_t>(b), c, 0, 0, 0);
  }
};

// ---- tile loaders -----------------------------------------------------------------------
// A loader owns a Regs type (what one thread keeps in flight for one stage) and
//   Loader(params, batch, row0, rows_total, tid)   per-thread offsets, computed once
//   gload<TAIL>(regs, kt)                          issue the global loads of stage kt; TAIL = the
//                                                  stage may extend past the end of K (zero fill)
//   lstore_piece(regs, lds_tile, pc, np)           convert + store piece pc of np of the stage
//   lstore(regs, lds_tile)                         the whole stage
// Store work is counted in UNITS; piece pc handles the units u with u * np / UNITS == pc.
// Loaders assume a matrix (one batch) spans less than 4 GiB (checked on the host).

// Plain row-major [rows, k_bytes] source (activations of every kind, weights stored [N, K]).
template <int ROWS, int NT>
struct RowLoader {
  typedef RowFrag Frag;
  static constexpr bool DIRECT = false;
  static constexpr bool PREFETCH2 = false;
  static constexpr int SLOTS = ROWS * 8;  // 16-byte chunks per stage
  static constexpr int PASSES = (SLOTS + NT - 1) / NT;
  static constexpr bool PARTIAL = SLOTS % NT != 0;
  static constexpr int UNITS = PASSES;
  static_assert(PASSES == 1 || (NT / 8) % 8 == 0, "pass stride must keep the swizzle phase");
  struct Params {
    const uint8_t* base;   // element [0, 0] of batch 0
    int64_t ld;            // row pitch in bytes
    int64_t batch_stride;  // bytes between batches
    int64_t k_bytes;       // bytes of K per row (multiple of 16)
  };
  struct Regs {
    uint4_t v[PASSES];
  };
  const uint8_t* base;    // uniform
  uint32_t voff[PASSES];  // per lane: row * ld + chunk * 16
  uint32_t loff;          // per lane: LDS offset of pass 0
  int kb_lane;            // chunk * 16
  int k_bytes;
  bool active;  // this thread has a slot in the (partial) last pass

  __device__ __forceinline__ RowLoader(const Params& p, int batch, int row0, int rows_total, int tid)
      : base(p.base + batch * p.batch_stride + (int64_t)row0 * p.ld), k_bytes((int)p.k_bytes) {
    const int rows_valid = rows_total - row0;
    const int chunk = tid & 7;
    kb_lane = chunk * 16;
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      int row = (ps * NT + tid) >> 3;
      row = row < rows_valid ? row : rows_valid - 1;  // clamp: loads stay in bounds, results are masked later
      voff[ps] = (uint32_t)row * (uint32_t)p.ld + (uint32_t)kb_lane;
    }
    loff = (uint32_t)lds_off(tid >> 3, chunk);
    active = !PARTIAL || ((PASSES - 1) * NT + tid) < SLOTS;
  }

  template <bool TAIL>
  __device__ __forceinline__ void gload(Regs& r, int kt, uint8_t* /*lds_next*/ = nullptr) const {
    const uint8_t* sb = base + (int64_t)kt * kStageBytes;
    if (!TAIL) {
#pragma unroll
      for (int ps = 0; ps < PASSES; ++ps) r.v[ps] = *(const uint4_t*)(sb + voff[ps]);
    } else {
      const bool ok = kt * kStageBytes + kb_lane < k_bytes;
#pragma unroll
      for (int ps = 0; ps < PASSES; ++ps) {
        uint4_t v = *(const uint4_t*)(ok ? sb + voff[ps] : base + (voff[ps] - kb_lane));
        if (!ok) v = uint4_t{0u, 0u, 0u, 0u};
        r.v[ps] = v;
      }
    }
  }
  __device__ __forceinline__ void lstore_piece(const Regs& r, uint8_t* lds, int pc, int np) const {
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      if (ps * np / UNITS != pc) continue;
      if (PARTIAL && ps == PASSES - 1 && !active) continue;
      *(uint4_t*)(lds + loff + ps * (NT / 8) * kStageBytes) = r.v[ps];
    }
  }
  __device__ __forceinline__ void lstore(const Regs& r, uint8_t* lds) const { lstore_piece(r, lds, 0, 1); }
};

// Same source and LDS layout as RowLoader, but full stages travel global -> LDS without passing
// through registers (global_load_lds_dwordx4): one wavefront instruction fills 8 rows x 128 B =
// 1 KB of the tile, lane l landing at byte 16*l of that KB.  The chunk swizzle is therefore applied
// on the global side: the lane that lands on (row, physical chunk pc) fetches logical chunk
// pc ^ (row & 7) of that row (the 8 lanes of a row still cover one 128-byte line).  A partial
// last stage needs zero fill, which the direct path cannot do; it goes through registers.
template <int ROWS, int NT>
struct RowLoaderDirect {
  typedef RowFrag Frag;
  static constexpr bool DIRECT = true;
  static constexpr bool PREFETCH2 = false;
  static constexpr int WAVES = NT / 64;
  static constexpr int INSTR = ROWS / 8;          // wavefront-instructions per stage
  static constexpr int PER_WAVE = INSTR / WAVES;  // ... per wavefront
  static constexpr int UNITS = PER_WAVE;
  static_assert(ROWS % 8 == 0 && INSTR % WAVES == 0 && PER_WAVE >= 1, "tile does not split into whole wavefront loads");
  typedef typename RowLoader<ROWS, NT>::Params Params;
  struct Regs {
    uint4_t v[PER_WAVE];
    bool pending;  // a register-path (tail) stage waits to be stored
  };
  const uint8_t* base;      // uniform
  uint32_t voff[PER_WAVE];  // per lane: row * ld + logical chunk * 16
  uint32_t wave_off;        // uniform: LDS offset of this wavefront's first KB
  uint32_t lane_off;        // lane * 16
  int kb_lane, k_bytes;

  __device__ __forceinline__ RowLoaderDirect(const Params& p, int batch, int row0, int rows_total, int tid)
      : base(p.base + batch * p.batch_stride + (int64_t)row0 * p.ld), k_bytes((int)p.k_bytes) {
    const int rows_valid = rows_total - row0;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    wave_off = addr::direct_lds_off(0, wave, 0, WAVES);
    lane_off = addr::direct_lds_off(lane, 0, 0, WAVES);
    kb_lane = addr::rd_chunk(lane) * 16;  // rows of one instruction start at a multiple of 8
#pragma unroll
    for (int j = 0; j < PER_WAVE; ++j) voff[j] = addr::rd_voff(lane, wave, j, WAVES, rows_valid, (uint32_t)p.ld);
  }

  // The direct loads are written as inline assembly on purpose: while a compiler-visible direct load is
  // outstanding the compiler turns every LDS wait into a wait for everything (it must assume the load
  // may also return through the LDS counter), which serialises the operand reads and LDS stores of the
  // whole stage.  The kernel waits for them by hand (wait_direct) before the barrier that publishes
  // the buffer.
  template <bool TAIL>
  __device__ __forceinline__ void gload(Regs& r, int kt, uint8_t* lds_next) const {
    typedef __attribute__((address_space(3))) uint8_t* lptr_t;
    if (!TAIL) {
      r.pending = false;
      const uint8_t* sb = uniform_ptr(base + (int64_t)kt * kStageBytes);
      const uint32_t l0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lptr_t)lds_next + wave_off);
#pragma unroll
      for (int j = 0; j < PER_WAVE; ++j)
        asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(l0 + addr::direct_lds_off(0, 0, j, WAVES)),
                     "v"(voff[j]), "s"(sb)
                     : "memory");
    } else {
      r.pending = true;
      const uint8_t* sb = base + (int64_t)kt * kStageBytes;
      const bool ok = kt * kStageBytes + kb_lane < k_bytes;
#pragma unroll
      for (int j = 0; j < PER_WAVE; ++j) {
        uint4_t v = *(const uint4_t*)(ok ? sb + voff[j] : base + (voff[j] - kb_lane));
        if (!ok) v = uint4_t{0u, 0u, 0u, 0u};
        r.v[j] = v;
      }
    }
  }
  __device__ __forceinline__ void lstore_piece(const Regs& r, uint8_t* lds, int pc, int np) const {
    if (!r.pending) return;
#pragma unroll
    for (int j = 0; j < PER_WAVE; ++j) {
      if (j * np / UNITS != pc) continue;
      *(uint4_t*)(lds + wave_off + addr::direct_lds_off(0, 0, j, WAVES) + lane_off) = r.v[j];
    }
  }
  __device__ __forceinline__ void lstore(const Regs& r, uint8_t* lds) const { lstore_piece(r, lds, 0, 1); }
};

// int8 source stored [K, N] (N contiguous): rows of k are copied unchanged into a [128 k][BN] LDS
// tile; the transposition happens in the operand read (KNFrag8).
struct I8KNParams {
  const uint8_t* base;  // B[0, 0] of batch 0
  int64_t ld;           // bytes per k row (= N)
  int64_t batch_stride;
  int64_t k_total;  // K
};

// The tile is filled by direct global -> LDS loads: one wavefront instruction covers
// 1024 / BN consecutive k rows; the lane landing on (k, physical chunk pc) fetches logical chunk
// pc ^ kn_swz(k) of that k row.  A partial last stage (rows past K must read as zero) goes through
// registers.
template <int BN, int NT>
struct I8KNLoaderDirect {
  typedef KNFrag8<BN> Frag;
  static constexpr bool DIRECT = true;
  static constexpr bool PREFETCH2 = false;
  static constexpr int CH = BN / 16;              // 16-byte chunks per k row
  static constexpr int KPI = 64 / CH;             // k rows per wavefront instruction
  static constexpr int WAVES = NT / 64;
  static constexpr int INSTR = kStageBytes / KPI;  // wavefront instructions per stage
  static constexpr int PER_WAVE = INSTR / WAVES;
  static constexpr int UNITS = PER_WAVE;
  static_assert(INSTR % WAVES == 0 && PER_WAVE >= 1, "tile does not split into whole wavefront loads");
  typedef I8KNParams Params;
  struct Regs {
    uint4_t v[PER_WAVE];
    bool pending;
  };
  const uint8_t* base;
  uint32_t voff[PER_WAVE];  // per lane: k * ld + logical chunk * 16
  uint32_t wave_off, lane_off;
  int k_lane;  // k row of this lane inside instruction 0 of wavefront 0
  int wave, k_total;

  __device__ __forceinline__ I8KNLoaderDirect(const Params& p, int batch, int col0, int cols_total, int tid)
      : base(p.base + batch * p.batch_stride + col0), k_total((int)p.k_total) {
    const int cols_valid = cols_total - col0;
    const int lane = tid & 63;
    wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    wave_off = addr::direct_lds_off(0, wave, 0, WAVES);
    lane_off = addr::direct_lds_off(lane, 0, 0, WAVES);
    k_lane = lane / CH;
#pragma unroll
    for (int j = 0; j < PER_WAVE; ++j) voff[j] = addr::kn_voff<BN>(lane, wave, j, WAVES, cols_valid, (uint32_t)p.ld);
    ld_ = (uint32_t)p.ld;
  }
  uint32_t ld_;

  template <bool TAIL>
  __device__ __forceinline__ void gload(Regs& r, int kt, uint8_t* lds_next) const {
    typedef __attribute__((address_space(3))) uint8_t* lptr_t;
    if (!TAIL) {
      r.pending = false;
      const uint8_t* sb = uniform_ptr(base + (int64_t)kt * kStageBytes * ld_);
      const uint32_t l0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lptr_t)lds_next + wave_off);
#pragma unroll
      for (int j = 0; j < PER_WAVE; ++j)
        asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(l0 + addr::direct_lds_off(0, 0, j, WAVES)),
                     "v"(voff[j]), "s"(sb)
                     : "memory");
    } else {
      r.pending = true;
      const uint8_t* sb = base + (int64_t)kt * kStageBytes * ld_;
#pragma unroll
      for (int j = 0; j < PER_WAVE; ++j) {
        const int k = addr::kn_k<BN>(0, wave, j, WAVES) + k_lane;
        const bool ok = kt * kStageBytes + k < k_total;
        uint4_t v = *(const uint4_t*)(ok ? sb + voff[j] : base + (voff[j] - (uint32_t)k * ld_));
        if (!ok) v = uint4_t{0u, 0u, 0u, 0u};
        r.v[j] = v;
      }
    }
  }
  __device__ __forceinline__ void lstore_piece(const Regs& r, uint8_t* lds, int pc, int np) const {
    if (!r.pending) return;
#pragma unroll
    for (int j = 0; j < PER_WAVE; ++j) {
      if (j * np / UNITS != pc) continue;
      *(uint4_t*)(lds + wave_off + addr::direct_lds_off(0, 0, j, WAVES) + lane_off) = r.v[j];
    }
  }
  __device__ __forceinline__ void lstore(const Regs& r, uint8_t* lds) const { lstore_piece(r, lds, 0, 1); }
};

// 16-bit source stored [K, N], N a multiple of 8 (16-byte chunks): the tile is filled by direct global -> LDS loads, one
// wavefront instruction per 512 / BN consecutive k rows; a partial last stage (rows past K must read as zero) goes
// through registers.  Other N go through the register loader (H16KNLoader).
struct H16KNParams {
  const uint8_t* base;  // B[0, 0] of batch 0
  int64_t ld;           // bytes per k row (= 2 N)
  int64_t batch_stride;
  int64_t k_total;
};
template <int BN, int NT>
struct H16KNLoaderDirect {
  typedef KNFrag16<BN> Frag;
  static constexpr bool DIRECT = true;
  static constexpr bool PREFETCH2 = false;
  static constexpr int CH = BN / 8;     // 16-byte chunks per k row
  static constexpr int KPI = 64 / CH;   // k rows per wavefront instruction
  static constexpr int WAVES = NT / 64;
  static constexpr int INSTR = 64 / KPI;  // 64 k rows per stage
  static constexpr int PER_WAVE = INSTR / WAVES;
  static constexpr int UNITS = PER_WAVE;
  static_assert(INSTR % WAVES == 0 && PER_WAVE >= 1, "tile does not split into whole wavefront loads");
  typedef H16KNParams Params;
  struct Regs {
    uint4_t v[PER_WAVE];
    bool pending;
  };
  const uint8_t* base;
  uint32_t voff[PER_WAVE];
  uint32_t wave_off, lane_off, ld_;
  int k_lane, wave, k_total;
  __device__ __forceinline__ H16KNLoaderDirect(const Params& p, int batch, int col0, int cols_total, int tid)
      : base(p.base + batch * p.batch_stride + (int64_t)col0 * 2), ld_((uint32_t)p.ld), k_total((int)p.k_total) {
    const int lane = tid & 63;
    wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    wave_off = addr::direct_lds_off(0, wave, 0, WAVES);
    lane_off = addr::direct_lds_off(lane, 0, 0, WAVES);
    k_lane = lane / CH;
#pragma unroll
    for (int j = 0; j < PER_WAVE; ++j) voff[j] = addr::kn16_voff<BN>(lane, wave, j, WAVES, cols_total - col0, ld_);
  }
  template <bool TAIL>
  __device__ __forceinline__ void gload(Regs& r, int kt, uint8_t* lds_next) const {
    typedef __attribute__((address_space(3))) uint8_t* lptr_t;
    if (!TAIL) {
      r.pending = false;
      const uint8_t* sb = uniform_ptr(base + (int64_t)kt * 64 * ld_);
      const uint32_t l0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lptr_t)lds_next + wave_off);
#pragma unroll
      for (int j = 0; j < PER_WAVE; ++j)
        asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(l0 + addr::direct_lds_off(0, 0, j, WAVES)), "v"(voff[j]),
                     "s"(sb)
                     : "memory");
    } else {
      r.pending = true;
      const uint8_t* sb = base + (int64_t)kt * 64 * ld_;
#pragma unroll
      for (int j = 0; j < PER_WAVE; ++j) {
        const int k = addr::kn16_k<BN>(0, wave, j, WAVES) + k_lane;
        const bool ok = kt * 64 + k < k_total;
        uint4_t v = *(const uint4_t*)(ok ? sb + voff[j] : base + (voff[j] - (uint32_t)k * ld_));  // (rows past K: row 0, then zeroed)
        if (!ok) v = uint4_t{0u, 0u, 0u, 0u};
        r.v[j] = v;
      }
    }
  }
  __device__ __forceinline__ void lstore_piece(const Regs& r, uint8_t* lds, int pc, int np) const {
    if (!r.pending) return;
#pragma unroll
    for (int j = 0; j < PER_WAVE; ++j) {
      if (j * np / UNITS != pc) continue;
      *(uint4_t*)(lds + wave_off + addr::direct_lds_off(0, 0, j, WAVES) + lane_off) = r.v[j];
    }
  }
  __device__ __forceinline__ void lstore(const Regs& r, uint8_t* lds) const { lstore_piece(r, lds, 0, 1); }
};

// ---- epilogues ----------------------------------------------------------------------------
// store(m, n, acc): acc holds C[m, n .. n+3]
struct EpiFloat {  // fp32 accumulators -> f16 / bf16 / f32
  struct Params {
    void* C;
    int64_t ldc;
    int64_t batch_stride;  // elements
    int out_dtype;
  };
  Params p;
  int64_t boff;
  __device__ __forceinline__ EpiFloat(const Params& pp, int batch) : p(pp), boff(batch * pp.batch_stride) {}
  // staged epilogue interface: element size of C, the four outputs of one accumulator in C's type (x, y only for
  // 16-bit types), the byte address of C[m, n], and the row pitch in elements
  static constexpr bool STAGED = true;
  __device__ __forceinline__ int out_bytes() const { return p.out_dtype == TLQ_F32 ? 4 : 2; }
  __device__ __forceinline__ int64_t pitch() const { return p.ldc; }
  __device__ __forceinline__ uint8_t* addr_of(int m, int n) const {
    return (uint8_t*)p.C + (boff + (int64_t)m * p.ldc + n) * out_bytes();
  }
  __device__ __forceinline__ uint4_t pack(int /*m*/, int /*n*/, const float4_t& acc, int /*M*/, int /*N*/) const {
    if (p.out_dtype == TLQ_F32) return bitcast<uint4_t>(acc);
    uint4_t o{0u, 0u, 0u, 0u};
    if (p.out_dtype == TLQ_F16) {
      half_t h[4] = {(half_t)acc[0], (half_t)acc[1], (half_t)acc[2], (half_t)acc[3]};
      const uint2_t u = bitcast<uint2_t>(h);
      o.x = u.x, o.y = u.y;
    } else {
      o.x = pack_bf16x2(acc[0], acc[1]);
      o.y = pack_bf16x2(acc[2], acc[3]);
    }
    return o;
  }
  __device__ __forceinline__ void store(int m, int n, const float4_t& acc, int M, int N) const {
    if (m >= M || n >= N) return;
    const int64_t idx = boff + (int64_t)m * p.ldc + n;
    if (n + 3 < N) {
      if (p.out_dtype == TLQ_F32) {
        *(float4_t*)((float*)p.C + idx) = acc;
      } else if (p.out_dtype == TLQ_F16) {
        half_t h[4] = {(half_t)acc[0], (half_t)acc[1], (half_t)acc[2], (half_t)acc[3]};
        *(uint2_t*)((half_t*)p.C + idx) = bitcast<uint2_t>(h);
      } else {
        uint2_t o;
        o.x = pack_bf16x2(acc[0], acc[1]);
        o.y = pack_bf16x2(acc[2], acc[3]);
        *(uint2_t*)((uint16_t*)p.C + idx) = o;
      }
    } else {
      for (int i = 0; i < 4 && n + i < N; ++i) store_out(p.C, idx + i, acc[i], p.out_dtype);
    }
  }
};

struct EpiAtomicAdd {  // fp32 accumulators added into C (split-K: several work-groups share an output tile)
  struct Params {
    float* C;
    int64_t ldc;
  };
  Params p;
  __device__ __forceinline__ EpiAtomicAdd(const Params& pp, int /*split*/) : p(pp) {}
  static constexpr bool STAGED = false;  // atomic adds go out element by element
  __device__ __forceinline__ int out_bytes() const { return 4; }
  __device__ __forceinline__ int64_t pitch() const { return p.ldc; }
  __device__ __forceinline__ uint8_t* addr_of(int, int) const { return nullptr; }
  __device__ __forceinline__ uint4_t pack(int, int, const float4_t&, int, int) const { return uint4_t{0u, 0u, 0u, 0u}; }
  __device__ __forceinline__ void store(int m, int n, const float4_t& acc, int M, int N) const {
    if (m >= M || n >= N) return;
    float* c = p.C + (int64_t)m * p.ldc + n;
    for (int i = 0; i < 4 && n + i < N; ++i) unsafeAtomicAdd(c + i, acc[i]);
  }
};

struct EpiAtomicAddI32 {  // int32 accumulators added into C (split-K; integer adds commute, so the sum is exact in any order)
  struct Params {
    int32_t* C;
    int64_t ldc;
  };
  Params p;
  __device__ __forceinline__ EpiAtomicAddI32(const Params& pp, int /*split*/) : p(pp) {}
  static constexpr bool STAGED = false;
  __device__ __forceinline__ int out_bytes() const { return 4; }
  __device__ __forceinline__ int64_t pitch() const { return p.ldc; }
  __device__ __forceinline__ uint8_t* addr_of(int, int) const { return nullptr; }
  __device__ __forceinline__ uint4_t pack(int, int, const int4_t&, int, int) const { return uint4_t{0u, 0u, 0u, 0u}; }
  __device__ __forceinline__ void store(int m, int n, const int4_t& acc, int M, int N) const {
    if (m >= M || n >= N) return;
    int32_t* c = p.C + (int64_t)m * p.ldc + n;
    for (int i = 0; i < 4 && n + i < N; ++i) atomicAdd(c + i, acc[i]);
  }
};

struct EpiInt32 {  // raw int32 accumulators
  struct Params {
    int32_t* C;
    int64_t ldc;
    int64_t batch_stride;
  };
  Params p;
  int64_t boff;
  __device__ __forceinline__ EpiInt32(const Params& pp, int batch) : p(pp), boff(batch * pp.batch_stride) {}
  static constexpr bool STAGED = true;
  __device__ __forceinline__ int out_bytes() const { return 4; }
  __device__ __forceinline__ int64_t pitch() const { return p.ldc; }
  __device__ __forceinline__ uint8_t* addr_of(int m, int n) const { return (uint8_t*)(p.C + boff + (int64_t)m * p.ldc + n); }
  __device__ __forceinline__ uint4_t pack(int, int, const int4_t& acc, int, int) const { return bitcast<uint4_t>(acc); }
  __device__ __forceinline__ void store(int m, int n, const int4_t& acc, int M, int N) const {
    if (m >= M || n >= N) return;
    const int64_t idx = boff + (int64_t)m * p.ldc + n;
    if (n + 3 < N) {
      *(int4_t*)(p.C + idx) = acc;
    } else {
      for (int i = 0; i < 4 && n + i < N; ++i) p.C[idx + i] = acc[i];
    }
  }
};

// int32 accumulators -> fp32 (RNE) -> * scale_a[m] -> * scale_b[n] -> out dtype (RNE); each
// multiply rounds to fp32 on its own (the file is compiled with -ffp-contract=off).
struct EpiRescale {
  struct Params {
    void* C;
    int64_t ldc;
    int64_t batch_stride;  // elements of C per batch
    const float* scale_a;  // [batch * M] or null
    const float* scale_b;  // [n_scale_b] or null
    int64_t n_scale_b;     // 1 or N
    int64_t scale_a_batch_stride;
    int out_dtype;
  };
  Params p;
  int64_t boff;
  const float* sa;
  __device__ __forceinline__ EpiRescale(const Params& pp, int batch)
      : p(pp), boff(batch * pp.batch_stride), sa(pp.scale_a ? pp.scale_a + batch * pp.scale_a_batch_stride : nullptr) {}
  // m < M and n < N
  __device__ __forceinline__ float4_t scaled(int m, int n, const int4_t& acc, int N) const {
    float4_t f;
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = (float)acc[i];
    if (sa) {
      const float a = sa[m];
#pragma unroll
      for (int i = 0; i < 4; ++i) f[i] = f[i] * a;
    }
    if (p.scale_b) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int nn = (n + i < N) ? n + i : N - 1;
        f[i] = f[i] * (p.n_scale_b == 1 ? p.scale_b[0] : p.scale_b[nn]);
      }
    }
    return f;
  }
  __device__ __forceinline__ EpiFloat as_float() const {
    EpiFloat::Params fp{p.C, p.ldc, 0, p.out_dtype};
    EpiFloat ef(fp, 0);
    ef.boff = boff;
    return ef;
  }
  static constexpr bool STAGED = true;
  static constexpr bool HAS_SCALES = true;
  // The scales a lane needs for its TN x TM accumulators: one per row tile, four per column tile.  Fetched in one go
  // (indices clamped into the arrays) before the tile is packed: fetched per accumulator, each tile paid a memory round
  // trip per use (measured on 256 x 256 int8 tiles: 18.7 us of fixed cost per tile against 7 us for the plain epilogue).
  template <int TM, int TN>
  struct Scales {
    float a[TM];
    float4_t b[TN];
  };
  template <int TM, int TN>
  __device__ __forceinline__ Scales<TM, TN> load_scales(int m_base, int n_base, int lane, int M, int N) const {
    Scales<TM, TN> s;
    const int r16 = lane & 15, q = lane >> 4;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      int m = m_base + tm * 16 + r16;
      m = m < M ? m : M - 1;
      s.a[tm] = sa ? sa[m] : 1.0f;
    }
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const int n = n_base + tn * 16 + q * 4;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int nn = (n + i < N) ? n + i : N - 1;
        s.b[tn][i] = p.scale_b ? (p.n_scale_b == 1 ? p.scale_b[0] : p.scale_b[nn]) : 1.0f;
      }
    }
    return s;
  }
  // same arithmetic as scaled(): convert, times the row scale, times the column scales (absent scales multiply by an
  // exact 1.0f, which changes nothing)
  __device__ __forceinline__ uint4_t pack_scaled(int m, int n, const int4_t& acc, float a, const float4_t& b, int M, int N) const {
    float4_t f;
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = ((float)acc[i] * a) * b[i];
    return as_float().pack(m, n, f, M, N);
  }
  __device__ __forceinline__ int out_bytes() const { return p.out_dtype == TLQ_F32 ? 4 : 2; }
  __device__ __forceinline__ int64_t pitch() const { return p.ldc; }
  __device__ __forceinline__ uint8_t* addr_of(int m, int n) const { return as_float().addr_of(m, n); }
  __device__ __forceinline__ uint4_t pack(int m, int n, const int4_t& acc, int M, int N) const {
    if (m >= M || n >= N) return uint4_t{0u, 0u, 0u, 0u};  // never stored; keeps the scale loads inside their arrays
    return as_float().pack(m, n, scaled(m, n, acc, N), M, N);
  }
  __device__ __forceinline__ void store(int m, int n, const int4_t& acc, int M, int N) const {
    if (m >= M || n >= N) return;
    as_float().store(m, n, scaled(m, n, acc, N), M, N);
  }
};

// Writes a wavefront's accumulators (TN x TM MFMA tiles: lane (r16, q) holds C[m = 16 tm + r16][n = 16 tn + 4 q + 0..3])
// to C.  Stored straight from the registers a lane would write 8 (16-bit output) or 16 bytes of a row while its 15
// neighbours write to 15 other rows: 32-byte pieces of 16 different cache lines per instruction, which the memory system
// does not merge back into whole lines (measured: 1.8-2.5 x the output bytes written, and an epilogue of 17 us for a
// 32 MB output).  So the tile takes a detour through a wavefront-private piece of LDS (free once the main loop is
// over): accumulators are written as [row][128 B] with the operand tiles' chunk swizzle, 128 bytes of output per row
// and pass, and read back row-wise, 16 bytes per lane, eight lanes per row -- every store instruction then writes eight
// whole 128-byte lines.  Needs 16-byte aligned rows of C (pitch and N multiples of 16 bytes); otherwise, and for
// tilings whose wavefront rows are shorter than 128 bytes, the direct path is used.
// epilogues with per-row / per-column scales fetch them once per wavefront tile (HAS_SCALES); the others pack directly
template <class Epi, typename = void>
struct EpiHasScales : std::false_type {};
template <class Epi>
struct EpiHasScales<Epi, std::enable_if_t<Epi::HAS_SCALES>> : std::true_type {};
struct NoScales {};
template <class Epi, int TM, int TN>
__device__ __forceinline__ auto fetch_scales(const Epi& epi, int m_base, int n_base, int lane, int M, int N) {
  if constexpr (EpiHasScales<Epi>::value)
    return epi.template load_scales<TM, TN>(m_base, n_base, lane, M, N);
  else
    return NoScales{};
}
template <class Epi, class S, class A>
__device__ __forceinline__ uint4_t pack_with(const Epi& epi, const S& sc, int m, int n, const A& acc, int tm, int tn, int M, int N) {
  if constexpr (EpiHasScales<Epi>::value)
    return epi.pack_scaled(m, n, acc, sc.a[tm], sc.b[tn], M, N);
  else
    return epi.pack(m, n, acc, M, N);
}

template <class Epi, int TM, int TN, class Acc, class S>
__device__ __forceinline__ void write_tile_with(const Epi& epi, const S& scales, Acc (&acc)[TN][TM], uint8_t* region, int lane, int m_base,
                                                int n_base, int M, int N) {
  const int r16 = lane & 15, q = lane >> 4;
  const int osz = epi.out_bytes();
  bool staged = false;
  // (whole passes of 128 output bytes per row only: a wavefront tile whose width is not a multiple of a pass goes the direct way)
  if constexpr (Epi::STAGED)
    staged = ((epi.pitch() * osz) & 15) == 0 && ((N * osz) & 15) == 0 && TN * 16 * osz >= 128 && (TN * 16 * osz) % 128 == 0;
  if (!staged) {
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) epi.store(m_base + tm * 16 + r16, n_base + tn * 16 + q * 4, acc[tn][tm], M, N);
    return;
  }
  auto run = [&](auto osz_tag) {
    constexpr int OSZ = decltype(osz_tag)::value;
    constexpr int TNP = 128 / (16 * OSZ);  // MFMA tile columns per pass: 128 bytes of output per row
    if constexpr (TN % TNP == 0) {
#pragma unroll
      for (int p0 = 0; p0 < TN; p0 += TNP) {
#pragma unroll
        for (int t = 0; t < TNP; ++t)
#pragma unroll
          for (int tm = 0; tm < TM; ++tm) {
            const int row = tm * 16 + r16;
            const uint4_t v = pack_with<Epi>(epi, scales, m_base + row, n_base + (p0 + t) * 16 + q * 4, acc[p0 + t][tm], tm, p0 + t, M, N);
            const int byte = (t * 16 + q * 4) * OSZ;  // offset inside the 128-byte row of this pass
            uint8_t* dst = region + lds_off(row, byte >> 4) + (byte & 15);
            if (OSZ == 2)
              *(uint2_t*)dst = uint2_t{v.x, v.y};
            else
              *(uint4_t*)dst = v;
          }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < 2 * TM; ++j) {
          const int row = j * 8 + (lane >> 3), chunk = lane & 7;
          const uint4_t v = *(const uint4_t*)(region + lds_off(row, chunk));
          const int m = m_base + row, n = n_base + p0 * 16 + chunk * (16 / OSZ);
          if (m < M && n < N) *(uint4_t*)epi.addr_of(m, n) = v;
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        __builtin_amdgcn_wave_barrier();  // the next pass overwrites the rows
      }
    }
  };
  if (osz == 2)
    run(std::integral_constant<int, 2>{});
  else
    run(std::integral_constant<int, 4>{});
}

// the same with the scales fetched here (callers with registers to spare fetch them before their main loop instead)
template <class Epi, int TM, int TN, class Acc>
__device__ __forceinline__ void write_tile(const Epi& epi, Acc (&acc)[TN][TM], uint8_t* region, int lane, int m_base, int n_base,
                                           int M, int N) {
  const auto scales = fetch_scales<Epi, TM, TN>(epi, m_base, n_base, lane, M, N);
  write_tile_with<Epi, TM, TN>(epi, scales, acc, region, lane, m_base, n_base, M, N);
}

// Work-group -> tile.  Consecutive hardware ids are dealt round-robin to the 8 XCDs; give
// every XCD a contiguous range of logical tiles, and order the tiles of a matrix in bands of four
// tile rows walked column by column, so that the 32 tiles an XCD runs at a time form a 4 x 8
// block: they share four activation panels and eight weight panels in that XCD's L2 instead of
// two and sixteen (a third less traffic past the L2 on square problems).  The band height is a launch
// parameter.
struct TileCoord {
  int batch, m0, n0;
};
template <int BM, int BN>
__device__ __forceinline__ TileCoord tile_of_block(int tiles_m, int tiles_n, int GM) {
  const int total = gridDim.x;
  int lid = blockIdx.x;
  if ((total & 7) == 0) lid = (lid & 7) * (total >> 3) + (lid >> 3);
  const int per_batch = tiles_m * tiles_n;
  TileCoord t;
  t.batch = lid / per_batch;
  const int rem = lid - t.batch * per_batch;
  const int band = rem / (GM * tiles_n);
  const int r = rem - band * (GM * tiles_n);
  const int rows = tiles_m - band * GM < GM ? tiles_m - band * GM : GM;  // the last band may be lower
  t.m0 = (band * GM + r % rows) * BM;
  t.n0 = (r / rows) * BN;
  return t;
}

// ---- the kernel -----------------------------------------------------------------------------
template <class Mma, class AL, class WL, class Epi, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM* WN * 64, (WM * WN >= 8 ? 2 : 1)) void gemm_mfma_kernel(
    typename AL::Params pa, typename WL::Params pw, typename Epi::Params pe, int M, int N, int kt_each, int k_tail,
    int tiles_m, int tiles_n, int band_rows, int kt_total) {
  constexpr int TM = BM / WM / 16;  // 16-row activation tiles per wave
  constexpr int TN = BN / WN / 16;  // 16-row weight tiles per wave
  constexpr int A_TILE = BM * kStageBytes, W_TILE = BN * kStageBytes;
  extern __shared__ __align__(16) uint8_t smem[];
  uint8_t* const ldsA0 = smem;
  uint8_t* const ldsW0 = smem + 2 * A_TILE;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15;
  const int q = lane >> 4;
  const int wave_m0 = (wave % WM) * (BM / WM);
  const int wave_n0 = (wave / WM) * (BN / WN);
  const TileCoord tc = tile_of_block<BM, BN>(tiles_m, tiles_n, band_rows);
  const int m0 = tc.m0, n0 = tc.n0, batch = tc.batch;
  // K slices (the "batches" of a split launch) may be uneven: the last one holds what is left of kt_total stages
  const int KT = kt_total > 0 && kt_total - batch * kt_each < kt_each ? kt_total - batch * kt_each : kt_each;

  AL al(pa, batch, m0, M, tid);
  WL wl(pw, batch, n0, N, tid);
  typename AL::Regs ra;
  typename WL::Regs rw;

  typename Mma::acc_t acc[TN][TM];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn)
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = typename Mma::acc_t{0, 0, 0, 0};

  const typename AL::Frag fragA(lane, wave_m0);
  const typename WL::Frag fragW(lane, wave_n0);

  // One stage: 2 k-steps x TN weight tiles x TM activation tiles of MFMAs on buffer CUR.  When
  // FILL, the conversion + LDS stores of the next stage (already in registers) are cut into
  // 2*TN pieces and one piece follows every TM MFMAs, so that the VALU / LDS-store work runs in
  // the shadow of the MFMAs (this wavefront's and the other wavefront's on the same SIMD).
  constexpr int NP = 2 * TN;  // pieces per stage
  // first pieces: activation stores (none when they travel directly), the rest: weight conversion
  constexpr int NPA = AL::DIRECT ? 0 : NP / 2;
  // hand-issued direct loads are invisible to the compiler's wait insertion
  auto wait_direct = [&]() {
    if (AL::DIRECT || WL::DIRECT) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  };
  auto stage = [&](int cur, auto fill_tag) {
    constexpr bool FILL = decltype(fill_tag)::value;
    const uint8_t* la = ldsA0 + cur * A_TILE;
    const uint8_t* lw = ldsW0 + cur * W_TILE;
    uint8_t* na = ldsA0 + (cur ^ 1) * A_TILE;
    uint8_t* nw = ldsW0 + (cur ^ 1) * W_TILE;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      uint4_t wf[TN], af[TM];
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) wf[tn] = fragW.read(lw, ks, tn);
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) af[tm] = fragA.read(la, ks, tm);
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = Mma::mma(wf[tn], af[tm], acc[tn][tm]);
        if (FILL) {
          const int pc = ks * TN + tn;
          if (pc < NPA)
            al.lstore_piece(ra, na, pc, NPA);
          else
            wl.lstore_piece(rw, nw, pc - NPA, NP - NPA);
          if (NPA == 0 && pc == 0) al.lstore(ra, na);  // direct loader: only a partial last stage stores anything
        }
      }
    }
  };

  // prologue: stage 0 into buffer 0
  if (KT == 1 && k_tail) {
    al.template gload<true>(ra, 0, ldsA0);
    wl.template gload<true>(rw, 0, ldsW0);
  } else {
    al.template gload<false>(ra, 0, ldsA0);
    wl.template gload<false>(rw, 0, ldsW0);
  }
  al.lstore(ra, ldsA0);
  wl.lstore(rw, ldsW0);
  wait_direct();
  __syncthreads();

  const int last_full = k_tail ? KT - 2 : KT - 1;  // highest stage that is whole (loadable without the tail path)
  if constexpr (WL::PREFETCH2) {
    // Converting loader: the weights of stage t+1 are converted during stage t from registers that were
    // loaded during stage t-1, so the conversion never waits on a load issued in the same stage and the
    // compiler is free to spread it between the MFMAs.  Costs one more register set (a few registers).
    typename WL::Regs rw_next;
    auto wload = [&](typename WL::Regs& r, int s) {
      if (s < KT) {
        if (k_tail && s == KT - 1)
          wl.template gload<true>(r, s, ldsW0 + (s & 1) * W_TILE);
        else
          wl.template gload<false>(r, s, ldsW0 + (s & 1) * W_TILE);
      }
    };
    wload(rw_next, 1);
    for (int kt = 0; kt + 1 < KT; ++kt) {
      rw = rw_next;
      wload(rw_next, kt + 2);
      if (k_tail && kt + 1 == KT - 1)
        al.template gload<true>(ra, kt + 1, ldsA0 + ((kt + 1) & 1) * A_TILE);
      else
        al.template gload<false>(ra, kt + 1, ldsA0 + ((kt + 1) & 1) * A_TILE);
      stage(kt & 1, std::true_type{});
      wait_direct();
      __syncthreads();
    }
  } else {
    // Stages 0 .. KT-2 compute and fill.  Only the load of stage KT-1 can be a partial stage.
    int kt = 0;
    for (; kt + 1 <= last_full; ++kt) {
      al.template gload<false>(ra, kt + 1, ldsA0 + ((kt + 1) & 1) * A_TILE);
      wl.template gload<false>(rw, kt + 1, ldsW0 + ((kt + 1) & 1) * W_TILE);
      stage(kt & 1, std::true_type{});
      wait_direct();
      __syncthreads();
    }
    if (kt + 1 < KT) {  // the partial last stage
      al.template gload<true>(ra, kt + 1, ldsA0 + ((kt + 1) & 1) * A_TILE);
      wl.template gload<true>(rw, kt + 1, ldsW0 + ((kt + 1) & 1) * W_TILE);
      stage(kt & 1, std::true_type{});
      wait_direct();
      __syncthreads();
      ++kt;
    }
  }
  if (KT > 0) stage((KT - 1) & 1, std::false_type{});

  Epi epi(pe, batch);
  // the operand tiles are no longer needed once every wavefront is past its last stage: each wavefront then stages its
  // outputs through its own TM * 16 rows x 128 B of LDS
  static_assert(WM * WN * TM * 16 * kStageBytes <= 2 * (A_TILE + W_TILE), "staging area exceeds the operand tiles");
  if constexpr (Epi::STAGED) __syncthreads();
  write_tile<Epi, TM, TN>(epi, acc, smem + wave * (TM * 16 * kStageBytes), lane, m0 + wave_m0, n0 + wave_n0, M, N);
}

// Host-side launcher: sets the dynamic LDS size and launches one work-group per tile.
// tile rows per band of the work-group -> tile order, for tuning runs (0 = each launcher's own choice: measured best
// were 2 for the int8 kernels, 4 for the plain 16-bit GEMM and 8 for the fused W4A16 kernel; 1 = plain row-major)
extern thread_local int g_gemm_band_rows;

// 128 x 128 or 256 x 256 output tiles?  The large tiles need half the operand traffic per product and run 1.25 - 1.3 PFLOP/s
// (bf16) where the small ones reach 1.0 - 1.07, both with every CU busy; but one large tile per CU is a whole round, and
// a launch with 128 of them leaves half the machine idle.  Fill = tiles / (rounds x CUs); the small tiles are taken
// when their fill, weighted by 0.72, beats the large tiles' (measured on fifteen shapes: every choice this rule makes
// was the faster one, e.g. M = 2048, N = 4096: 248 against 322 us; M = 3072, N = 4096: 99 (large) against 111 us).
inline double tile_fill(int64_t batch, int64_t M, int64_t N, int64_t tile) {
  int cus = tlq_device_cu_count();
  if (cus <= 0) cus = 256;
  const int64_t t = batch * ceil_div(M, tile) * ceil_div(N, tile);
  return (double)t / (double)(ceil_div(t, (int64_t)cus) * cus);
}
// (`weight`: pace of the small tiles relative to the large ones at equal fill; 0.65 for the fused W4A16 tile kernel,
// whose small tiles also dequantise every weight twice as often.)
inline bool prefer_small_tiles(int64_t batch, int64_t M, int64_t N, double weight = 0.72) {
  if (M <= 128) return true;
  return tile_fill(batch, M, N, 128) * weight > tile_fill(batch, M, N, 256);
}

// ---- K slices of a one-batch GEMM with few activation rows ---------------------------------------------
// The count of non-empty slices when every slice but the last has ceil(stages / count) stages.
inline int64_t whole_slices(int64_t stages, int64_t count) {
  if (count > stages) count = stages;
  if (count < 1) count = 1;
  return ceil_div(stages, ceil_div(stages, count));
}

// Number of K slices (whole 128-byte stages) for one batch of M rows against N weight rows of k_bytes bytes: 1 = do not
// cut.  Tiles are 32 x 128 (M <= 32) or 128 x 128.  The estimate behind the choice, in microseconds: an under-filled
// launch is paced by what one work-group streams, (BM + BN) * k_bytes at about 40 GB/s (times `pace` for a slower
// loader); s slices divide that and add the cost of their sums -- a pass over one [M, N] 32-bit matrix per slice
// (`buffers`), or atomic adds into one matrix at about 10 ns per thousand.  `forced` > 1 is a requested count.
inline int slice_choice(int64_t M, int64_t N, int64_t k_bytes, bool buffers, double pace, int forced) {
  if (k_bytes % kStageBytes != 0) return 1;
  const int64_t stages = k_bytes / kStageBytes;
  if (forced > 1) return (int)whole_slices(stages, forced);
  const int tile = M <= 32 ? 32 : 128;
  const int64_t tiles = ceil_div(M, (int64_t)tile) * ceil_div(N, (int64_t)128);
  int cus = tlq_device_cu_count();
  if (cus <= 0) cus = 256;
  const int64_t places = (int64_t)cus * (tile == 32 ? 4 : 2);  // work-groups the machine holds at once (LDS per work-group)
  if (tiles * 2 > places) return 1;
  const double one = (double)(tile + 128) * (double)k_bytes / 40e3 * pace;
  const double mn = (double)M * (double)N;
  double best = one;
  int64_t best_s = 1;
  for (int64_t want = 2; want * tiles <= places && want * 2 <= stages; ++want) {
    const int64_t sl = whole_slices(stages, want);
    if (sl != want) continue;  // the same cut as a smaller request
    const double sums = buffers ? 3.0 + (double)sl * mn * 8 / 4e6 : 5.0 + (double)sl * mn / 100e3;
    const double t = one * (double)ceil_div(stages, sl) / (double)stages + sums;
    if (t < best * (best_s == 1 ? 0.85 : 0.97)) best = t, best_s = sl;
  }
  return (int)best_s;
}

template <class Mma, class AL, class WL, class Epi, int BM, int BN, int WM, int WN>
int launch_gemm(const typename AL::Params& pa, const typename WL::Params& pw, const typename Epi::Params& pe,
                int64_t batch, int64_t M, int64_t N, int64_t k_bytes, hipStream_t st, const char* what, int band_rows = 4,
                int kt_total = 0) {
  // kt_total > 0: the batches are slices of K of k_bytes each (whole stages), the last one shorter: kt_total stages in all
  auto kern = gemm_mfma_kernel<Mma, AL, WL, Epi, BM, BN, WM, WN>;
  constexpr int lds_bytes = 2 * (BM + BN) * kStageBytes;  // two stages
  static bool attr_set = false;  // per instantiation; idempotent, so a race only repeats the call
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) {
      set_error("%s: cannot reserve %d bytes of LDS: %s", what, lds_bytes, hipGetErrorString(e));
      return 1;
    }
    attr_set = true;
  }
  const int64_t tiles_m = ceil_div(M, BM), tiles_n = ceil_div(N, BN);
  const int64_t blocks = batch * tiles_m * tiles_n;
  if (blocks <= 0) return 0;
  if (blocks > 0x7fffffff) {
    set_error("%s: too many tiles", what);
    return 1;
  }
  const int KT = (int)ceil_div(k_bytes, kStageBytes);
  const int k_tail = (k_bytes % kStageBytes) != 0;
  if (kt_total > 0 && (k_tail || (batch - 1) * KT >= kt_total || batch * KT < kt_total)) {
    set_error("%s: %lld slices of %d stages do not cover %d stages", what, (long long)batch, KT, kt_total);
    return 1;
  }
  kern<<<(unsigned)blocks, WM * WN * 64, lds_bytes, st>>>(pa, pw, pe, (int)M, (int)N, KT, k_tail, (int)tiles_m,
                                                          (int)tiles_n, g_gemm_band_rows > 0 ? g_gemm_band_rows : band_rows, kt_total);
  char detail[96];
  snprintf(detail, sizeof(detail), "gemm_mfma_kernel %dx%d tiles, two stages%s", BM, BN, WL::DIRECT ? "" : ", weights through registers");
  return check_launch(what, detail) ? 0 : 1;
}

}  // namespace tlq
