// Address arithmetic of the MFMA GEMM tile loaders, written as host-callable functions: the kernels
// (gemm_core.h, gemm_slots.h) take every global byte offset and every LDS offset of a direct
// global -> LDS load and of an operand-fragment read from here, and the host
// walker in gemm_addr_check.hip evaluates the same functions for every thread, stage and tile of a
// launch and compares them with the extents of the buffers, without a GPU.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tlq {
namespace addr {

constexpr int kStage = 128;  // bytes of K per stage and row

// [rows][128 B] operand tile: 16-byte chunk index XOR-swizzled by the row
__host__ __device__ inline int row_swz(int row) { return row & 7; }
__host__ __device__ inline int row_lds_off(int row, int chunk) { return row * kStage + ((chunk ^ row_swz(row)) << 4); }

// ---- direct row loader: one wavefront instruction moves 8 rows x 128 B = 1 KB ---------------------
// Instruction j of wavefront `wave` (of `waves`) covers tile rows (j * waves + wave) * 8 .. + 7; lane l
// lands at byte 16 * l of that KB, i.e. on row l / 8, physical chunk l % 8, and therefore fetches the
// logical chunk (l % 8) ^ (row & 7) of that row.
__host__ __device__ inline int rd_row(int lane, int wave, int j, int waves) { return (j * waves + wave) * 8 + (lane >> 3); }
__host__ __device__ inline int rd_chunk(int lane) { return (lane & 7) ^ ((lane >> 3) & 7); }
// byte offset from the tile's first row, stage 0; rows past the matrix are clamped to its last row
__host__ __device__ inline uint32_t rd_voff(int lane, int wave, int j, int waves, int rows_valid, uint32_t ld) {
  int row = rd_row(lane, wave, j, waves);
  row = row < rows_valid ? row : rows_valid - 1;
  return (uint32_t)row * ld + (uint32_t)(rd_chunk(lane) * 16);
}
// LDS byte offset inside the operand tile where that lane's 16 bytes land
__host__ __device__ inline uint32_t direct_lds_off(int lane, int wave, int j, int waves) {
  return (uint32_t)wave * 1024u + (uint32_t)(j * waves) * 1024u + (uint32_t)lane * 16u;
}
// operand fragment read of a [rows][128 B] tile: lane (row = lane % 16, k-group = lane / 16), 16-row tile t of the
// wavefront's rows, k-step ks
__host__ __device__ inline uint32_t rowfrag_base(int lane, int wave_row0) {
  return (uint32_t)row_lds_off(lane & 15, lane >> 4) + (uint32_t)(wave_row0 * kStage);
}
__host__ __device__ inline uint32_t rowfrag_off(uint32_t base, int ks, int t) {
  return (base ^ (uint32_t)(ks << 6)) + (uint32_t)(t * 16 * kStage);
}

// ---- int8 [K, N] source copied unchanged into a [128 k][BN] tile -------------------------------------
template <int BN>
__host__ __device__ inline int kn_swz(int k) {
  static_assert(BN == 128 || BN == 256, "tile width");
  return BN == 256 ? ((k & 7) | (((k >> 4) & 1) << 3)) : (((k >> 1) & 3) | (((k >> 4) & 1) << 2));
}
// one wavefront instruction covers 1024 / BN consecutive k rows
template <int BN>
__host__ __device__ inline int kn_k(int lane, int wave, int j, int waves) {
  return (j * waves + wave) * (1024 / BN) + lane / (BN / 16);
}
template <int BN>
__host__ __device__ inline uint32_t kn_voff(int lane, int wave, int j, int waves, int cols_valid, uint32_t ld) {
  const int k = kn_k<BN>(lane, wave, j, waves);
  const int pc = lane % (BN / 16);
  int col = (pc ^ kn_swz<BN>(k)) * 16;
  col = col < cols_valid ? col : cols_valid - 16;  // whole chunks are clamped; those columns are masked later
  return (uint32_t)k * ld + (uint32_t)col;
}
// ds_read_b64_tr_b8 fragment offsets (see KNFrag8): tile column block t of the wavefront
template <int BN>
__host__ __device__ inline uint32_t knfrag_off(int lane, int wave_row0, int t) {
  const int r16 = lane & 15, q = lane >> 4;
  const int krow = q * 16 + (r16 >> 1);
  const int sw = kn_swz<BN>(krow);
  return (uint32_t)(krow * BN + 8 * (r16 & 1)) + (uint32_t)((((wave_row0 >> 4) + t) ^ sw) << 4);
}

// ---- five-slot schedule (gemm_slots.h): tile t = 2 * stage (+ 1 for the weights) lives in slot t % 5 ----
constexpr int kSlots = 5;
__host__ __device__ inline int slot_of_tile(int t) { return t % kSlots; }
// The order in which one wavefront issues tile loads, waits, passes barriers and multiplies.  Loads retire in issue
// order; wait_tiles(keep) returns when all of this wavefront's loads but those of the youngest tile have landed
// (keep) or all of them (!keep).  The kernel and the host-side checker both run this function.
template <class Ops>
__host__ __device__ inline void slots_schedule(int KT, Ops& ops) {
  ops.issue_a(0);
  ops.issue_w(0);
  if (KT > 1) ops.issue_a(1);
  ops.wait_tiles(KT > 1);
  ops.barrier();
  for (int k = 0; k < KT; ++k) {
    if (k + 1 < KT) ops.issue_w(k + 1);  // into the slot of A(k - 1)
    if (k + 2 < KT) ops.issue_a(k + 2);  // into the slot of W(k - 1)
    ops.compute(k);
    if (k + 1 < KT) {
      ops.wait_tiles(k + 2 < KT);  // A(k + 1) and W(k + 1) are in; A(k + 2) may still be on its way
      ops.barrier();               // ... for every wavefront, and everyone has read the tiles of stage k
    }
  }
}

}  // namespace addr
}  // namespace tlq
