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

// ---- 16-bit source stored [K, N] (N contiguous): a stage is 64 k rows of BN columns (BN = 256 | 128, rows of 2 BN bytes),
// copied as it is; the operand read transposes (ds_read_b64_tr_b16: lane i of a group of 16 supplies 8 bytes R[i]; lane j
// receives the 16-bit values h = 0 .. 3 = R[4 h + j / 4][j % 4] -- established by probing).  With lane i supplying the row
// of k = i / 4 at columns n_t + 4 (i % 4), lane j receives k = 0 .. 3 of column n_t + j; a second read four rows on
// completes the eight values of an MFMA operand.  16-byte chunks of a k row are XOR-swizzled by an even number, which
// keeps the 8-byte halves of a chunk together and spreads the eight rows a half-wavefront touches over all banks.
__host__ __device__ inline int kn16_swz(int k) { return ((k & 3) << 1) | (((k >> 3) & 1) << 3); }
// one wavefront instruction covers 512 / BN consecutive k rows
template <int BN>
__host__ __device__ inline int kn16_k(int lane, int wave, int j, int waves) {
  static_assert(BN == 128 || BN == 256, "tile width");
  return (j * waves + wave) * (512 / BN) + lane / (BN / 8);
}
template <int BN>
__host__ __device__ inline uint32_t kn16_voff(int lane, int wave, int j, int waves, int cols_valid, uint32_t ld_bytes) {
  const int k = kn16_k<BN>(lane, wave, j, waves);
  const int pc = lane % (BN / 8);
  int colb = (pc ^ kn16_swz(k)) * 16;
  colb = colb < cols_valid * 2 ? colb : cols_valid * 2 - 16;  // whole chunks are clamped; those columns are masked at the store
  return (uint32_t)k * ld_bytes + (uint32_t)colb;
}
// operand read of column block t (16 columns) of a wavefront whose columns start at wave_col0; k-step ks adds 32 rows,
// the second read 4 rows (neither changes the swizzle)
template <int BN>
__host__ __device__ inline uint32_t kn16frag_off(int lane, int wave_col0, int t) {
  const int i = lane & 15, q = lane >> 4;
  const int krow = 8 * q + (i >> 2);
  const int chunk = (wave_col0 >> 3) + 2 * t + ((i & 3) >> 1);
  return (uint32_t)(krow * 2 * BN) + (uint32_t)((chunk ^ kn16_swz(krow)) << 4) + (uint32_t)(8 * (i & 1));
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

// ---- streaming W4A16 kernel for small and middle M (gemm_w4a16_stream.hip) ---------------------------------------
// One step is 128 values of K.  A work-group of 8 wavefronts owns 256 weight rows (wavefront w: rows 32 w .. 32 w + 31,
// two 16-row MFMA tiles) and 16 * TM activation rows.
// Packed weights: [16 rows][64 B] per MFMA tile, private to the wavefront.  One direct load covers a tile (lane l lands
// on row l / 4, 16-byte piece l % 4 and fetches logical piece (l % 4) ^ sw_swz(row)); the operand read of lane
// (row r16, k-group q) takes logical piece q: the four 32-bit words 4 q .. 4 q + 3 = values 32 q .. 32 q + 31 of the step.
// The swizzles of both tiles were chosen by measuring the 16-byte reads of eight wavefronts over whole families of
// layouts (every 4 x 4 bit matrix for the activations, 24 row orders x 256 piece swizzles for the weights): with
// pieces swizzled by row / 4 and chunks by the row number itself a read took 61 clocks instead of 37 in bank conflicts.
__host__ __device__ inline int sw_swz(int row) { return (row >> 1) & 3; }
__host__ __device__ inline int sw_row(int lane) { return lane >> 2; }
__host__ __device__ inline int sw_piece(int lane) { return (lane & 3) ^ sw_swz(sw_row(lane)); }
__host__ __device__ inline uint32_t sw_frag_off(int lane) {  // inside the 1 KB tile
  const int r16 = lane & 15, q = lane >> 4;
  return (uint32_t)(r16 * 64 + ((q ^ sw_swz(r16)) << 4));
}
// Activations: [16 TM rows][256 B], shared by the work-group.  Direct load I (of 4 TM) covers rows 4 I .. 4 I + 3 (lane
// l: row 4 I + l / 16, physical chunk l % 16, logical chunk (l % 16) ^ sa_swz(row)); lane (m = r16, k-group q) reads
// logical chunk 4 q + ks for MFMA k-step ks, i.e. the eight values that word 4 q + ks of the weights holds.
// sa_swz: the row number's low four bits rotated left by one.
__host__ __device__ inline int sa_swz(int row) { return ((row << 1) & 15) | ((row >> 3) & 1); }
__host__ __device__ inline int sa_row(int lane, int I) { return 4 * I + (lane >> 4); }
__host__ __device__ inline int sa_chunk(int lane, int I) { return (lane & 15) ^ sa_swz(sa_row(lane, I)); }
__host__ __device__ inline uint32_t sa_frag_off(int lane, int tm, int ks) {
  const int r16 = lane & 15, q = lane >> 4;
  return (uint32_t)((tm * 16 + r16) * 256 + (((4 * q + ks) ^ sa_swz(r16)) << 4));
}
// Ring of D steps: step s lives in slot s % D.  Every wavefront issues `per_step` load instructions per step, in
// step order, and loads retire in issue order: this wavefront's loads of step s have landed once at most the
// loads of the younger steps that were already issued are outstanding.  At the top of step s (before the loads of
// step s + D - 1 are issued) those are the steps s + 1 .. min(s + D - 2, last).
__host__ __device__ inline int stream_younger_steps(int s, int steps, int D) {
  const int last_issued = s + D - 2 < steps - 1 ? s + D - 2 : steps - 1;
  return last_issued - s > 0 ? last_issued - s : 0;
}

// ---- panel kernel for large M (gemm_w4a16_panel.hip): 128 activation rows x 512 weight rows per work-group ----------
// Steps of 128 values of K in two ring slots.  A slot is the activation tile [128 rows][256 B] (the streaming kernel's
// layout with eight 16-row tiles: direct load I = 8 j + wave, j = 0 .. 3, rows 4 I .. 4 I + 3) followed by the eight
// wavefronts' packed weights, four [16 rows][64 B] tiles each (wavefront w: weight rows 64 w + 16 tn + row).  Behind
// the ring every wavefront has two scale windows of 2 KB: [64 rows][8 groups] scales, then the same for zero points;
// lane l of the window's direct load fetches the eight groups (16 bytes) of row l.
constexpr int kPanelTM = 8, kPanelTN = 4;
constexpr uint32_t kPanelATile = 16 * kPanelTM * 256;
constexpr uint32_t kPanelSlot = kPanelATile + 8 * kPanelTN * 1024;
constexpr uint32_t kPanelScBuf = 2048;
__host__ __device__ inline uint32_t panel_a_lds(int wave, int j) { return (uint32_t)(j * 8 + wave) * 1024u; }
__host__ __device__ inline uint32_t panel_w_lds(int wave, int tn) { return kPanelATile + (uint32_t)(wave * kPanelTN + tn) * 1024u; }
__host__ __device__ inline uint32_t panel_sc_lds(int wave, int buf) { return 2 * kPanelSlot + (uint32_t)(wave * 2 + buf) * kPanelScBuf; }
__host__ __device__ inline uint32_t panel_sc_off(int row, int g) { return (uint32_t)(row * 16 + g * 2); }
// Source of a direct load = (first byte of the step in row 0) + block offset of the instruction (uniform) + lane offset.
// An instruction covers 16 weight rows (64 bytes per step and row) or 4 activation rows (256 bytes per step and row);
// with N % 16 == 0 and M % 4 == 0 it lies wholly inside the matrix or wholly outside, and an outside one repeats the
// last block of the matrix.
__host__ __device__ inline uint32_t panel_w_lane(int lane, int K) { return (uint32_t)sw_row(lane) * (uint32_t)(K >> 1) + (uint32_t)(sw_piece(lane) * 16); }
__host__ __device__ inline int64_t panel_w_block(int wave, int tn, int n0, int N, int K) {
  int n = n0 + wave * (16 * kPanelTN) + tn * 16;
  n = n + 16 <= N ? n : N - 16;
  return (int64_t)n * (K >> 1);
}
// lane l of activation load I = 8 j + wave: row 4 I + l / 16, logical chunk (l % 16) ^ sa_swz(that row); sa_swz depends on
// the row's low four bits = 4 (I % 4) + l / 16 only, and I % 4 = wave % 4 for every j
__host__ __device__ inline uint32_t panel_a_lane(int lane, int K) { return (uint32_t)(lane >> 4) * (uint32_t)K * 2u; }
__host__ __device__ inline uint32_t panel_a_chunk(int lane, int wave) { return (uint32_t)(((lane & 15) ^ sa_swz(4 * (wave & 3) + (lane >> 4))) * 16); }
__host__ __device__ inline int64_t panel_a_block(int wave, int j, int m0, int M, int K) {
  int m = m0 + 4 * (j * 8 + wave);
  m = m + 4 <= M ? m : M - 4;
  return (int64_t)m * K * 2;
}
// byte offset from element [0][first group of the window] of the scale / zero-point tensor [N][groups]
__host__ __device__ inline uint32_t panel_sc_voff(int lane, int wave, int n0, int N, int groups) {
  int n = n0 + wave * (16 * kPanelTN) + lane;
  n = n < N ? n : N - 1;
  return ((uint32_t)n * (uint32_t)groups) * 2u;
}

// ---- panel kernel with 256 activation rows (gemm_w4a16_panel256.hip): four wavefronts, 256 x 256 outputs per work-group
// A ring slot is the activation tile [256 rows][256 B] (sixteen 16-row tiles: direct load I = 4 j + wave, j = 0 .. 15, rows
// 4 I .. 4 I + 3) followed by the four wavefronts' packed weights, four [16 rows][64 B] tiles each.  Scales and zero
// points are gathered into registers: lane (row r16, k-group q) reads, for weight tile tn, the 2-byte value of row
// 64 wave + 16 tn + r16 and of the group its 32 values of the step lie in.
constexpr int kPanel2TM = 16, kPanel2TN = 4;
constexpr uint32_t kPanel2ATile = 16 * kPanel2TM * 256;
constexpr uint32_t kPanel2Slot = kPanel2ATile + 4 * kPanel2TN * 1024;
__host__ __device__ inline uint32_t panel2_a_lds(int wave, int j) { return (uint32_t)(j * 4 + wave) * 1024u; }
__host__ __device__ inline uint32_t panel2_w_lds(int wave, int tn) { return kPanel2ATile + (uint32_t)(wave * kPanel2TN + tn) * 1024u; }
__host__ __device__ inline int64_t panel2_a_block(int wave, int j, int m0, int M, int K) {
  int m = m0 + 4 * (j * 4 + wave);
  m = m + 4 <= M ? m : M - 4;
  return (int64_t)m * K * 2;
}
// byte offsets into a scale / zero-point tensor [N][groups] of 2-byte values: row block of the tile (uniform), the group of
// step `step` of the matrix (uniform), the lane's row and -- for groups of fewer than 128 values -- its k-group's group
__host__ __device__ inline int64_t panel2_sc_block(int wave, int tn, int n0, int N, int groups) {
  int n = n0 + wave * (16 * kPanel2TN) + tn * 16;
  n = n + 16 <= N ? n : N - 16;
  return (int64_t)n * groups * 2;
}
__host__ __device__ inline int64_t panel2_sc_step(int step, int gshift) { return (((int64_t)step << 7) >> gshift) * 2; }
__host__ __device__ inline uint32_t panel2_sc_lane(int lane, int groups, int gshift) {
  const int r16 = lane & 15, q = lane >> 4;
  return (uint32_t)(r16 * groups + ((q << 5) >> gshift)) * 2u;
}

// The kernel's schedule of a step of 64 slots (a slot = one activation tile against the wavefront's four weight tiles)
// for its three kinds of loads, and the two waits that follow from it.  Loads retire in issue order, so a wait for "at
// most n outstanding" stands for "all but the youngest n have landed".
//   slot  0 .. 15: one load each of the activation tile of step s + 1
//   slot 16 .. 23: one gather each of the scales / zero points of step s + 2
//   slot 58 .. 61: one load each of the wavefront's packed weights of step s + 2
// The wait in front of slot kPanel2WaitWSlot needs the packed weights of step s + 1 (issued one step earlier); the wait in
// front of slot kPanel2BarrierSlot needs the activation tile and the gathers issued in this step (the gathers are
// compiler-visible loads whose wait the compiler writes itself, for everything issued before: no load may be
// younger there), and the barrier behind it separates the last operand read of this step's tile (slot
// kPanel2BarrierSlot - 1 reads kPanel2Ahead - 1 slots ahead) from the first read of the next.
enum { kPanel2LoadNone = 0, kPanel2LoadA, kPanel2LoadScale, kPanel2LoadW };
constexpr int kPanel2Slots = 4 * kPanel2TM, kPanel2Ahead = 8;
constexpr int kPanel2WaitWSlot = 32, kPanel2BarrierSlot = kPanel2Slots - (kPanel2Ahead - 1);
// Packed word ks + 2 (of step s + 1 from phase 2 on) of weight tile wt is read in slot kPanel2WordSlot + wt of phase ks;
// the dequantiser constants of tile tn for step s + 1 are made in slot kPanel2ExpanderSlot + 4 tn, between the last piece of
// expansion that uses the old ones (slot 32 + 4 tn + 3) and the first that uses the new ones (slot 48 + 4 tn).
constexpr int kPanel2WordSlot = 8, kPanel2ExpanderSlot = 40, kPanel2WSlot = kPanel2BarrierSlot + 1;
__host__ __device__ constexpr int panel2_slot_load(int t) {
  return t < 16 ? kPanel2LoadA : t < 24 ? kPanel2LoadScale : (t >= kPanel2WSlot && t < kPanel2WSlot + kPanel2TN) ? kPanel2LoadW : kPanel2LoadNone;
}
__host__ __device__ constexpr int panel2_slot_load_index(int t) { return t < 16 ? t : t < 24 ? t - 16 : t - kPanel2WSlot; }
__host__ __device__ constexpr int panel2_loads_in(int t0, int t1) {  // loads issued in slots t0 .. t1 - 1 of one step
  int n = 0;
  for (int t = t0; t < t1; ++t) n += panel2_slot_load(t) != kPanel2LoadNone;
  return n;
}
constexpr int kPanel2WaitW = panel2_loads_in(kPanel2WSlot + kPanel2TN, kPanel2Slots) + panel2_loads_in(0, kPanel2WaitWSlot);
constexpr int kPanel2WaitA = panel2_loads_in(24, kPanel2BarrierSlot);
static_assert(kPanel2WaitW == 24 && kPanel2WaitA == 0 && kPanel2BarrierSlot == 57 && kPanel2WSlot + kPanel2TN <= kPanel2Slots,
              "the 256-row panel kernel's waits");

// ---- panel kernel for middle M (gemm_w4a16_panelm.hip): the 256-row kernel's four wavefronts and slot structure on
// 16 TM activation rows (TM = 4 or 8), 256 weight rows, a ring of D slots and the 128-row kernel's scale windows in LDS.
// Ring slot: activation tile [16 TM rows][256 B] (direct load I = 4 j + wave, j = 0 .. TM - 1, rows 4 I .. 4 I + 3, as in
// the 256-row kernel) + the four wavefronts' packed weights, four [16 rows][64 B] tiles each; behind the ring two scale
// windows per wavefront ([scales | zero points][64 rows][8 groups] of 2 bytes, see the 128-row kernel).
// A step of 128 values of K is 4 TM slots of four MFMAs (phase ks = slots ks TM .. ks TM + TM - 1).  Step s issues, in this
// order: the TM loads of the activation tile of step s + D - 1 (slots 0 .. TM - 1), at the first step of a scale window
// the two loads of the next window (slot TM), and from slot 2 TM + 1 on (the step's last packed word was read in phase 1)
// the four loads of the wavefront's packed weights of step s + D.  Loads retire in issue order; the two waits of a step are written for the FEWEST
// loads that can be younger than what they wait for (no window loads), so a step with window loads waits a little more:
//   slot 2 TM (its packed words are read from there on): the packed weights of step s + 1, issued in step s + 1 - D;
//        younger: steps s + 2 - D .. s - 1 whole and this step's activation loads
//   slot B: the activation tile of step s + 1, issued in step s + 2 - D; younger: that step's weights, steps
//        s + 3 - D .. s - 1 whole and all of this step's loads
// The barrier at slot B stands behind the last operand read of this step's tile (slot B - 1 reads AR - 1 slots ahead);
// slots B .. 4 TM - 1 read the first operands of step s + 1.  A window's loads, issued in step x, have landed behind the
// slot-B wait of step x + D - 2 and are first looked at at the top of the window's last step: a window must span D steps.
__host__ __device__ constexpr int panelm_depth(int tm) { return tm >= 16 ? 2 : tm >= 8 ? 3 : 4; }
__host__ __device__ constexpr int panelm_ahead(int tm) { return tm >= 8 ? 8 : 4; }
__host__ __device__ constexpr int panelm_slots(int tm) { return 4 * tm; }
__host__ __device__ constexpr int panelm_barrier_slot(int tm) { return 4 * tm - (panelm_ahead(tm) - 1); }
__host__ __device__ constexpr int panelm_w_slot(int tm) { return 2 * tm + 1; }
__host__ __device__ constexpr int panelm_step_loads(int tm) { return tm + kPanel2TN; }  // without window loads
__host__ __device__ constexpr int panelm_wait_w(int tm) { return (panelm_depth(tm) - 2) * panelm_step_loads(tm) + tm; }
__host__ __device__ constexpr int panelm_wait_a(int tm) { return kPanel2TN + (panelm_depth(tm) - 3) * panelm_step_loads(tm) + panelm_step_loads(tm); }
static_assert(panelm_depth(4) >= 3 && panelm_depth(8) >= 3, "the waits are written for rings of three slots or more");
static_assert(panelm_w_slot(4) + kPanel2TN <= panelm_barrier_slot(4) && panelm_w_slot(8) + kPanel2TN <= panelm_barrier_slot(8),
              "the weight loads are issued between the wait for the next step's weights and the barrier");
static_assert(panelm_wait_w(8) == 20 && panelm_wait_a(8) == 16 && panelm_wait_w(4) == 20 && panelm_wait_a(4) == 20, "the middle-M panel kernel's waits");
__host__ __device__ constexpr uint32_t panelm_a_tile(int tm) { return (uint32_t)tm * 4096u; }
__host__ __device__ constexpr uint32_t panelm_slot_bytes(int tm) { return panelm_a_tile(tm) + 4u * kPanel2TN * 1024u; }
__host__ __device__ constexpr uint32_t panelm_w_lds(int tm, int wave, int tn) { return panelm_a_tile(tm) + (uint32_t)(wave * kPanel2TN + tn) * 1024u; }
__host__ __device__ constexpr uint32_t panelm_sc_lds(int tm, int wave, int buf) {
  return (uint32_t)panelm_depth(tm) * panelm_slot_bytes(tm) + (uint32_t)(wave * 2 + buf) * kPanelScBuf;
}
__host__ __device__ constexpr uint32_t panelm_lds_bytes(int tm) { return panelm_sc_lds(tm, 4, 0); }
static_assert(panelm_lds_bytes(8) <= 160 * 1024 && panelm_lds_bytes(4) <= 160 * 1024, "ring and scale windows fit the CU's LDS");

// ---- decode kernel (1 .. 32 activation rows): wavefront w of a work-group owns values 256 s .. 256 s + 255 of K
// (s = chunk * waves + w) for every weight row.  A work item is one 16-row weight tile: two [16 rows][64 B] packed
// pieces (k-blocks kb = 0, 1 of the slice, 128 values each) plus the scales / zero points of the 16 rows for the
// slice.  Work-group b handles tiles b, b + grid, ...; the ts-th of them lives in ring slot ts % 3.
constexpr int kDecSlice = 256;
constexpr int kDecTileSlots = 3;
constexpr uint32_t kDecSlotBytes = 2048 + 512;  // packed piece kb 0 | kb 1 | scale dwords (256 B) | zero dwords (256 B)
__host__ __device__ inline int dec_red_buffers(int mt) { return mt == 1 ? 2 : 1; }
__host__ __device__ inline uint32_t dec_red_base() { return kDecTileSlots * kDecSlotBytes; }
__host__ __device__ inline uint32_t dec_wave_bytes(int mt) { return dec_red_base() + (uint32_t)(dec_red_buffers(mt) * mt) * 1024u; }
// Packed weights: the lane's byte offset from the first byte of (tile t, slice, kb = 0); kb = 1 is 64 bytes further.
// In the last tile the rows past N repeat row N - 1.
__host__ __device__ inline uint32_t dec_w_lane(int lane, int64_t t, int64_t N, int64_t K) {
  int64_t n = t * 16 + sw_row(lane);
  n = n < N ? n : N - 1;
  return (uint32_t)((n - t * 16) * (K / 2) + sw_piece(lane) * 16);
}
__host__ __device__ inline int64_t dec_w_base(int64_t t, int64_t K, int64_t k0) { return t * 16 * (K / 2) + k0 / 2; }
// Activations of a slice: per k-block kb and 16-row tile mt a [16 rows][256 B] block, fetched by four direct loads of
// 1 KB (load i: rows 4 i .. 4 i + 3, lane l on row 4 i + l / 16, physical 16-byte piece l % 16, which receives logical
// piece (l % 16) ^ (row % 8)) into 4 KB of the wavefront's LDS, and read back as MFMA operands: lane (m = r16, k-group q)
// takes logical piece 4 q + j for k-step j, the eight values 32 q + 8 j .. of the k-block.  Rows past M repeat the last.
// dec_a_off: byte offset of the lane's 16 bytes inside A.
__host__ __device__ inline int64_t dec_a_off(int lane, int mt, int kb, int i, int64_t M, int64_t K, int64_t k0) {
  const int row = 4 * i + (lane >> 4);
  int64_t m = mt * 16 + row;
  m = m < M ? m : M - 1;
  return (m * K + k0 + kb * 128) * 2 + (((lane & 15) ^ (row & 7)) << 4);
}
__host__ __device__ inline uint32_t dec_a_frag(int lane, int j) {  // inside the 4 KB block
  const int r16 = lane & 15, q = lane >> 4;
  return (uint32_t)(r16 * 256 + (((4 * q + j) ^ (r16 & 7)) << 4));
}
// Scales / zero points of a tile and slice: 256 / group values per row, fetched as dwords (two values).  Lane l of the
// first 16 nd lanes (nd dwords per row: 1, 2, 4 for groups of >= 128, 64, 32) gathers dword l / 16 of row l % 16 and
// lands on cell l of the 256-byte area.  dec_sc_elem: the first of the (up to) two values of that dword, for tile 0.
__host__ __device__ inline int dec_sc_dwords(int gshift) { return gshift >= 7 ? 1 : (gshift == 6 ? 2 : 4); }
__host__ __device__ inline int64_t dec_sc_elem(int lane, int64_t t, int64_t N, int64_t groups, int64_t k0, int gshift) {
  int64_t n = t * 16 + (lane & 15);
  n = n < N ? n : N - 1;
  return n * groups + (k0 >> gshift) + 2 * (lane >> 4);
}
// byte offset of the aligned dword that holds value `elem`
__host__ __device__ inline uint32_t dec_sc_off(int64_t elem) { return (uint32_t)((elem * 2) & ~(int64_t)3); }
// where lane (row r16, k-group q) finds the scale of its k-block kb: cell and half of the dword.  With groups of 256
// values or more one value serves the whole slice, and it is the low or high half according to its index in the tensor.
__host__ __device__ inline uint32_t dec_sc_cell(int lane, int kb, int gshift) {
  const int gi = gshift >= 8 ? 0 : ((kb * 128 + 32 * (lane >> 4)) >> gshift);
  return (uint32_t)(((gi >> 1) * 16 + (lane & 15)) * 4);
}
__host__ __device__ inline uint32_t dec_sc_half(int lane, int kb, int64_t groups, int64_t k0, int gshift) {
  if (gshift >= 8) return (uint32_t)((((int64_t)(lane & 15) * groups + (k0 >> gshift)) & 1) * 16);
  return (uint32_t)((((kb * 128 + 32 * (lane >> 4)) >> gshift) & 1) * 16);
}
// Loads still allowed in flight when k-block kb of the ts-th tile is read.  Per tile four loads are issued, in the order
// scale gather, zero gather, piece 0, piece 1; tile ts + 2 is issued at the top of iteration ts.
__host__ __device__ inline int dec_wait_count(int ts, int kb, int my_tiles) {
  int younger = my_tiles - 1 - ts;
  younger = younger > 2 ? 2 : younger;
  return 4 * younger + (kb == 0 ? 1 : 0);
}

// ---- GEMV ring kernel (one or two activation rows): a work-group owns `rows_per_block` consecutive weight rows, wavefront w
// takes rows w, w + waves, ... of them.  A packed row travels global -> LDS directly (no registers on the way), in
// `iters` instructions of 1 KB (lane l moves chunk 64 it + l, 16 bytes), into one of the wavefront's `depth` private
// slots; the activations and the work-group's scales / zero points are staged the same way, 16 bytes per lane.
// LDS map (bytes): [ring: waves x depth x iters KB][activations, mt x K x 2][scales][zero points], each area a whole number of KB
// so that a wave-wide instruction whose last lanes repeat the final piece still lands inside its area.
struct RingLayout {
  uint32_t ring, act, s, z, total;
};
__host__ __device__ inline uint32_t ring_kb(uint32_t bytes) { return (bytes + 1023u) & ~1023u; }
__host__ __device__ inline RingLayout ring_layout(int waves, int depth, int iters, int K, int rows_per_block, int groups, int mt) {
  RingLayout l;
  l.ring = 0;
  l.act = (uint32_t)(waves * depth * iters) * 1024u;
  l.s = l.act + ring_kb((uint32_t)(K * mt) * 2u);
  l.z = l.s + ring_kb((uint32_t)(rows_per_block * groups) * 2u);
  l.total = l.z + ring_kb((uint32_t)(rows_per_block * groups) * 2u);
  return l;
}
// weight instruction `it` of a row: byte offset of the lane's 16 bytes inside the row (chunks past the row repeat the
// last one: their lanes multiply by a zero scale), and the LDS offset of the instruction's 1 KB
__host__ __device__ inline uint32_t ring_w_voff(int lane, int it, int chunks) {
  int c = it * 64 + lane;
  c = c < chunks ? c : chunks - 1;
  return (uint32_t)c * 16u;
}
__host__ __device__ inline uint32_t ring_w_lds(int wave, int slot, int it, int depth, int iters) {
  return (uint32_t)((wave * depth + slot) * iters + it) * 1024u;
}
// staging: a tensor of `pieces` 16-byte pieces; the instruction that starts at piece p0 (a multiple of 64) moves piece
// min(p0 + lane, pieces - 1) to bytes 16 (p0 + lane) of the area
__host__ __device__ inline uint32_t ring_stage_voff(int p0, int lane, int pieces) {
  int p = p0 + lane;
  p = p < pieces ? p : pieces - 1;
  return (uint32_t)p * 16u;
}
// The activations (chunk c = 32 values = four 16-byte pieces) are read back by lane c, piece j of all lanes in one
// instruction: with the pieces in order, lanes four apart sit on the same banks and such a read takes 3.4 times its
// cycles (measured: 128 against 37 clocks).  Piece j of chunk c is therefore kept at position (j + c / 4) % 4 of the
// chunk's 64 bytes; the direct load fetches the piece that belongs at the position it lands on.
__host__ __device__ inline int ring_act_logical(int P) {  // the piece (4 c + j) that physical piece P of the area holds
  const int c = P >> 2;
  return (c << 2) | (((P & 3) - (c >> 2)) & 3);
}
__host__ __device__ inline uint32_t ring_act_lds(int c, int j) { return (uint32_t)(((c << 2) | ((j + (c >> 2)) & 3)) * 16); }
__host__ __device__ inline uint32_t ring_act_voff(int p0, int lane, int pieces) {  // pieces: a multiple of 4
  int P = p0 + lane;
  P = P < pieces ? P : pieces - 1;
  return (uint32_t)ring_act_logical(P) * 16u;
}
// rows of wavefront `wave`, and the loads it may leave in flight when it reads its i-th row (row i + depth is issued
// after row i has been read; loads retire in issue order)
__host__ __device__ inline int ring_my_rows(int rows, int wave, int waves) { return wave < rows ? (rows - wave + waves - 1) / waves : 0; }
__host__ __device__ inline int ring_younger_rows(int i, int my_rows, int depth) {
  const int y = my_rows - 1 - i;
  return y < depth - 1 ? y : depth - 1;
}

}  // namespace addr
}  // namespace tlq
