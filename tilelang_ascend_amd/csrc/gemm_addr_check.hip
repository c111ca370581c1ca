// Host-side walkers over the address arithmetic of the MFMA GEMM kernels (gemm_addr.h).  They evaluate, for every
// work-group, thread, load instruction and stage of a launch, the very functions the kernels use, and check that
//   * every global byte read lies inside the operand matrix,
//   * every direct load lands inside its LDS tile, every 16-byte cell of the tile is written exactly once, and holds
//     the (row, K chunk) that the operand-fragment read of that cell expects,
//   * the five-slot schedule never overwrites a tile that has not been multiplied and never multiplies a tile whose
//     loads were not waited for.
// No GPU is needed: these run in the CPU-only test suite and can be called before a launch.
#include <utility>
#include <vector>

#include "gemm_addr.h"
#include "tlq_common.h"

namespace tlq {
namespace {

#define CHECK_OR_FAIL(cond, ...) \
  do {                           \
    if (!(cond)) {               \
      set_error(__VA_ARGS__);    \
      return 1;                  \
    }                            \
  } while (0)

// Row-major operand [rows_total, k_bytes] (pitch = k_bytes), tiles of `tile_rows` rows loaded by `threads` threads.
int check_row_direct(int64_t rows_total, int64_t k_bytes, int tile_rows, int threads) {
  CHECK_OR_FAIL(tile_rows % 8 == 0 && threads % 64 == 0, "row loader: tile rows %d / threads %d", tile_rows, threads);
  const int waves = threads / 64, instr = tile_rows / 8;
  CHECK_OR_FAIL(instr % waves == 0 && instr >= waves, "row loader: %d load instructions do not split over %d wavefronts", instr, waves);
  CHECK_OR_FAIL(k_bytes > 0 && k_bytes % 16 == 0 && rows_total > 0, "row loader: bad matrix %lld x %lld bytes",
                (long long)rows_total, (long long)k_bytes);
  CHECK_OR_FAIL(rows_total * k_bytes < ((int64_t)1 << 32), "row loader: the matrix spans 4 GiB or more");
  const int per_wave = instr / waves;
  const int64_t extent = rows_total * k_bytes;
  const int KT = (int)((k_bytes + addr::kStage - 1) / addr::kStage);
  const bool tail = k_bytes % addr::kStage != 0;
  const int last_full = tail ? KT - 2 : KT - 1;
  const uint32_t ld = (uint32_t)k_bytes;
  std::vector<int> cell(tile_rows * 8);
  for (int64_t row0 = 0; row0 < rows_total; row0 += tile_rows) {
    const int rows_valid = (int)(rows_total - row0);
    std::fill(cell.begin(), cell.end(), -1);
    for (int wave = 0; wave < waves; ++wave)
      for (int j = 0; j < per_wave; ++j)
        for (int lane = 0; lane < 64; ++lane) {
          const uint32_t voff = addr::rd_voff(lane, wave, j, waves, rows_valid, ld);
          const int kb_lane = addr::rd_chunk(lane) * 16;
          // whole stages: direct loads of 16 bytes
          for (int kt = 0; kt <= last_full; ++kt) {
            const int64_t o = row0 * k_bytes + (int64_t)voff + (int64_t)kt * addr::kStage;
            CHECK_OR_FAIL(o >= 0 && o + 16 <= extent, "row loader: tile row %lld wave %d instr %d lane %d stage %d reads [%lld, +16) of %lld",
                          (long long)row0, wave, j, lane, kt, (long long)o, (long long)extent);
          }
          if (tail) {  // the partial stage: lanes past the end of the row re-read the row's first bytes and zero them
            const bool ok = (int64_t)(KT - 1) * addr::kStage + kb_lane < k_bytes;
            const int64_t o = row0 * k_bytes + (ok ? (int64_t)voff + (int64_t)(KT - 1) * addr::kStage : (int64_t)voff - kb_lane);
            CHECK_OR_FAIL(o >= 0 && o + 16 <= extent, "row loader: tail stage reads [%lld, +16) of %lld", (long long)o, (long long)extent);
          }
          // LDS side
          const uint32_t l = addr::direct_lds_off(lane, wave, j, waves);
          CHECK_OR_FAIL(l % 16 == 0 && l + 16 <= (uint32_t)tile_rows * addr::kStage, "row loader: LDS offset %u outside the %d-row tile", l,
                        tile_rows);
          CHECK_OR_FAIL(cell[l / 16] == -1, "row loader: LDS cell %u written twice", l / 16);
          const int row = addr::rd_row(lane, wave, j, waves), chunk = addr::rd_chunk(lane);
          CHECK_OR_FAIL(row < tile_rows, "row loader: row %d outside the tile", row);
          CHECK_OR_FAIL((uint32_t)addr::row_lds_off(row, chunk) == l, "row loader: (row %d, chunk %d) lands at %u, the operand read expects %d", row,
                        chunk, l, addr::row_lds_off(row, chunk));
          cell[l / 16] = row * 8 + chunk;
        }
    for (size_t c = 0; c < cell.size(); ++c) CHECK_OR_FAIL(cell[c] >= 0, "row loader: LDS cell %zu never written", c);
    // operand reads: every (16-row tile, k-step, lane) reads the cell that holds (its row, its chunk)
    for (int wave_row0 = 0; wave_row0 < tile_rows; wave_row0 += 16)
      for (int lane = 0; lane < 64; ++lane) {
        const uint32_t base = addr::rowfrag_base(lane, wave_row0);
        for (int ks = 0; ks < 2; ++ks) {
          const uint32_t off = addr::rowfrag_off(base, ks, 0);
          CHECK_OR_FAIL(off + 16 <= (uint32_t)tile_rows * addr::kStage, "operand read at %u outside the tile", off);
          const int want = (wave_row0 + (lane & 15)) * 8 + ks * 4 + (lane >> 4);
          CHECK_OR_FAIL(cell[off / 16] == want, "operand read (row0 %d lane %d k-step %d) finds cell %d, expects %d", wave_row0, lane, ks,
                        cell[off / 16], want);
        }
      }
  }
  return 0;
}

// int8 operand stored [K, N] (pitch N), tiles of BN columns x 128 k rows.
template <int BN>
int check_kn_direct(int64_t K, int64_t N, int threads) {
  CHECK_OR_FAIL(threads % 64 == 0, "[K,N] loader: threads %d", threads);
  const int waves = threads / 64, kpi = 1024 / BN, instr = addr::kStage / kpi;
  CHECK_OR_FAIL(instr % waves == 0 && instr >= waves, "[K,N] loader: %d load instructions do not split over %d wavefronts", instr, waves);
  CHECK_OR_FAIL(K > 0 && N >= 16 && N % 16 == 0, "[K,N] loader: bad matrix K=%lld N=%lld", (long long)K, (long long)N);
  CHECK_OR_FAIL(K * N < ((int64_t)1 << 32), "[K,N] loader: the matrix spans 4 GiB or more");
  const int per_wave = instr / waves;
  const int64_t extent = K * N;
  const int KT = (int)((K + addr::kStage - 1) / addr::kStage);
  const bool tail = K % addr::kStage != 0;
  const int last_full = tail ? KT - 2 : KT - 1;
  std::vector<int> cell(addr::kStage * BN / 16);
  for (int64_t col0 = 0; col0 < N; col0 += BN) {
    const int cols_valid = (int)(N - col0);
    std::fill(cell.begin(), cell.end(), -1);
    for (int wave = 0; wave < waves; ++wave)
      for (int j = 0; j < per_wave; ++j)
        for (int lane = 0; lane < 64; ++lane) {
          const uint32_t voff = addr::kn_voff<BN>(lane, wave, j, waves, cols_valid, (uint32_t)N);
          const int k = addr::kn_k<BN>(lane, wave, j, waves);
          CHECK_OR_FAIL(k < addr::kStage, "[K,N] loader: k row %d outside the stage", k);
          for (int kt = 0; kt <= last_full; ++kt) {
            const int64_t o = col0 + (int64_t)voff + (int64_t)kt * addr::kStage * N;
            CHECK_OR_FAIL(o >= 0 && o + 16 <= extent, "[K,N] loader: col %lld wave %d instr %d lane %d stage %d reads [%lld, +16) of %lld",
                          (long long)col0, wave, j, lane, kt, (long long)o, (long long)extent);
          }
          if (tail) {  // k rows past K re-read k row 0 of the stage base ... of the matrix (then zeroed)
            const bool ok = (int64_t)(KT - 1) * addr::kStage + k < K;
            const int64_t o = col0 + (ok ? (int64_t)voff + (int64_t)(KT - 1) * addr::kStage * N : (int64_t)voff - (int64_t)k * N);
            CHECK_OR_FAIL(o >= 0 && o + 16 <= extent, "[K,N] loader: tail stage reads [%lld, +16) of %lld", (long long)o, (long long)extent);
          }
          const uint32_t l = addr::direct_lds_off(lane, wave, j, waves);
          CHECK_OR_FAIL(l % 16 == 0 && l + 16 <= (uint32_t)addr::kStage * BN, "[K,N] loader: LDS offset %u outside the tile", l);
          CHECK_OR_FAIL(cell[l / 16] == -1, "[K,N] loader: LDS cell %u written twice", l / 16);
          const int pc = lane % (BN / 16);
          CHECK_OR_FAIL(l == (uint32_t)(k * BN + pc * 16), "[K,N] loader: lane lands at %u, not on (k %d, chunk %d)", l, k, pc);
          cell[l / 16] = k * (BN / 16) + (pc ^ addr::kn_swz<BN>(k));  // the logical 16-column chunk this cell holds
        }
    for (size_t c = 0; c < cell.size(); ++c) CHECK_OR_FAIL(cell[c] >= 0, "[K,N] loader: LDS cell %zu never written", c);
    // transposing operand reads: lane (r16, q) of column block t supplies the row of k = 16 q + r16 / 2 (+ 8 for the second
    // read, + 64 for k-step 1) at columns 16 (wave_row0 / 16 + t) + 8 (r16 % 2)
    for (int wave_row0 = 0; wave_row0 + 64 <= BN; wave_row0 += 64)
      for (int t = 0; t < 4; ++t)
        for (int lane = 0; lane < 64; ++lane)
          for (int ks = 0; ks < 2; ++ks)
            for (int h = 0; h < 2; ++h) {
              const uint32_t off = addr::knfrag_off<BN>(lane, wave_row0, t) + (uint32_t)(ks * 64 * BN + h * 8 * BN);
              CHECK_OR_FAIL(off + 8 <= (uint32_t)addr::kStage * BN, "[K,N] operand read at %u outside the tile", off);
              const int k = (lane >> 4) * 16 + ((lane & 15) >> 1) + 8 * h + 64 * ks;
              const int want = k * (BN / 16) + (wave_row0 >> 4) + t;
              CHECK_OR_FAIL(cell[off / 16] == want && (int)(off % 16) == 8 * (lane & 1), "[K,N] operand read (lane %d t %d) finds cell %d, expects %d",
                            lane, t, cell[off / 16], want);
            }
  }
  return 0;
}

// 16-bit [K, N] source in tiles of BN columns: every direct load inside the matrix (the partial last stage's register loads
// too), every LDS cell of the [64 k][2 BN bytes] tile written once, every transposing operand read on the chunk that holds
// its rows and columns, and no bank met twice by a half-wavefront.
template <int BN>
int check_kn16_direct(int64_t K, int64_t N, int threads) {
  CHECK_OR_FAIL(threads % 64 == 0, "[K,N] 16-bit loader: threads %d", threads);
  const int waves = threads / 64, kpi = 512 / BN, instr = 64 / kpi, RB = 2 * BN;
  CHECK_OR_FAIL(instr % waves == 0 && instr >= waves, "[K,N] 16-bit loader: %d load instructions do not split over %d wavefronts", instr, waves);
  CHECK_OR_FAIL(K >= 1 && N >= 8 && N % 8 == 0, "[K,N] 16-bit loader: bad matrix K=%lld N=%lld", (long long)K, (long long)N);
  CHECK_OR_FAIL(K * N * 2 < ((int64_t)1 << 32), "[K,N] 16-bit loader: the matrix spans 4 GiB or more");
  const int per_wave = instr / waves;
  const int64_t ld = N * 2, extent = K * ld;
  const int KT = (int)((K + 63) / 64);
  const bool tail = K % 64 != 0;
  const int last_full = tail ? KT - 2 : KT - 1;
  std::vector<int> cell(64 * (BN / 8));
  for (int64_t col0 = 0; col0 < N; col0 += BN) {
    const int cols_valid = (int)(N - col0);
    std::fill(cell.begin(), cell.end(), -1);
    for (int wave = 0; wave < waves; ++wave)
      for (int j = 0; j < per_wave; ++j)
        for (int lane = 0; lane < 64; ++lane) {
          const uint32_t voff = addr::kn16_voff<BN>(lane, wave, j, waves, cols_valid, (uint32_t)ld);
          const int k = addr::kn16_k<BN>(lane, wave, j, waves);
          CHECK_OR_FAIL(k < 64, "[K,N] 16-bit loader: k row %d outside the stage", k);
          CHECK_OR_FAIL((int64_t)voff - (int64_t)k * ld >= 0 && (int64_t)voff - (int64_t)k * ld + 16 <= ld - col0 * 2,
                        "[K,N] 16-bit loader: lane %d reads past the end of its k row", lane);
          for (int kt = 0; kt <= last_full; ++kt) {
            const int64_t o = col0 * 2 + (int64_t)voff + (int64_t)kt * 64 * ld;
            CHECK_OR_FAIL(o >= 0 && o + 16 <= extent, "[K,N] 16-bit loader: col %lld wave %d instr %d lane %d stage %d reads [%lld, +16) of %lld",
                          (long long)col0, wave, j, lane, kt, (long long)o, (long long)extent);
          }
          if (tail) {  // k rows past K re-read k row 0 of the matrix (then zeroed)
            const bool ok = (int64_t)(KT - 1) * 64 + k < K;
            const int64_t o = col0 * 2 + (ok ? (int64_t)voff + (int64_t)(KT - 1) * 64 * ld : (int64_t)voff - (int64_t)k * ld);
            CHECK_OR_FAIL(o >= 0 && o + 16 <= extent, "[K,N] 16-bit loader: tail stage reads [%lld, +16) of %lld", (long long)o, (long long)extent);
          }
          const uint32_t l = addr::direct_lds_off(lane, wave, j, waves);
          CHECK_OR_FAIL(l % 16 == 0 && l + 16 <= 64u * RB, "[K,N] 16-bit loader: LDS offset %u outside the tile", l);
          CHECK_OR_FAIL(cell[l / 16] == -1, "[K,N] 16-bit loader: LDS cell %u written twice", l / 16);
          const int pc = lane % (BN / 8);
          CHECK_OR_FAIL(l == (uint32_t)(k * RB + pc * 16), "[K,N] 16-bit loader: lane lands at %u, not on (k %d, chunk %d)", l, k, pc);
          cell[l / 16] = k * (BN / 8) + (pc ^ addr::kn16_swz(k));  // the logical chunk (8 columns) this cell holds
        }
    for (size_t c = 0; c < cell.size(); ++c) CHECK_OR_FAIL(cell[c] >= 0, "[K,N] 16-bit loader: LDS cell %zu never written", c);
    // operand reads: lane (i, q) of column block t supplies the row of k = 8 q + i / 4 (+ 4 for the second read, + 32 for
    // k-step 1) at columns wave_col0 + 16 t + 4 (i % 4) .. + 3
    for (int wave_col0 = 0; wave_col0 + 64 <= BN; wave_col0 += 64)
      for (int t = 0; t < 4; ++t)
        for (int ks = 0; ks < 2; ++ks)
          for (int h = 0; h < 2; ++h) {
            int bank_use[2][64] = {};
            for (int lane = 0; lane < 64; ++lane) {
              const uint32_t off = addr::kn16frag_off<BN>(lane, wave_col0, t) + (uint32_t)(ks * 32 * RB + h * 4 * RB);
              CHECK_OR_FAIL(off + 8 <= 64u * RB, "[K,N] 16-bit operand read at %u outside the tile", off);
              const int i = lane & 15, q = lane >> 4;
              const int k = 8 * q + (i >> 2) + 4 * h + 32 * ks;
              const int col = wave_col0 + 16 * t + 4 * (i & 3);
              const int want = k * (BN / 8) + col / 8;
              CHECK_OR_FAIL(cell[off / 16] == want && (int)(off % 16) == 2 * (col % 8),
                            "[K,N] 16-bit operand read (lane %d t %d) finds cell %d at byte %u, expects cell %d byte %d", lane, t, cell[off / 16],
                            off % 16, want, 2 * (col % 8));
              ++bank_use[lane >> 5][(off / 4) % 64];
              ++bank_use[lane >> 5][(off / 4 + 1) % 64];
            }
            for (int half = 0; half < 2; ++half)
              for (int b = 0; b < 64; ++b)
                CHECK_OR_FAIL(bank_use[half][b] <= 1, "[K,N] 16-bit operand read: bank %d used %d times by one half-wavefront", b, bank_use[half][b]);
          }
  }
  return 0;
}

// One wavefront running addr::slots_schedule; every tile is `loads_per_tile` load instructions of that wavefront.
struct SlotsSim {
  int loads_per_tile;
  std::vector<int> in_flight;  // tile ids of the load instructions not yet known to have landed, oldest first
  int owner[addr::kSlots];     // tile id whose data (or pending load) occupies the slot, -1 = empty
  bool landed[addr::kSlots];   // the owner's loads have been waited for
  bool published[addr::kSlots];  // ... and a barrier has passed since (every wavefront's part is in)
  std::vector<char> multiplied;  // per tile id
  int error = 0;
  char msg[160] = "";
  SlotsSim(int KT, int lpt) : loads_per_tile(lpt), multiplied(2 * KT, 0) {
    for (int s = 0; s < addr::kSlots; ++s) owner[s] = -1, landed[s] = published[s] = false;
  }
  void fail(const char* what, int t) {
    if (!error) snprintf(msg, sizeof(msg), "five-slot schedule: %s (tile %d)", what, t);
    error = 1;
  }
  void issue(int t) {
    const int s = addr::slot_of_tile(t);
    if (owner[s] >= 0 && !multiplied[owner[s]]) fail("a load overwrites a tile that was not multiplied yet", owner[s]);
    // other wavefronts may still be multiplying the previous owner unless a barrier followed its stage
    if (owner[s] >= 0 && multiplied[owner[s]] == 2) fail("a load overwrites a tile other wavefronts may still read", owner[s]);
    owner[s] = t, landed[s] = published[s] = false;
    for (int i = 0; i < loads_per_tile; ++i) in_flight.push_back(t);
  }
  void issue_a(int s) { issue(2 * s); }
  void issue_w(int s) { issue(2 * s + 1); }
  void wait_tiles(bool keep) {
    const size_t leave = keep ? 4 : 0;  // the literal operand of s_waitcnt vmcnt in the kernel
    while (in_flight.size() > leave) {
      const int t = in_flight.front();
      in_flight.erase(in_flight.begin());
      bool more = false;
      for (int u : in_flight) more |= (u == t);
      if (!more && owner[addr::slot_of_tile(t)] == t) landed[addr::slot_of_tile(t)] = true;
    }
  }
  void barrier() {
    for (int s = 0; s < addr::kSlots; ++s) published[s] = landed[s];
    for (auto& m : multiplied)
      if (m == 2) m = 1;  // everyone is past that stage now
  }
  void compute(int k) {
    for (int t = 2 * k; t <= 2 * k + 1; ++t) {
      const int s = addr::slot_of_tile(t);
      if (owner[s] != t) fail("the slot of a tile to be multiplied holds another tile", t);
      else if (!published[s]) fail("a tile is multiplied before its loads were waited for and published by a barrier", t);
      multiplied[t] = 2;  // 2 = by this wavefront, other wavefronts may lag until the next barrier
    }
  }
};

// Streaming W4A16 kernel: packed weights [N, K / 2], activations [M, K] of 2-byte values, 16 * tm activation rows and
// 256 weight rows per work-group, steps of 128 values of K.
int check_stream(int64_t M, int64_t N, int64_t K, int tm) {
  CHECK_OR_FAIL(tm == 2 || tm == 4 || tm == 6 || tm == 8, "stream: %d activation tiles", tm);
  CHECK_OR_FAIL(M > 0 && N > 0 && K >= 128 && K % 128 == 0, "stream: bad shape");
  CHECK_OR_FAIL(N * (K / 2) < ((int64_t)1 << 32) && M * K * 2 < ((int64_t)1 << 32), "stream: a matrix spans 4 GiB or more");
  const int64_t w_extent = N * (K / 2), a_extent = M * K * 2;
  const int steps = (int)(K / 128), la = tm / 2;
  std::vector<int> cell(1024 / 16), acell(tm * 16 * 16);
  for (int64_t n0 = 0; n0 < N; n0 += 256)
    for (int wave = 0; wave < 8; ++wave)
      for (int tn = 0; tn < 2; ++tn) {
        std::fill(cell.begin(), cell.end(), -1);
        for (int lane = 0; lane < 64; ++lane) {
          int64_t n = n0 + wave * 32 + tn * 16 + addr::sw_row(lane);
          n = n < N ? n : N - 1;
          const int64_t voff = n * (K / 2) + addr::sw_piece(lane) * 16;
          for (int st = 0; st < steps; ++st) {
            const int64_t o = voff + (int64_t)st * 64;
            CHECK_OR_FAIL(o >= 0 && o + 16 <= w_extent, "stream: weight load at [%lld, +16) of %lld", (long long)o, (long long)w_extent);
          }
          cell[lane] = addr::sw_row(lane) * 4 + addr::sw_piece(lane);  // the lane lands on 16-byte cell `lane` of the 1 KB tile
        }
        for (int lane = 0; lane < 64; ++lane) {
          const uint32_t off = addr::sw_frag_off(lane);
          CHECK_OR_FAIL(off % 16 == 0 && off + 16 <= 1024, "stream: weight operand read at %u", off);
          CHECK_OR_FAIL(cell[off / 16] == (lane & 15) * 4 + (lane >> 4), "stream: weight operand read of lane %d finds cell %d", lane, cell[off / 16]);
        }
      }
  for (int64_t m0 = 0; m0 < M; m0 += 16 * tm) {
    std::fill(acell.begin(), acell.end(), -1);
    for (int wave = 0; wave < 8; ++wave)
      for (int j = 0; j < la; ++j) {
        const int I = j * 8 + wave;
        CHECK_OR_FAIL(I < 4 * tm, "stream: activation load instruction %d of %d", I, 4 * tm);
        for (int lane = 0; lane < 64; ++lane) {
          const int row = addr::sa_row(lane, I), chunk = addr::sa_chunk(lane, I);
          CHECK_OR_FAIL(row < 16 * tm && chunk >= 0 && chunk < 16, "stream: activation row %d chunk %d", row, chunk);
          int64_t m = m0 + row;
          m = m < M ? m : M - 1;
          const int64_t voff = m * K * 2 + chunk * 16;
          for (int st = 0; st < steps; ++st) {
            const int64_t o = voff + (int64_t)st * 256;
            CHECK_OR_FAIL(o >= 0 && o + 16 <= a_extent, "stream: activation load at [%lld, +16) of %lld", (long long)o, (long long)a_extent);
          }
          const int at = I * 64 + lane;  // 16-byte cell inside the activation tile
          CHECK_OR_FAIL(at < (int)acell.size() && acell[at] == -1, "stream: activation cell %d written twice", at);
          CHECK_OR_FAIL(at == row * 16 + (lane & 15), "stream: activation lane lands on cell %d, not on its row", at);
          acell[at] = row * 16 + chunk;
        }
      }
    for (size_t c = 0; c < acell.size(); ++c) CHECK_OR_FAIL(acell[c] >= 0, "stream: activation cell %zu never written", c);
    for (int t = 0; t < tm; ++t)
      for (int ks = 0; ks < 4; ++ks)
        for (int lane = 0; lane < 64; ++lane) {
          const uint32_t off = addr::sa_frag_off(lane, t, ks);
          CHECK_OR_FAIL(off % 16 == 0 && off + 16 <= (uint32_t)tm * 4096, "stream: activation operand read at %u", off);
          const int want = (t * 16 + (lane & 15)) * 16 + 4 * (lane >> 4) + ks;
          CHECK_OR_FAIL(acell[off / 16] == want, "stream: activation operand read (lane %d, k-step %d) finds cell %d, expects %d", lane, ks,
                        acell[off / 16], want);
        }
  }
  return 0;
}

// Panel kernel (large M): 128 activation rows x 512 weight rows per work-group, steps of 128 values of K in two ring
// slots, scale windows of eight groups behind the ring.  Walks every work-group tile of an M x N problem: global
// extents of all three kinds of loads over every step / window of a slice plan, LDS extents and coverage of a slot,
// agreement of the landing cells with the operand reads, and that the LDS map stays within 160 KB.
int check_panel(int64_t M, int64_t N, int64_t K, int64_t group, int slice_steps) {
  CHECK_OR_FAIL(M >= 4 && N >= 16 && M % 4 == 0 && N % 16 == 0 && K >= 128 && K % 128 == 0, "panel: bad shape");
  CHECK_OR_FAIL(group >= 32 && (group & (group - 1)) == 0 && K % group == 0 && (K / group) % 8 == 0, "panel: group %lld on K %lld",
                (long long)group, (long long)K);
  const int64_t groups = K / group;
  CHECK_OR_FAIL(N * (K / 2) < ((int64_t)1 << 32) && M * K * 2 < ((int64_t)1 << 32) && N * groups * 2 < ((int64_t)1 << 32),
                "panel: a matrix spans 4 GiB or more");
  const int steps_total = (int)(K / 128);
  const int window = (int)(group >= 128 ? 8 * (group / 128) : 8 / (128 / group));
  CHECK_OR_FAIL(slice_steps >= 1 && (slice_steps % window == 0 || slice_steps >= steps_total), "panel: slices of %d steps are not whole windows of %d",
                slice_steps, window);
  const int TM = addr::kPanelTM, TN = addr::kPanelTN;
  const int64_t w_extent = N * (K / 2), a_extent = M * K * 2, s_extent = N * groups * 2;
  const uint32_t lds_total = addr::panel_sc_lds(7, 1) + addr::kPanelScBuf;
  CHECK_OR_FAIL(lds_total <= 160 * 1024, "panel: %u bytes of LDS", lds_total);
  const int slices = (steps_total + slice_steps - 1) / slice_steps;
  std::vector<int> cell(addr::kPanelSlot / 16);
  for (int64_t m0 = 0; m0 < M; m0 += 16 * TM)
    for (int64_t n0 = 0; n0 < N; n0 += 8 * 16 * TN) {
      std::fill(cell.begin(), cell.end(), -1);
      for (int wave = 0; wave < 8; ++wave) {
        for (int j = 0; j < 4; ++j) {
          const uint32_t l0 = addr::panel_a_lds(wave, j);
          const int I = j * 8 + wave;
          for (int lane = 0; lane < 64; ++lane) {
            const int64_t blk = addr::panel_a_block(wave, j, (int)m0, (int)M, (int)K);
            const int64_t voff = blk + addr::panel_a_lane(lane, (int)K) + addr::panel_a_chunk(lane, wave);
            CHECK_OR_FAIL(voff >= 0 && voff + (int64_t)(steps_total - 1) * 256 + 16 <= a_extent, "panel: activation load at %lld of %lld",
                          (long long)voff, (long long)a_extent);
            // inside the matrix the lane fetches the row and chunk its landing cell stands for
            if (m0 + 4 * I + 4 <= M)
              CHECK_OR_FAIL(voff == ((int64_t)(m0 + addr::sa_row(lane, I)) * K) * 2 + addr::sa_chunk(lane, I) * 16, "panel: activation lane %d of load %d fetches the wrong bytes", lane, I);
            const uint32_t at = l0 / 16 + lane;
            CHECK_OR_FAIL(at < addr::kPanelATile / 16 && cell[at] == -1, "panel: activation cell %u written twice or outside the tile", at);
            const int row = addr::sa_row(lane, I), chunk = addr::sa_chunk(lane, I);
            CHECK_OR_FAIL((int)at == row * 16 + (lane & 15), "panel: activation lane lands on cell %u, not on its row", at);
            cell[at] = row * 16 + chunk;
          }
        }
        for (int tn = 0; tn < TN; ++tn) {
          const uint32_t l0 = addr::panel_w_lds(wave, tn);
          for (int lane = 0; lane < 64; ++lane) {
            const int64_t voff = addr::panel_w_block(wave, tn, (int)n0, (int)N, (int)K) + addr::panel_w_lane(lane, (int)K);
            CHECK_OR_FAIL(voff >= 0 && voff + (int64_t)(steps_total - 1) * 64 + 16 <= w_extent, "panel: weight load at %lld of %lld",
                          (long long)voff, (long long)w_extent);
            if (n0 + wave * 64 + tn * 16 + 16 <= N)
              CHECK_OR_FAIL(voff == (int64_t)(n0 + wave * 64 + tn * 16 + addr::sw_row(lane)) * (K / 2) + addr::sw_piece(lane) * 16, "panel: weight lane %d fetches the wrong bytes", lane);
            const uint32_t at = l0 / 16 + lane;
            CHECK_OR_FAIL(at >= addr::kPanelATile / 16 && at < addr::kPanelSlot / 16 && cell[at] == -1, "panel: weight cell %u written twice or outside the slot", at);
            cell[at] = addr::sw_row(lane) * 4 + addr::sw_piece(lane);
          }
          for (int lane = 0; lane < 64; ++lane) {
            const uint32_t off = l0 + addr::sw_frag_off(lane);
            CHECK_OR_FAIL(off % 16 == 0 && off + 16 <= addr::kPanelSlot, "panel: weight operand read at %u", off);
            CHECK_OR_FAIL(cell[off / 16] == (lane & 15) * 4 + (lane >> 4), "panel: weight operand read of lane %d finds cell %d", lane, cell[off / 16]);
          }
        }
        // scale windows: lane l fetches 16 bytes of row n0 + 64 wave + l for every window of every slice
        for (int lane = 0; lane < 64; ++lane) {
          const int64_t voff = addr::panel_sc_voff(lane, wave, (int)n0, (int)N, (int)groups);
          for (int sl = 0; sl < slices; ++sl) {
            const int step0 = sl * slice_steps;
            const int steps = steps_total - step0 < slice_steps ? steps_total - step0 : slice_steps;
            const int64_t g0 = ((int64_t)step0 * 128) / group;
            const int nwin = (steps + window - 1) / window;
            for (int w = 0; w < nwin; ++w) {
              const int64_t o = voff + (g0 + 8 * w) * 2;
              CHECK_OR_FAIL(o >= 0 && o + 16 <= s_extent && o % 16 == 0, "panel: scale load at [%lld, +16) of %lld", (long long)o, (long long)s_extent);
              CHECK_OR_FAIL((g0 + 8 * w) % groups + 8 <= groups, "panel: a scale window crosses the end of a row of the scale tensor");
            }
          }
          for (int buf = 0; buf < 2; ++buf) {
            const uint32_t at = addr::panel_sc_lds(wave, buf) + 1024u + (uint32_t)lane * 16u;
            CHECK_OR_FAIL(at + 16 <= lds_total, "panel: scale window at %u", at);
          }
        }
        for (int row = 0; row < 16 * TN; ++row)
          for (int g = 0; g < 8; ++g)
            CHECK_OR_FAIL(addr::panel_sc_off(row, g) + 2 <= 1024 && addr::panel_sc_off(row, g) == (uint32_t)(row * 16 + g * 2), "panel: scale read");
      }
      for (uint32_t c = 0; c < addr::kPanelSlot / 16; ++c) CHECK_OR_FAIL(cell[c] >= 0, "panel: cell %u of the slot never written", c);
      for (int t = 0; t < TM; ++t)
        for (int ks = 0; ks < 4; ++ks)
          for (int lane = 0; lane < 64; ++lane) {
            const uint32_t off = addr::sa_frag_off(lane, t, ks);
            CHECK_OR_FAIL(off % 16 == 0 && off + 16 <= addr::kPanelATile, "panel: activation operand read at %u", off);
            const int want = (t * 16 + (lane & 15)) * 16 + 4 * (lane >> 4) + ks;
            CHECK_OR_FAIL(cell[off / 16] == want, "panel: activation operand read (lane %d, k-step %d) finds cell %d, expects %d", lane, ks, cell[off / 16], want);
          }
    }
  return 0;
}

// Panel kernel with 256 activation rows: 256 x 256 outputs per work-group of four wavefronts, steps of 128 values of K in
// two ring slots, scales / zero points gathered into registers.  Walks every work-group tile: global extents of the
// activation, weight and scale loads over every step of every slice (and of the steps past the end, which repeat the
// last), LDS extents and coverage of a slot, agreement of the landing cells with the operand reads.
int check_panel256(int64_t M, int64_t N, int64_t K, int64_t group, int slice_steps) {
  CHECK_OR_FAIL(M >= 4 && N >= 16 && M % 4 == 0 && N % 16 == 0 && K >= 128 && K % 128 == 0, "panel256: bad shape");
  CHECK_OR_FAIL(group >= 32 && (group & (group - 1)) == 0 && K % group == 0, "panel256: group %lld on K %lld", (long long)group, (long long)K);
  const int64_t groups = K / group;
  int gshift = 0;
  while (((int64_t)1 << gshift) < group) ++gshift;
  CHECK_OR_FAIL(N * (K / 2) < ((int64_t)1 << 32) && M * K * 2 < ((int64_t)1 << 32) && N * groups * 2 < ((int64_t)1 << 32),
                "panel256: a matrix spans 4 GiB or more");
  const int steps_total = (int)(K / 128);
  CHECK_OR_FAIL(slice_steps >= 1 && (slice_steps * 128 % group == 0 || group % (slice_steps * 128) == 0 || slice_steps >= steps_total),
                "panel256: slices of %d steps are neither whole groups nor an even part of one", slice_steps);
  const int TM = addr::kPanel2TM, TN = addr::kPanel2TN;
  const int64_t w_extent = N * (K / 2), a_extent = M * K * 2, s_extent = N * groups * 2;
  CHECK_OR_FAIL(2 * addr::kPanel2Slot <= 160 * 1024, "panel256: %u bytes of LDS", 2 * addr::kPanel2Slot);
  std::vector<int> cell(addr::kPanel2Slot / 16);
  for (int64_t m0 = 0; m0 < M; m0 += 16 * TM)
    for (int64_t n0 = 0; n0 < N; n0 += 4 * 16 * TN) {
      std::fill(cell.begin(), cell.end(), -1);
      for (int wave = 0; wave < 4; ++wave) {
        for (int j = 0; j < 16; ++j) {
          const uint32_t l0 = addr::panel2_a_lds(wave, j);
          const int I = j * 4 + wave;
          for (int lane = 0; lane < 64; ++lane) {
            const int64_t voff = addr::panel2_a_block(wave, j, (int)m0, (int)M, (int)K) + addr::panel_a_lane(lane, (int)K) + addr::panel_a_chunk(lane, wave);
            CHECK_OR_FAIL(voff >= 0 && voff + (int64_t)(steps_total - 1) * 256 + 16 <= a_extent, "panel256: activation load at %lld of %lld",
                          (long long)voff, (long long)a_extent);
            const uint32_t at = l0 / 16 + lane;
            CHECK_OR_FAIL(at < addr::kPanel2ATile / 16 && cell[at] == -1, "panel256: activation cell %u written twice or outside the tile", at);
            const int row = addr::sa_row(lane, I), chunk = addr::sa_chunk(lane, I);
            CHECK_OR_FAIL((int)at == row * 16 + (lane & 15), "panel256: activation lane lands on cell %u, not on its row", at);
            if (m0 + 4 * I + 4 <= M)
              CHECK_OR_FAIL(voff == ((int64_t)(m0 + row) * K) * 2 + chunk * 16, "panel256: activation lane %d of load %d fetches the wrong bytes", lane, I);
            cell[at] = row * 16 + chunk;
          }
        }
        for (int tn = 0; tn < TN; ++tn) {
          const uint32_t l0 = addr::panel2_w_lds(wave, tn);
          for (int lane = 0; lane < 64; ++lane) {
            const int64_t voff = addr::panel_w_block(wave, tn, (int)n0, (int)N, (int)K) + addr::panel_w_lane(lane, (int)K);
            CHECK_OR_FAIL(voff >= 0 && voff + (int64_t)(steps_total - 1) * 64 + 16 <= w_extent, "panel256: weight load at %lld of %lld",
                          (long long)voff, (long long)w_extent);
            if (n0 + wave * 64 + tn * 16 + 16 <= N)
              CHECK_OR_FAIL(voff == (int64_t)(n0 + wave * 64 + tn * 16 + addr::sw_row(lane)) * (K / 2) + addr::sw_piece(lane) * 16, "panel256: weight lane %d fetches the wrong bytes", lane);
            const uint32_t at = l0 / 16 + lane;
            CHECK_OR_FAIL(at >= addr::kPanel2ATile / 16 && at < addr::kPanel2Slot / 16 && cell[at] == -1, "panel256: weight cell %u written twice or outside the slot", at);
            cell[at] = addr::sw_row(lane) * 4 + addr::sw_piece(lane);
          }
          for (int lane = 0; lane < 64; ++lane) {
            const uint32_t off = l0 + addr::sw_frag_off(lane);
            CHECK_OR_FAIL(off % 16 == 0 && off + 16 <= addr::kPanel2Slot, "panel256: weight operand read at %u", off);
            CHECK_OR_FAIL(cell[off / 16] == (lane & 15) * 4 + (lane >> 4), "panel256: weight operand read of lane %d finds cell %d", lane, cell[off / 16]);
          }
          // the gathers of scales / zero points: the value of (row, group of the lane's 32 values) for every step
          for (int lane = 0; lane < 64; ++lane)
            for (int step = 0; step < steps_total; ++step) {
              const int64_t o = addr::panel2_sc_block(wave, tn, (int)n0, (int)N, (int)groups) + addr::panel2_sc_step(step, gshift) + addr::panel2_sc_lane(lane, (int)groups, gshift);
              CHECK_OR_FAIL(o >= 0 && o + 2 <= s_extent && o % 2 == 0, "panel256: scale gather at %lld of %lld", (long long)o, (long long)s_extent);
              if (n0 + wave * 64 + tn * 16 + 16 <= N) {
                const int64_t row = n0 + wave * 64 + tn * 16 + (lane & 15);
                const int64_t g = ((int64_t)step * 128 + 32 * (lane >> 4)) / group;
                CHECK_OR_FAIL(o == (row * groups + g) * 2, "panel256: scale gather of lane %d at step %d reads group %lld of row %lld", lane, step,
                              (long long)((o / 2) % groups), (long long)((o / 2) / groups));
              }
            }
        }
      }
      for (uint32_t c = 0; c < addr::kPanel2Slot / 16; ++c) CHECK_OR_FAIL(cell[c] >= 0, "panel256: cell %u of the slot never written", c);
      for (int t = 0; t < TM; ++t)
        for (int ks = 0; ks < 4; ++ks)
          for (int lane = 0; lane < 64; ++lane) {
            const uint32_t off = addr::sa_frag_off(lane, t, ks);
            CHECK_OR_FAIL(off == ((addr::sa_frag_off(lane, 0, 0) ^ (uint32_t)(ks << 4)) + (uint32_t)(t * 16 * 256)), "panel256: the k-step offset is not an exclusive-or");
            CHECK_OR_FAIL(off % 16 == 0 && off + 16 <= addr::kPanel2ATile, "panel256: activation operand read at %u", off);
            const int want = (t * 16 + (lane & 15)) * 16 + 4 * (lane >> 4) + ks;
            CHECK_OR_FAIL(cell[off / 16] == want, "panel256: activation operand read (lane %d, k-step %d) finds cell %d, expects %d", lane, ks, cell[off / 16], want);
          }
    }
  return 0;
}

// Middle-M panel kernel: 16 tm x 256 outputs per work-group of four wavefronts (tm = 4 or 8), a ring of D slots, scale
// windows in LDS.  Walks every work-group tile: global extents of the activation, weight and scale-window loads over every
// step and window of every slice, LDS extents and coverage of a ring slot and of the window buffers, agreement of the
// landing cells with the operand reads.
int check_panelm(int64_t M, int64_t N, int64_t K, int64_t group, int tm, int slice_steps) {
  CHECK_OR_FAIL(tm == 4 || tm == 8, "panelm: %d activation tiles per work-group", tm);
  CHECK_OR_FAIL(M >= 4 && N >= 16 && M % 4 == 0 && N % 16 == 0 && K >= 128 && K % 128 == 0, "panelm: bad shape");
  CHECK_OR_FAIL(group >= 32 && (group & (group - 1)) == 0 && K % group == 0 && (K / group) % 8 == 0, "panelm: group %lld on K %lld",
                (long long)group, (long long)K);
  const int64_t groups = K / group;
  CHECK_OR_FAIL(N * (K / 2) < ((int64_t)1 << 32) && M * K * 2 < ((int64_t)1 << 32) && N * groups * 2 < ((int64_t)1 << 32),
                "panelm: a matrix spans 4 GiB or more");
  const int steps_total = (int)(K / 128);
  const int window = (int)(group >= 128 ? 8 * (group / 128) : 8 / (128 / group));
  CHECK_OR_FAIL(window >= addr::panelm_depth(tm), "panelm: windows of %d steps on a ring of %d slots", window, addr::panelm_depth(tm));
  CHECK_OR_FAIL(slice_steps >= 1 && (slice_steps % window == 0 || slice_steps >= steps_total), "panelm: slices of %d steps are not whole windows of %d",
                slice_steps, window);
  const int TN = addr::kPanel2TN;
  const int64_t w_extent = N * (K / 2), a_extent = M * K * 2, s_extent = N * groups * 2;
  const uint32_t slot_bytes = addr::panelm_slot_bytes(tm), a_tile = addr::panelm_a_tile(tm), lds_total = addr::panelm_lds_bytes(tm);
  CHECK_OR_FAIL(lds_total <= 160 * 1024 && addr::panelm_sc_lds(tm, 0, 0) == (uint32_t)addr::panelm_depth(tm) * slot_bytes, "panelm: %u bytes of LDS", lds_total);
  const int slices = (steps_total + slice_steps - 1) / slice_steps;
  std::vector<int> cell(slot_bytes / 16);
  for (int64_t m0 = 0; m0 < M; m0 += 16 * tm)
    for (int64_t n0 = 0; n0 < N; n0 += 4 * 16 * TN) {
      std::fill(cell.begin(), cell.end(), -1);
      for (int wave = 0; wave < 4; ++wave) {
        for (int j = 0; j < tm; ++j) {
          const uint32_t l0 = addr::panel2_a_lds(wave, j);
          const int I = j * 4 + wave;
          for (int lane = 0; lane < 64; ++lane) {
            const int64_t voff = addr::panel2_a_block(wave, j, (int)m0, (int)M, (int)K) + addr::panel_a_lane(lane, (int)K) + addr::panel_a_chunk(lane, wave);
            CHECK_OR_FAIL(voff >= 0 && voff + (int64_t)(steps_total - 1) * 256 + 16 <= a_extent, "panelm: activation load at %lld of %lld",
                          (long long)voff, (long long)a_extent);
            const uint32_t at = l0 / 16 + lane;
            CHECK_OR_FAIL(at < a_tile / 16 && cell[at] == -1, "panelm: activation cell %u written twice or outside the tile", at);
            const int row = addr::sa_row(lane, I), chunk = addr::sa_chunk(lane, I);
            CHECK_OR_FAIL((int)at == row * 16 + (lane & 15), "panelm: activation lane lands on cell %u, not on its row", at);
            if (m0 + 4 * I + 4 <= M)
              CHECK_OR_FAIL(voff == ((int64_t)(m0 + row) * K) * 2 + chunk * 16, "panelm: activation lane %d of load %d fetches the wrong bytes", lane, I);
            cell[at] = row * 16 + chunk;
          }
        }
        for (int tn = 0; tn < TN; ++tn) {
          const uint32_t l0 = addr::panelm_w_lds(tm, wave, tn);
          for (int lane = 0; lane < 64; ++lane) {
            const int64_t voff = addr::panel_w_block(wave, tn, (int)n0, (int)N, (int)K) + addr::panel_w_lane(lane, (int)K);
            CHECK_OR_FAIL(voff >= 0 && voff + (int64_t)(steps_total - 1) * 64 + 16 <= w_extent, "panelm: weight load at %lld of %lld",
                          (long long)voff, (long long)w_extent);
            if (n0 + wave * 64 + tn * 16 + 16 <= N)
              CHECK_OR_FAIL(voff == (int64_t)(n0 + wave * 64 + tn * 16 + addr::sw_row(lane)) * (K / 2) + addr::sw_piece(lane) * 16, "panelm: weight lane %d fetches the wrong bytes", lane);
            const uint32_t at = l0 / 16 + lane;
            CHECK_OR_FAIL(at >= a_tile / 16 && at < slot_bytes / 16 && cell[at] == -1, "panelm: weight cell %u written twice or outside the slot", at);
            cell[at] = addr::sw_row(lane) * 4 + addr::sw_piece(lane);
          }
          for (int lane = 0; lane < 64; ++lane) {
            const uint32_t off = l0 + addr::sw_frag_off(lane);
            CHECK_OR_FAIL(off % 16 == 0 && off + 16 <= slot_bytes, "panelm: weight operand read at %u", off);
            CHECK_OR_FAIL(cell[off / 16] == (lane & 15) * 4 + (lane >> 4), "panelm: weight operand read of lane %d finds cell %d", lane, cell[off / 16]);
          }
        }
        // scale windows: lane l fetches 16 bytes of row n0 + 64 wave + l for every window of every slice
        for (int lane = 0; lane < 64; ++lane) {
          const int64_t voff = addr::panel_sc_voff(lane, wave, (int)n0, (int)N, (int)groups);
          for (int sl = 0; sl < slices; ++sl) {
            const int step0 = sl * slice_steps;
            const int steps = steps_total - step0 < slice_steps ? steps_total - step0 : slice_steps;
            const int64_t g0 = ((int64_t)step0 * 128) / group;
            const int nwin = (steps + window - 1) / window;
            for (int w = 0; w < nwin; ++w) {
              const int64_t o = voff + (g0 + 8 * w) * 2;
              CHECK_OR_FAIL(o >= 0 && o + 16 <= s_extent && o % 16 == 0, "panelm: scale load at [%lld, +16) of %lld", (long long)o, (long long)s_extent);
              CHECK_OR_FAIL((g0 + 8 * w) % groups + 8 <= groups, "panelm: a scale window crosses the end of a row of the scale tensor");
            }
            // the group a lane reads for step s of the slice lies in the window the kernel reads it from
            for (int s2 = 0; s2 < steps; ++s2)
              for (int q = 0; q < 4; ++q) {
                const int w = s2 / window, pos = s2 - w * window;
                const int64_t gl = ((int64_t)pos * 128 + q * 32) / group;
                CHECK_OR_FAIL(gl >= 0 && gl < 8 && g0 + 8 * w + gl == ((int64_t)(step0 + s2) * 128 + q * 32) / group, "panelm: step %d reads group %lld of its window", s2, (long long)gl);
              }
          }
          for (int buf = 0; buf < 2; ++buf) {
            const uint32_t at = addr::panelm_sc_lds(tm, wave, buf) + 1024u + (uint32_t)lane * 16u;
            CHECK_OR_FAIL(at + 16 <= lds_total && at >= (uint32_t)addr::panelm_depth(tm) * slot_bytes, "panelm: scale window at %u", at);
          }
        }
      }
      for (uint32_t c = 0; c < slot_bytes / 16; ++c) CHECK_OR_FAIL(cell[c] >= 0, "panelm: cell %u of the slot never written", c);
      for (int t = 0; t < tm; ++t)
        for (int ks = 0; ks < 4; ++ks)
          for (int lane = 0; lane < 64; ++lane) {
            const uint32_t off = addr::sa_frag_off(lane, t, ks);
            CHECK_OR_FAIL(off == ((addr::sa_frag_off(lane, 0, 0) ^ (uint32_t)(ks << 4)) + (uint32_t)(t * 16 * 256)), "panelm: the k-step offset is not an exclusive-or");
            CHECK_OR_FAIL(off % 16 == 0 && off + 16 <= a_tile, "panelm: activation operand read at %u", off);
            const int want = (t * 16 + (lane & 15)) * 16 + 4 * (lane >> 4) + ks;
            CHECK_OR_FAIL(cell[off / 16] == want, "panelm: activation operand read (lane %d, k-step %d) finds cell %d, expects %d", lane, ks, cell[off / 16], want);
          }
    }
  return 0;
}

// The middle-M kernel's schedule, played through for one wavefront: `steps` steps with windows of `window` steps, loads
// issued in the kernel's order and retired in issue order, the two waits leaving wait_w / wait_a of them outstanding.
// Every LDS read must find its data landed (the shared activation tile: landed and behind a barrier), every load into a
// ring slot or window buffer must come after the last read of what it held (the shared tile: with a barrier between).
int check_panelm_schedule(int tm, int steps, int window, int wait_w, int wait_a) {
  CHECK_OR_FAIL((tm == 4 || tm == 8) && steps >= 1 && steps <= 256 && window >= 1 && wait_w >= 0 && wait_a >= 0, "panelm schedule: bad arguments");
  const int D = addr::panelm_depth(tm), AR = addr::panelm_ahead(tm), S = addr::panelm_slots(tm), B = addr::panelm_barrier_slot(tm);
  const int WS = addr::panelm_w_slot(tm), TN = addr::kPanel2TN, word_slot = tm >= 8 ? tm / 2 : 0;
  enum { LA = 1, LW, LSC };
  struct Load { int kind, idx; };
  std::vector<Load> fifo;
  const int X = steps + D + 2, nwin = (steps + window - 1) / window;
  std::vector<int> landed_a(X, 0), landed_w(X, 0), landed_sc(nwin + 2, 0), published_a(X, 0);
  std::vector<int64_t> last_read_a(X, -1), last_read_w(X, -1), last_read_sc(nwin + 2, -1), barrier_times;
  int64_t now = -1;
  auto issue = [&](int kind, int idx) { fifo.push_back(Load{kind, idx}); };
  auto wait = [&](size_t n) {
    while (fifo.size() > n) {
      const Load l = fifo.front();
      fifo.erase(fifo.begin());
      (l.kind == LA ? landed_a : l.kind == LW ? landed_w : landed_sc)[l.idx]++;
    }
  };
  auto barrier = [&]() {
    for (int st = 0; st < X; ++st) published_a[st] = landed_a[st] >= tm;
    barrier_times.push_back(now);
  };
  auto barrier_between = [&](int64_t t0, int64_t t1) {
    for (int64_t b : barrier_times)
      if (b > t0 && b <= t1) return true;
    return false;
  };
  // prologue
  for (int i = 0; i < 2; ++i) issue(LSC, 0);
  for (int i = 0; i < TN; ++i) issue(LW, 0);
  for (int i = 0; i < D - 1; ++i) {
    for (int j = 0; j < tm; ++j) issue(LA, i);
    for (int j = 0; j < TN; ++j) issue(LW, i + 1);
  }
  wait(0);
  barrier();
  for (int s = 0; s < steps; ++s) {
    const int win = s / window, pos = s - win * window;
    const int nwin_idx = pos + 1 == window ? win + 1 : win;
    for (int t = 0; t < S; ++t) {
      now = (int64_t)s * S + t;
      const int ks = t / tm, slot_in_phase = t % tm;
      if (t == 2 * tm) {
        wait((size_t)wait_w);
        CHECK_OR_FAIL(landed_w[s + 1] >= TN, "panelm schedule: step %d: the next step's packed weights have not landed at their wait", s);
      }
      if (t == B) {
        wait((size_t)wait_a);
        CHECK_OR_FAIL(landed_a[s + 1] >= tm, "panelm schedule: step %d: the next activation tile has not landed at the barrier", s);
        barrier();
      }
      // behind MFMA 1 of the slot
      if (t < tm) {
        if (t == 0 && s >= 1)
          CHECK_OR_FAIL(barrier_between(last_read_a[s - 1], now - 1), "panelm schedule: step %d: the tile of step %d may still be read", s, s - 1);
        issue(LA, s + D - 1);  // into the slot of step s - 1
      }
      if (t == tm && pos == 0 && win + 1 < nwin) {
        if (win >= 1) CHECK_OR_FAIL(last_read_sc[win - 1] < now, "panelm schedule: window %d is overwritten while it is read", win - 1);
        issue(LSC, win + 1);
        issue(LSC, win + 1);
      }
      if (t >= WS && t < WS + TN) {
        CHECK_OR_FAIL(ks >= 2 && last_read_w[s] >= 0 && last_read_w[s] < now, "panelm schedule: step %d slot %d: this step's words are not all read", s, t);
        issue(LW, s + D);  // into the slot of step s
      }
      const int at = t + AR - 1, a_step = at < S ? s : s + 1;
      CHECK_OR_FAIL(published_a[a_step], "panelm schedule: step %d slot %d reads an operand of step %d before the barrier that publishes it", s, t, a_step);
      last_read_a[a_step] = now;
      if (slot_in_phase >= word_slot && slot_in_phase < word_slot + TN) {
        const int w_step = ks < 2 ? s : s + 1;
        CHECK_OR_FAIL(landed_w[w_step] >= TN, "panelm schedule: step %d slot %d reads a word of step %d that has not landed", s, t, w_step);
        last_read_w[w_step] = now;
      }
      if (t == 2 * tm && s + 1 < steps) {  // the scales of step s + 1
        CHECK_OR_FAIL(landed_sc[nwin_idx] >= 2, "panelm schedule: step %d reads scales of window %d, which has not landed", s, nwin_idx);
        last_read_sc[nwin_idx] = now;
      }
    }
    // the zero points of the next window are looked at at the top of the last step of a window: by then (the end of the
    // step before) they must have landed
    if (s + 1 < steps) {
      const int win1 = (s + 1) / window, pos1 = (s + 1) - win1 * window;
      if (pos1 + 1 == window && win1 + 1 < nwin)
        CHECK_OR_FAIL(landed_sc[win1 + 1] >= 2, "panelm schedule: the zero points of window %d are looked at before they have landed", win1 + 1);
    }
  }
  return 0;
}

// The 256-row panel kernel's schedule, played through for one wavefront over `steps` steps: loads issued per
// addr::panel2_slot_load retire in issue order, the two waits leave addr::kPanel2WaitW / kPanel2WaitA of them outstanding;
// every LDS read must find its data landed (for the shared activation tile: landed and behind a barrier), every load
// into a ring slot must come after the last read of what the slot held (for the shared tile: with a barrier between),
// and the dequantiser constants of a step must be made from that step's gathers.  (The wait counts are arguments so that
// a test can show that wrong ones fail.)
int check_panel256_schedule(int steps, int wait_w, int wait_a) {
  CHECK_OR_FAIL(steps >= 1 && steps <= 64 && wait_w >= 0 && wait_a >= 0, "panel256 schedule: bad arguments");
  struct Load { int kind, step; };
  std::vector<Load> fifo;  // oldest first
  const int S = steps + 4;
  std::vector<int> landed_a(S, 0), landed_w(S, 0), landed_sc(S, 0), published_a(S, 0);
  std::vector<int64_t> last_read_a(S, -1), last_read_w(S, -1), barrier_times;
  int64_t now = -1;
  int pinned_sc = -1;
  auto issue = [&](int kind, int step) { fifo.push_back(Load{kind, step}); };
  auto wait = [&](size_t n) {
    while (fifo.size() > n) {
      const Load l = fifo.front();
      fifo.erase(fifo.begin());
      (l.kind == addr::kPanel2LoadA ? landed_a : l.kind == addr::kPanel2LoadW ? landed_w : landed_sc)[l.step]++;
    }
  };
  auto barrier = [&]() {
    for (int st = 0; st < S; ++st) published_a[st] = landed_a[st] == 16;  // (every wavefront has waited for its own part)
    barrier_times.push_back(now);
  };
  auto barrier_between = [&](int64_t t0, int64_t t1) {  // a barrier at a time in (t0, t1]
    for (int64_t b : barrier_times)
      if (b > t0 && b <= t1) return true;
    return false;
  };
  // prologue (as the kernel's)
  for (int i = 0; i < 8; ++i) issue(addr::kPanel2LoadScale, 0);
  for (int i = 0; i < 4; ++i) issue(addr::kPanel2LoadW, 0);
  for (int i = 0; i < 16; ++i) issue(addr::kPanel2LoadA, 0);
  wait(0);  // (the compiler's own, at the first touch of the gathered values)
  CHECK_OR_FAIL(landed_sc[0] == 8, "panel256 schedule: the first gathers have not landed behind the prologue's first wait");
  for (int i = 0; i < 8; ++i) issue(addr::kPanel2LoadScale, 1);
  for (int i = 0; i < 4; ++i) issue(addr::kPanel2LoadW, 1);
  wait(0);
  CHECK_OR_FAIL(landed_sc[1] == 8 && landed_w[0] == 4 && landed_a[0] == 16, "panel256 schedule: the prologue's second wait leaves step 0 incomplete");
  pinned_sc = 1;
  barrier();
  for (int s = 0; s < steps; ++s)
    for (int t = 0; t < addr::kPanel2Slots; ++t) {
      now = (int64_t)s * addr::kPanel2Slots + t;
      const int ks = t / addr::kPanel2TM, tm = t % addr::kPanel2TM;
      if (t == addr::kPanel2WaitWSlot) {
        wait((size_t)wait_w);
        CHECK_OR_FAIL(landed_w[s + 1] == 4, "panel256 schedule: step %d: the next step's packed weights have not landed at their wait", s);
      }
      if (t >= addr::kPanel2ExpanderSlot && t < addr::kPanel2ExpanderSlot + 4 * addr::kPanel2TN && (t - addr::kPanel2ExpanderSlot) % 4 == 0)
        CHECK_OR_FAIL(pinned_sc == s + 1, "panel256 schedule: step %d slot %d: constants made from the gathers of step %d", s, t, pinned_sc);
      if (t == addr::kPanel2BarrierSlot) {
        wait((size_t)wait_a);
        CHECK_OR_FAIL(landed_a[s + 1] == 16 && landed_sc[s + 2] == 8, "panel256 schedule: step %d: activation tile or gathers not landed at the barrier", s);
        pinned_sc = s + 2;
        barrier();
      }
      // behind MFMA 1: the slot's load, the operand read kPanel2Ahead - 1 slots on, a packed word
      const int kind = addr::panel2_slot_load(t);
      if (kind == addr::kPanel2LoadA) {
        if (s >= 1)
          CHECK_OR_FAIL(barrier_between(last_read_a[s - 1], now - 1), "panel256 schedule: step %d slot %d: the tile of step %d may still be read", s, t, s - 1);
        issue(kind, s + 1);
      } else if (kind == addr::kPanel2LoadW) {
        CHECK_OR_FAIL(last_read_w[s] >= 0 && last_read_w[s] < now, "panel256 schedule: step %d slot %d: this step's words are not all read", s, t);
        CHECK_OR_FAIL(ks >= 2, "panel256 schedule: packed weights overwritten before the phase that reads this step's last word has passed");
        CHECK_OR_FAIL(t > addr::kPanel2BarrierSlot, "panel256 schedule: a direct load in flight where the compiler waits for the gathers");
        issue(kind, s + 2);
      } else if (kind == addr::kPanel2LoadScale) {
        issue(kind, s + 2);
      }
      const int at = t + addr::kPanel2Ahead - 1;
      const int a_step = at < addr::kPanel2Slots ? s : s + 1;
      CHECK_OR_FAIL(published_a[a_step], "panel256 schedule: step %d slot %d reads an operand of step %d before the barrier that publishes it", s, t, a_step);
      last_read_a[a_step] = now;
      if (tm >= addr::kPanel2WordSlot && tm < addr::kPanel2WordSlot + addr::kPanel2TN) {
        const int w_step = ks < 2 ? s : s + 1;
        CHECK_OR_FAIL(landed_w[w_step] == 4, "panel256 schedule: step %d slot %d reads a word of step %d that has not landed", s, t, w_step);
        last_read_w[w_step] = now;
      }
    }
  return 0;
}

// The ring: step s occupies slot s % D; at the top of step s the wavefront waits until only `younger` steps' loads are
// outstanding, passes the barrier, and then issues step s + D - 1 into the slot of step s - 1.
int check_stream_ring(int steps, int D) {
  CHECK_OR_FAIL(steps >= 1 && D >= 2 && D <= 8, "stream ring: bad arguments");
  std::vector<int> slot(D, -1), queue;  // slot owner; issued and not yet known to have landed (oldest first)
  std::vector<char> landed(steps, 0), done(steps, 0);
  for (int s = 0; s < D - 1 && s < steps; ++s) slot[s % D] = s, queue.push_back(s);
  for (int s = 0; s < steps; ++s) {
    const int younger = addr::stream_younger_steps(s, steps, D);
    while ((int)queue.size() > younger) landed[queue.front()] = 1, queue.erase(queue.begin());
    CHECK_OR_FAIL(landed[s], "stream ring: step %d multiplied before its loads were waited for", s);
    // barrier: every wavefront is past step s - 1
    if (s >= 1) done[s - 1] = 1;
    if (s + D - 1 < steps) {
      const int t = s + D - 1, sl = t % D;
      CHECK_OR_FAIL(slot[sl] < 0 || done[slot[sl]], "stream ring: step %d overwrites step %d which may still be read", t, slot[sl]);
      slot[sl] = t, queue.push_back(t);
    }
    CHECK_OR_FAIL(slot[s % D] == s, "stream ring: the slot of step %d holds step %d", s, slot[s % D]);
  }
  CHECK_OR_FAIL(queue.empty() || queue.back() <= steps - 1, "stream ring: bookkeeping");
  return 0;
}

// Decode kernel (1 .. 32 activation rows): every global access of every work-group, wavefront, item and lane of a
// launch with `grid_x` x `chunks` work-groups of `waves` wavefronts, and the LDS cells the operands are read from.
int check_decode(int64_t M, int64_t N, int64_t K, int64_t group, int mt, int chunks, int waves, int grid_x) {
  CHECK_OR_FAIL(M >= 1 && M <= 16 * mt && (mt == 1 || mt == 2), "decode: %lld activation rows in %d tiles", (long long)M, mt);
  CHECK_OR_FAIL(N >= 1 && K >= addr::kDecSlice && K % addr::kDecSlice == 0, "decode: bad shape");
  CHECK_OR_FAIL(group >= 32 && (group & (group - 1)) == 0 && K % group == 0, "decode: bad group %lld", (long long)group);
  CHECK_OR_FAIL(N * (K / 2) < ((int64_t)1 << 32) && M * K * 2 < ((int64_t)1 << 32), "decode: a matrix spans 4 GiB or more");
  const int64_t slices = K / addr::kDecSlice, groups = K / group, tiles = (N + 15) / 16;
  CHECK_OR_FAIL(chunks >= 1 && waves >= 1 && waves <= 16 && (int64_t)chunks * waves >= slices && (int64_t)(chunks - 1) * waves < slices,
                "decode: %d chunks of %d wavefronts do not cover %lld slices", chunks, waves, (long long)slices);
  CHECK_OR_FAIL(grid_x >= 1 && grid_x <= tiles, "decode: %d work-groups for %lld tiles", grid_x, (long long)tiles);
  // wavefront (ts mt + a) % waves adds up activation tile a of the ts-th weight tile: two tiles need two wavefronts
  CHECK_OR_FAIL(waves >= mt, "decode: %d wavefront(s) cannot add up the partial sums of %d activation tiles", waves, mt);
  CHECK_OR_FAIL(((N * groups) & 1) == 0, "decode: scale tensors of an odd number of values");
  CHECK_OR_FAIL((int64_t)waves * addr::dec_wave_bytes(mt) <= 160 * 1024, "decode: LDS");
  int gshift = 0;
  while (((int64_t)1 << gshift) < group) ++gshift;
  const int64_t w_extent = N * (K / 2), a_extent = M * K * 2, sc_extent = N * groups * 2;
  // operand cells of the 1 KB weight tile: lane l lands on cell l = (row l / 4, logical piece sw_piece)
  for (int lane = 0; lane < 64; ++lane) {
    const uint32_t off = addr::sw_frag_off(lane);
    CHECK_OR_FAIL(off % 16 == 0 && off + 16 <= 1024, "decode: weight operand read at %u", off);
    const int src = off / 16;  // the lane that wrote this cell
    CHECK_OR_FAIL(addr::sw_row(src) == (lane & 15) && addr::sw_piece(src) == (lane >> 4), "decode: weight operand read of lane %d finds row %d piece %d",
                  lane, addr::sw_row(src), addr::sw_piece(src));
  }
  std::vector<char> tile_seen(tiles, 0);
  for (int bx = 0; bx < grid_x; ++bx)
    for (int64_t t = bx; t < tiles; t += grid_x) {
      CHECK_OR_FAIL(!tile_seen[t], "decode: tile %lld handled twice", (long long)t);
      tile_seen[t] = 1;
    }
  for (int64_t t = 0; t < tiles; ++t) CHECK_OR_FAIL(tile_seen[t], "decode: tile %lld never handled", (long long)t);
  std::vector<char> k_seen(K / 8, 0);  // 16-byte pieces of one activation row
  const int nd = addr::dec_sc_dwords(gshift);
  for (int chunk = 0; chunk < chunks; ++chunk)
    for (int wave = 0; wave < waves; ++wave) {
      const int64_t slice = (int64_t)chunk * waves + wave;
      if (slice >= slices) continue;
      const int64_t k0 = slice * addr::kDecSlice;
      for (int kb = 0; kb < 2; ++kb)
        for (int m_t = 0; m_t < mt; ++m_t) {
          int64_t cell[256];  // 16-byte cells of the 4 KB block: the offset inside A of what landed there
          for (int i = 0; i < 4; ++i)
            for (int lane = 0; lane < 64; ++lane) {
              const int64_t o = addr::dec_a_off(lane, m_t, kb, i, M, K, k0);
              CHECK_OR_FAIL(o >= 0 && o % 16 == 0 && o + 16 <= a_extent, "decode: activation load at [%lld, +16) of %lld", (long long)o,
                            (long long)a_extent);
              const int64_t base = (k0 + kb * 128) * 2;
              CHECK_OR_FAIL(o - base >= 0 && o - base < ((int64_t)1 << 32), "decode: activation offset does not fit 32 bits");
              cell[i * 64 + lane] = o;
            }
          for (int lane = 0; lane < 64; ++lane)
            for (int j = 0; j < 4; ++j) {
              const uint32_t off = addr::dec_a_frag(lane, j);
              CHECK_OR_FAIL(off % 16 == 0 && off + 16 <= 4096, "decode: activation operand read at %u", off);
              int64_t m = m_t * 16 + (lane & 15);
              m = m < M ? m : M - 1;
              const int64_t k = k0 + kb * 128 + 32 * (lane >> 4) + 8 * j;  // the eight values that word 4 q + j of the weights holds
              CHECK_OR_FAIL(cell[off / 16] == (m * K + k) * 2, "decode: activation operand of lane %d, k-step %d holds other values", lane, j);
              if (m_t == 0 && (lane & 15) == 0) k_seen[k / 8] = 1;
            }
        }
      for (int64_t t = 0; t < tiles; ++t) {
        const int64_t base = addr::dec_w_base(t, K, k0);
        for (int lane = 0; lane < 64; ++lane) {
          // the kernel keeps the lane parts of tile 0 and of the last tile only
          const uint32_t wl = t == tiles - 1 ? addr::dec_w_lane(lane, t, N, K) : addr::dec_w_lane(lane, 0, 16, K);
          int64_t n = t * 16 + addr::sw_row(lane);
          n = n < N ? n : N - 1;
          for (int kb = 0; kb < 2; ++kb) {
            const int64_t o = base + wl + kb * 64;
            CHECK_OR_FAIL(o >= 0 && o % 16 == 0 && o + 16 <= w_extent, "decode: weight load at [%lld, +16) of %lld", (long long)o, (long long)w_extent);
            CHECK_OR_FAIL(o == n * (K / 2) + (k0 + kb * 128) / 2 + addr::sw_piece(lane) * 16, "decode: weight load of lane %d reads another row or piece", lane);
          }
          if (lane < 16 * nd) {
            const int64_t e = t == tiles - 1 ? addr::dec_sc_elem(lane, t, N, groups, k0, gshift)
                                             : addr::dec_sc_elem(lane, 0, 16, groups, k0, gshift) + t * 16 * groups;
            const int64_t d = addr::dec_sc_off(e);
            CHECK_OR_FAIL(e >= 0 && d % 4 == 0 && d + 4 <= sc_extent, "decode: scale gather at [%lld, +4) of %lld", (long long)d, (long long)sc_extent);
            CHECK_OR_FAIL(e == addr::dec_sc_elem(lane, t, N, groups, k0, gshift), "decode: scale gather of lane %d in tile %lld", lane, (long long)t);
          }
        }
        // every lane finds the scale of its row and group: cell c of the area was written by gather lane c
        for (int lane = 0; lane < 64; ++lane)
          for (int kb = 0; kb < 2; ++kb) {
            const uint32_t cell = addr::dec_sc_cell(lane, kb, gshift);
            CHECK_OR_FAIL(cell % 4 == 0 && cell / 4 < (uint32_t)(16 * nd), "decode: scale read at %u outside the gathered cells", cell);
            const int src = (int)(cell / 4);
            const int64_t e = addr::dec_sc_elem(src, t, N, groups, k0, gshift);
            const int64_t value = (addr::dec_sc_off(e) >> 1) + (addr::dec_sc_half(lane, kb, groups, k0, gshift) >> 4);
            int64_t n = t * 16 + (lane & 15);
            const bool real_row = n < N;
            n = real_row ? n : N - 1;
            const int64_t want = n * groups + (k0 + kb * 128 + 32 * (lane >> 4)) / group;
            // rows past N are never stored: only their reads have to stay inside the area
            CHECK_OR_FAIL(!real_row || value == want, "decode: lane %d reads scale %lld instead of %lld (tile %lld, k-block %d)", lane,
                          (long long)value, (long long)want, (long long)t, kb);
          }
      }
    }
  for (int64_t c = 0; c < K / 8; ++c) CHECK_OR_FAIL(k_seen[c], "decode: values %lld .. of K are never multiplied", (long long)(c * 8));
  return 0;
}

// The ring of the decode kernel: the ts-th tile of a wavefront lives in slot ts % 3; tiles 0 and 1 are issued up front
// (slot 2 is scratch meanwhile); iteration ts issues tile ts + 2, then waits, before each k-block, until at most
// dec_wait_count loads are in flight.  A tile's loads, in issue order: scale gather, zero gather, piece 0, piece 1.
int check_decode_ring(int my_tiles) {
  CHECK_OR_FAIL(my_tiles >= 1, "decode ring: bad arguments");
  const int TS = addr::kDecTileSlots;
  std::vector<int> slot(TS, -1);
  std::vector<std::pair<int, int>> queue;  // (tile, load 0 .. 3), oldest first
  std::vector<char> read(my_tiles, 0);
  auto issue = [&](int ts) {
    for (int l = 0; l < 4; ++l) queue.push_back({ts, l});
    slot[ts % TS] = ts;
  };
  issue(0);
  if (my_tiles > 1) issue(1);
  CHECK_OR_FAIL(slot[2] < 0, "decode ring: the slot that stages the activations is in use during the prologue");
  for (int ts = 0; ts < my_tiles; ++ts) {
    if (ts + 2 < my_tiles) {
      const int sl = (ts + 2) % TS;
      CHECK_OR_FAIL(slot[sl] < 0 || read[slot[sl]], "decode ring: tile %d overwrites tile %d before it was read", ts + 2, slot[sl]);
      issue(ts + 2);
    }
    for (int kb = 0; kb < 2; ++kb) {
      const int allowed = addr::dec_wait_count(ts, kb, my_tiles);
      CHECK_OR_FAIL(allowed == 0 || allowed == 1 || allowed == 4 || allowed == 5 || allowed == 8 || allowed == 9,
                    "decode ring: wait count %d has no s_waitcnt case", allowed);
      while ((int)queue.size() > allowed) queue.erase(queue.begin());
      for (auto& e : queue)
        CHECK_OR_FAIL(!(e.first == ts && (e.second <= 2 || kb == 1)),  // k-block 0 needs the gathers and piece 0, k-block 1 all four
                      "decode ring: k-block %d of tile %d read while load %d of it may be in flight", kb, ts, e.second);
    }
    CHECK_OR_FAIL(slot[ts % TS] == ts, "decode ring: the slot of tile %d holds tile %d", ts, slot[ts % TS]);
    read[ts] = 1;
  }
  CHECK_OR_FAIL(queue.empty(), "decode ring: loads in flight at the end");
  return 0;
}

}  // namespace
}  // namespace tlq

using namespace tlq;

// GEMV ring kernel: every direct load of every work-group stays inside its tensor and inside its LDS area, the staging
// instructions cover every piece, every row is read by exactly one wavefront from the slot its loads went to, and no
// row is read while one of its loads may be in flight or overwritten before it was read.
int check_gemv_ring(int64_t M, int64_t N, int64_t K, int64_t group, int rows_per_block, int waves, int depth) {
  CHECK_OR_FAIL(M >= 1 && M <= 2 && N >= 1 && K >= 32 && K % 32 == 0 && group >= 32 && K % group == 0 && rows_per_block >= 1 && waves >= 1 &&
                    waves <= 16 && depth >= 1 && depth <= 3,
                "gemv ring: bad arguments");
  const int chunks = (int)(K / 32), groups = (int)(K / group), iters = (chunks + 63) / 64;
  CHECK_OR_FAIL(iters * depth <= 6, "gemv ring: %d loads per wavefront in flight have no s_waitcnt case", iters * depth);
  CHECK_OR_FAIL(groups % 8 == 0, "gemv ring: %d groups per row are not a whole number of 16-byte pieces", groups);
  const int64_t row_bytes = K / 2;
  const addr::RingLayout L = addr::ring_layout(waves, depth, iters, (int)K, rows_per_block, groups, (int)M);
  CHECK_OR_FAIL(L.total <= 160 * 1024, "gemv ring: %u bytes of LDS", L.total);
  const int64_t blocks = (N + rows_per_block - 1) / rows_per_block;
  const int64_t probe[6] = {0, 1, blocks / 2, blocks - 2, blocks - 1, blocks / 3};
  for (int pi = 0; pi < 6; ++pi) {
    const int64_t b = probe[pi];
    if (b < 0 || b >= blocks) continue;
    const int64_t r0 = b * rows_per_block, r1 = r0 + rows_per_block < N ? r0 + rows_per_block : N;
    // staging: activations, then scales / zero points of rows r0 .. r1 - 1
    const int a_pieces = chunks * 4 * (int)M, sz_pieces = (int)((r1 - r0) * groups / 8);
    for (int which = 0; which < 2; ++which) {
      const int pieces = which == 0 ? a_pieces : sz_pieces;
      const uint32_t area = which == 0 ? L.act : L.s, area_end = which == 0 ? L.s : L.z;
      const int64_t src_bytes = which == 0 ? M * K * 2 : (N - r0) * groups * 2;  // from the base pointer of the instruction
      std::vector<char> seen(pieces, 0);
      for (int w = 0; w < waves; ++w)
        for (int p0 = w * 64; p0 < pieces; p0 += waves * 64)
          for (int lane = 0; lane < 64; ++lane) {
            const uint32_t voff = which == 0 ? addr::ring_act_voff(p0, lane, pieces) : addr::ring_stage_voff(p0, lane, pieces);
            CHECK_OR_FAIL((int64_t)voff + 16 <= src_bytes, "gemv ring: staging read at byte %u of %lld", voff, (long long)src_bytes);
            const uint32_t dst = area + (uint32_t)p0 * 16u + (uint32_t)lane * 16u;
            CHECK_OR_FAIL(dst + 16 <= area_end, "gemv ring: staging write at LDS byte %u, area ends at %u", dst, area_end);
            if (p0 + lane < pieces) {
              // the activation pieces of a chunk are rotated (ring_act_logical); scales and zero points lie in order
              const int piece = which == 0 ? addr::ring_act_logical(p0 + lane) : p0 + lane;
              CHECK_OR_FAIL(piece >= 0 && piece < pieces && !seen[piece], "gemv ring: staging piece %d loaded twice or out of range", piece);
              CHECK_OR_FAIL(voff == (uint32_t)piece * 16u, "gemv ring: piece %d read from byte %u", piece, voff);
              seen[piece] = 1;
            }
          }
      for (int p = 0; p < pieces; ++p) CHECK_OR_FAIL(seen[p], "gemv ring: staging piece %d of %d never loaded", p, pieces);
      if (which == 0)  // the read of piece j of chunk c finds the position that holds it
        for (int c = 0; c < pieces / 4; ++c)
          for (int j = 0; j < 4; ++j) {
            const uint32_t off = addr::ring_act_lds(c, j);
            CHECK_OR_FAIL(off % 16 == 0 && (int)(off / 16) < pieces && addr::ring_act_logical((int)(off / 16)) == 4 * c + j,
                          "gemv ring: activation read (chunk %d, piece %d) at byte %u finds another piece", c, j, off);
          }
    }
    CHECK_OR_FAIL(L.z + (uint32_t)sz_pieces * 16u <= L.total && L.total - L.z == L.z - L.s, "gemv ring: zero-point area");
    // weights
    std::vector<int> reader((size_t)(r1 - r0), -1);
    for (int w = 0; w < waves; ++w) {
      const int my_rows = addr::ring_my_rows((int)(r1 - r0), w, waves);
      std::vector<int> slot(depth, -1);
      std::vector<char> read(my_rows > 0 ? my_rows : 1, 0);
      std::vector<int> queue;  // row index of each outstanding load, oldest first
      auto issue = [&](int i, int sl) -> int {
        const int64_t row = r0 + w + (int64_t)i * waves;
        CHECK_OR_FAIL(row < r1, "gemv ring: wavefront %d asks for row %lld past its work-group", w, (long long)row);
        CHECK_OR_FAIL(slot[sl] < 0 || read[slot[sl]], "gemv ring: row %d overwrites row %d before it was read", i, slot[sl]);
        for (int it = 0; it < iters; ++it) {
          for (int lane = 0; lane < 64; ++lane) {
            const int64_t src = row * row_bytes + addr::ring_w_voff(lane, it, chunks);
            CHECK_OR_FAIL(src + 16 <= N * row_bytes && addr::ring_w_voff(lane, it, chunks) + 16 <= row_bytes, "gemv ring: weight read past the row");
            const uint32_t dst = L.ring + addr::ring_w_lds(w, sl, it, depth, iters) + (uint32_t)lane * 16u;
            CHECK_OR_FAIL(dst + 16 <= L.act, "gemv ring: weight write at LDS byte %u, ring ends at %u", dst, L.act);
            CHECK_OR_FAIL(dst / (1024u * iters) == (uint32_t)(w * depth + sl), "gemv ring: weight write outside the slot");
          }
          queue.push_back(i);
        }
        slot[sl] = i;
        return 0;
      };
      for (int d = 0; d < depth; ++d)
        if (d < my_rows)
          if (int rc = issue(d, d)) return rc;
      int sl = 0;
      for (int i = 0; i < my_rows; ++i) {
        const int allowed = iters * addr::ring_younger_rows(i, my_rows, depth);
        while ((int)queue.size() > allowed) queue.erase(queue.begin());
        for (int q : queue) CHECK_OR_FAIL(q != i, "gemv ring: row %d read while one of its loads may be in flight", i);
        CHECK_OR_FAIL(slot[sl] == i, "gemv ring: slot %d holds row %d when row %d is read", sl, slot[sl], i);
        read[i] = 1;
        const int lrow = w + i * waves;
        CHECK_OR_FAIL(lrow < r1 - r0 && reader[lrow] < 0, "gemv ring: row %d read twice", lrow);
        CHECK_OR_FAIL((int64_t)(lrow * groups + groups) * 2 <= (int64_t)(L.z - L.s), "gemv ring: scale row outside its area");
        reader[lrow] = w;
        if (i + depth < my_rows)
          if (int rc = issue(i + depth, sl)) return rc;
        sl = sl + 1 == depth ? 0 : sl + 1;
      }
    }
    for (size_t r = 0; r < reader.size(); ++r) CHECK_OR_FAIL(reader[r] >= 0, "gemv ring: row %zu of work-group %lld never read", r, (long long)b);
  }
  return 0;
}

extern "C" {

int tlq_debug_check_gemm_addressing(int source_kind, int64_t rows, int64_t row_bytes, int tile, int threads) {
  if (source_kind == 0) return check_row_direct(rows, row_bytes, tile, threads);
  if (source_kind == 1) {
    if (tile == 256) return check_kn_direct<256>(rows, row_bytes, threads);
    if (tile == 128) return check_kn_direct<128>(rows, row_bytes, threads);
    set_error("tlq_debug_check_gemm_addressing: [K,N] tiles are 128 or 256 columns wide (got %d)", tile);
    return 1;
  }
  if (source_kind == 2) {
    if (tile == 256) return check_kn16_direct<256>(rows, row_bytes, threads);
    if (tile == 128) return check_kn16_direct<128>(rows, row_bytes, threads);
    set_error("tlq_debug_check_gemm_addressing: 16-bit [K,N] tiles are 128 or 256 columns wide (got %d)", tile);
    return 1;
  }
  set_error("tlq_debug_check_gemm_addressing: bad source kind %d", source_kind);
  return 1;
}

int tlq_debug_check_stream_addressing(int64_t M, int64_t N, int64_t K, int activation_tiles, int ring_depth) {
  if (int rc = check_stream(M, N, K, activation_tiles)) return rc;
  for (int steps = 1; steps <= 40; ++steps)
    if (int rc = check_stream_ring(steps, ring_depth)) return rc;
  return 0;
}

int tlq_debug_check_panel256_addressing(int64_t M, int64_t N, int64_t K, int64_t group, int slice_steps) {
  if (int rc = check_panel256(M, N, K, group, slice_steps)) return rc;
  for (int steps : {1, 2, 3, 4, 7})
    if (int rc = check_panel256_schedule(steps, addr::kPanel2WaitW, addr::kPanel2WaitA)) return rc;
  return 0;
}

int tlq_debug_check_panelm_addressing(int64_t M, int64_t N, int64_t K, int64_t group, int rows, int slice_steps) {
  if (rows != 64 && rows != 128) {
    set_error("tlq_debug_check_panelm_addressing: %d activation rows per work-group", rows);
    return 1;
  }
  const int tm = rows / 16;
  if (int rc = check_panelm(M, N, K, group, tm, slice_steps)) return rc;
  const int window = (int)(group >= 128 ? 8 * (group / 128) : 8 / (128 / group));
  const int steps_total = (int)(K / 128), slice = slice_steps < steps_total ? slice_steps : steps_total;
  for (int steps : {slice, steps_total % slice ? steps_total % slice : slice})
    if (int rc = check_panelm_schedule(tm, steps, window, addr::panelm_wait_w(tm), addr::panelm_wait_a(tm))) return rc;
  return 0;
}

int tlq_debug_check_panelm_schedule(int rows, int steps, int window, int wait_w, int wait_a) {
  const int tm = rows / 16;
  if (tm != 4 && tm != 8) return 1;
  return check_panelm_schedule(tm, steps, window, wait_w < 0 ? addr::panelm_wait_w(tm) : wait_w, wait_a < 0 ? addr::panelm_wait_a(tm) : wait_a);
}

int tlq_debug_check_panel256_schedule(int steps, int wait_w, int wait_a) {
  return check_panel256_schedule(steps, wait_w < 0 ? addr::kPanel2WaitW : wait_w, wait_a < 0 ? addr::kPanel2WaitA : wait_a);
}

int tlq_debug_check_panel_addressing(int64_t M, int64_t N, int64_t K, int64_t group, int slice_steps) {
  return check_panel(M, N, K, group, slice_steps);
}

int tlq_debug_check_decode_addressing(int64_t M, int64_t N, int64_t K, int64_t group, int activation_tiles, int chunks, int waves,
                                      int grid_x) {
  if (int rc = check_decode(M, N, K, group, activation_tiles, chunks, waves, grid_x)) return rc;
  for (int my_tiles = 1; my_tiles <= 16; ++my_tiles)
    if (int rc = check_decode_ring(my_tiles)) return rc;
  return 0;
}

int tlq_debug_check_slots_schedule(int stages, int loads_per_tile) {
  if (stages < 1 || loads_per_tile < 1) {
    set_error("tlq_debug_check_slots_schedule: bad arguments");
    return 1;
  }
  SlotsSim sim(stages, loads_per_tile);
  addr::slots_schedule(stages, sim);
  for (int t = 0; t < 2 * stages && !sim.error; ++t)
    if (!sim.multiplied[t]) sim.fail("a tile was never multiplied", t);
  if (sim.error) {
    set_error("%s", sim.msg);
    return 1;
  }
  return 0;
}

int tlq_debug_check_gemv_ring_addressing(int64_t M, int64_t N, int64_t K, int64_t group, int rows_per_block, int waves, int depth) {
  return check_gemv_ring(M, N, K, group, rows_per_block, waves, depth);
}

}  // extern "C"
