// extern "C" entry points of the GEMM family: argument validation, then dispatch.
// Every shape assumption a kernel makes is checked here, before anything is launched.
#include "tlq_common.h"
#include "gemm_core.h"

namespace tlq {
int gemv_w4a16(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t batch, int64_t M,
               int64_t N, int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, hipStream_t st);
bool gemv_ring_applies(int64_t M, int64_t N, int64_t K, int64_t group, int in_dtype, const void* scales, const void* zeros);
int w4a16_tail_rows(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t rows, int64_t K,
                    int64_t group, float zero_scalar, int in_dtype, int out_dtype, int w_layout, int64_t ldc, int64_t col0, hipStream_t st);
int gemv_w4a16_ring_interleaved(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t N,
                                int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, hipStream_t st);
int gemm_w4a16_mfma(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t N,
                    int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, hipStream_t st);
int64_t w4a16_mid_split(int64_t M, int64_t N, int64_t K, int64_t group);
double w4a16_mid_fill(int64_t M, int64_t N, int64_t K, int64_t group);
int gemm_w4a16_mfma_splitk(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M,
                           int64_t N, int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype,
                           int64_t split, float* partial, hipStream_t st);
struct StreamPlan {
  bool ok;
  int tm, m_blocks, n_blocks, split, slice_steps;
};
StreamPlan w4a16_stream_plan(int64_t M, int64_t N, int64_t K, int64_t group, int cus);
int gemm_w4a16_stream(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t N,
                      int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, int w_layout, const StreamPlan& p,
                      float* partial, hipStream_t st);
int gemm_w4a16_skinny(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t N,
                      int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, hipStream_t st);
int gemm_f16_plain(const void* A, const void* B, void* C, int64_t batch, int64_t M, int64_t N, int64_t K, int in_dtype,
                   int out_dtype, int b_layout, hipStream_t st);
int gemm_f16_splitk(const void* A, const void* B, float* C, int64_t M, int64_t N, int64_t K, int64_t split_k,
                    int in_dtype, int b_layout, hipStream_t st);
extern thread_local int g_f16_split;
int f16_split_choice(int64_t batch, int64_t M, int64_t N, int64_t K);
int gemm_f16_slices(const void* A, const void* B, void* C, float* partial, int64_t M, int64_t N, int64_t K, int64_t split,
                    int in_dtype, int out_dtype, int b_layout, hipStream_t st);
int gemm_i8_i32(const void* A, const void* B, void* C, int64_t batch, int64_t M, int64_t N, int64_t K, int b_layout,
                hipStream_t st);
int gemm_w8a8_rescale(const void* A, const void* B, const void* scale_a, const void* scale_b, void* C, int64_t batch,
                      int64_t M, int64_t N, int64_t K, int64_t n_scale_b, int b_layout, int out_dtype, hipStream_t st);
int gemm_w4a8_i32(const void* A, const void* Wp, void* C, int64_t M, int64_t N, int64_t K, int sign_mode,
                  hipStream_t st);
int i8_split_choice(int64_t batch, int64_t M, int64_t N, int64_t K, bool buffers, double pace = 1.0);
int gemm_w4a8_i32_splitk(const void* A, const void* Wp, void* C, int64_t M, int64_t N, int64_t K, int sign_mode,
                         int64_t split, int32_t* partial, hipStream_t st);
int gemm_i8_i32_splitk(const void* A, const void* B, int32_t* acc, int64_t M, int64_t N, int64_t K, int64_t split,
                       int b_layout, hipStream_t st);
int gemm_w8a8_rescale_splitk(const void* A, const void* B, const void* scale_a, const void* scale_b, void* C, int32_t* partial,
                             int64_t M, int64_t N, int64_t K, int64_t n_scale_b, int64_t split, int b_layout, int out_dtype,
                             hipStream_t st);

struct PanelPlan {
  bool ok;
  int tiles_m, tiles_n, split, slice_steps;
};
PanelPlan w4a16_panel_plan(int64_t M, int64_t N, int64_t K, int64_t group, int cus);
int gemm_w4a16_panel(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t N, int64_t K,
                     int64_t group, float zero_scalar, int in_dtype, int out_dtype, int w_layout, const PanelPlan& p, float* partial,
                     uint32_t* flag, hipStream_t st);
extern thread_local int g_panel_slice_steps;
thread_local int g_w4a16_panel = 0;  // tlq_tune_w4a16_panel: non-zero = no panel kernel is picked automatically
struct Panel2Plan {
  bool ok;
  int tiles_m, tiles_n, split, slice_steps;
};
Panel2Plan w4a16_panel256_plan(int64_t M, int64_t N, int64_t K, int64_t group, int cus);
int gemm_w4a16_panel256(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t N, int64_t K,
                        int64_t group, float zero_scalar, int in_dtype, int out_dtype, int w_layout, const Panel2Plan& p, float* partial,
                        hipStream_t st);
extern thread_local int g_panel2_slice_steps;
struct PanelMPlan {
  bool ok;
  int tm, tiles_m, tiles_n, split, slice_steps;
};
PanelMPlan w4a16_panelm_plan(int64_t M, int64_t N, int64_t K, int64_t group, int cus);
int gemm_w4a16_panelm(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t N, int64_t K,
                      int64_t group, float zero_scalar, int in_dtype, int out_dtype, const PanelMPlan& p, float* partial, hipStream_t st);
extern thread_local int g_panelm_slice_steps;
extern thread_local int g_panelm_rows;

struct DecodePlan {
  bool ok;
  int mt, chunks, waves, grid_x;
  int64_t lds_bytes;
};
DecodePlan w4a16_decode_plan(int64_t M, int64_t N, int64_t K, int64_t group, int cus);
int gemm_w4a16_decode(const void* A, const void* Wp, const void* scales, const void* zeros, void* C, int64_t M, int64_t N, int64_t K,
                      int64_t group, float zero_scalar, int in_dtype, int out_dtype, int w_layout, const DecodePlan& p, float* partial,
                      hipStream_t st);

thread_local int g_gemm_band_rows = 0;
thread_local int g_gemm_slots = 1;  // tlq_tune_gemm_slots: 0 = never the five-slot kernel, 1 = where it measured faster, 2 = wherever it can run
extern thread_local int g_gemm_f16_tile;
static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }
// compute units of the current device (256 when it cannot be asked, e.g. without a GPU)
static int cu_count_or_default() {
  const int n = tlq_device_cu_count();
  return n > 0 ? n : 256;
}
extern thread_local int g_stream_slice_steps;
thread_local int g_w4a16_stream = 1;  // 0: never pick the streaming kernel automatically (tuning runs)
thread_local int g_w4a16_decode = 1;  // 0: never pick the decode kernel automatically
// the tile loaders address one matrix with 32-bit byte offsets
static bool fits32(int64_t rows, int64_t row_bytes) { return rows * row_bytes < ((int64_t)1 << 32); }
static const int64_t kMaxDim = (int64_t)1 << 30;
// the table of tuned kernel choices (w4a16_choice.hip)
int w4a16_choice_lookup(int64_t M, int64_t N, int64_t K, int64_t group, int in_dtype);
void w4a16_choice_for_shape(int64_t M, int64_t N, int64_t K, void (*fn)(int algo, void* ctx), void* ctx);

}  // namespace tlq

// One scale / zero point per weight row (group = K) where K is no power of two: the fast kernels index groups by shifts, so
// the row's value is written out once per power-of-two group (the largest power of two that divides K, 1024 at most) into
// the tail of the workspace and the call runs with that group size -- the same arithmetic per weight, hence the same bits.
__global__ __launch_bounds__(256) void expand_row_values_kernel(const uint16_t* __restrict__ in, uint16_t* __restrict__ out, int64_t n_out,
                                                                int groups) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_out; i += (int64_t)gridDim.x * blockDim.x) out[i] = in[i / groups];
}
// A matrix of `cols` columns (rows packed) into the first `cols` columns of a matrix whose rows lie `ldc` elements apart.
template <typename E>
__global__ __launch_bounds__(256) void copy_into_wider_rows_kernel(const E* __restrict__ in, E* __restrict__ out, int64_t M, int64_t cols, int64_t ldc) {
  const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= cols) return;
  for (int64_t m = blockIdx.y; m < M; m += gridDim.y) out[m * ldc + c] = in[m * cols + c];
}
// The same for 16-bit elements, two at a time: pairs that are aligned in the OUTPUT (a row starts at element m * ldc, whose
// parity moves the pairs by one column), one 4-byte store each; the first or last column of a row alone where a pair straddles it.
__global__ __launch_bounds__(256) void copy_pairs_into_wider_rows_kernel(const uint16_t* __restrict__ in, uint16_t* __restrict__ out, int64_t M,
                                                                        int64_t cols, int64_t ldc) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (int64_t m = blockIdx.y; m < M; m += gridDim.y) {
    const int64_t o = m * ldc;
    const int64_t c0 = 2 * t - (o & 1);
    if (c0 >= cols) continue;
    const uint16_t* const src = in + m * cols;
    if (c0 >= 0 && c0 + 1 < cols)
      *(uint32_t*)(out + o + c0) = (uint32_t)src[c0] | ((uint32_t)src[c0 + 1] << 16);
    else if (c0 >= 0)
      out[o + c0] = src[c0];
    else
      out[o] = src[0];
  }
}
// A weight-row count that is no multiple of four (vocabularies of 50257 or 32001 rows): the multiple of 16 below runs through the
// usual choice into a packed result behind the workspace, which is then copied into C; the last rows go straight into C.
static int64_t ragged_head(int64_t N) { return N & ~(int64_t)15; }
static int64_t ragged_result_bytes(int64_t M, int64_t N, int out_bytes) { return (M * ragged_head(N) * out_bytes + 15) / 16 * 16; }
// (Also a multiple of four that is no multiple of eight above 512 rows, where the panel kernels are the choice and want multiples
// of 16 and the two passes multiples of eight, which leaves the tile kernel through registers: N = 4100, K = 4096, M = 1024 .. 4096:
// 63 - 150 against 92 - 239 us; N = 32004: 228 - 1082 against 275 - 1135 us -- while the packed result stays below 1 GiB.  With
// multiples of eight the two passes are level or ahead from 2048 rows on: N = 14344, M = 4096: 430 against 512 us.)
static bool ragged_rows_apply(int64_t M, int64_t N) {
  if (!(N >= 1 && M < tlq::kMaxDim && N < tlq::kMaxDim)) return false;
  if ((N & 3) != 0) return M > 32;  // (fewer than 16 weight rows: the last-rows kernel alone)
  if (N <= 16) return false;
  return (N & 7) != 0 && M > 512 && ragged_result_bytes(M, N, 4) <= ((int64_t)1 << 30);
}
static int64_t row_group_for(int64_t K) {  // largest power of two dividing K, 1024 at most
  int64_t g = K & -K;
  return g > 1024 ? 1024 : g;
}
static int64_t row_group_tensor_bytes(int64_t N, int64_t K) { return (N * (K / row_group_for(K)) * 2 + 15) / 16 * 16; }

using namespace tlq;

#define TLQ_CHECK_DIMS(name)                                                                                      \
  TLQ_REQUIRE(M >= 0 && N >= 0 && K >= 0 && M < kMaxDim && N < kMaxDim && K < kMaxDim, name ": bad shape M=%lld N=%lld K=%lld", \
              (long long)M, (long long)N, (long long)K)

extern "C" {

void tlq_tune_gemm_band(int tile_rows) { tlq::g_gemm_band_rows = tile_rows < 0 ? 0 : tile_rows; }
void tlq_tune_gemm_slots(int mode) { tlq::g_gemm_slots = mode < 0 ? 0 : (mode > 2 ? 2 : mode); }
int tlq_debug_gemm_tile(int64_t batch, int64_t M, int64_t N, int fused) {
  return tlq::prefer_small_tiles(batch, M, N, fused ? 0.65 : 0.72) ? 128 : 256;
}
void tlq_tune_gemm_tile(int tile) { tlq::g_gemm_f16_tile = (tile == 128 || tile == 256) ? tile : 0; }
void tlq_tune_w4a16_stream(int on) { tlq::g_w4a16_stream = on != 0; }
void tlq_tune_w4a16_stream_slice(int steps) { tlq::g_stream_slice_steps = steps; }
void tlq_tune_w4a16_decode(int on) { tlq::g_w4a16_decode = on != 0; }
void tlq_tune_w4a16_panel(int mode) { tlq::g_w4a16_panel = mode != 0 ? 1 : 0; }
void tlq_tune_w4a16_panel_slice(int steps) { tlq::g_panel_slice_steps = tlq::g_panel2_slice_steps = tlq::g_panelm_slice_steps = steps < 0 ? 0 : steps; }
void tlq_tune_w4a16_panelm_rows(int rows) { tlq::g_panelm_rows = (rows == 64 || rows == 128) ? rows : 0; }

int tlq_debug_panel_plan(int64_t M, int64_t N, int64_t K, int64_t group, int cus, void* plan_out) {
  if (!(M >= 1 && N >= 1 && K > 0 && group > 0 && M < kMaxDim && N < kMaxDim && K < kMaxDim)) return 0;
  const PanelPlan p = w4a16_panel_plan(M, N, K, group, cus);
  if (plan_out) {
    int64_t* o = (int64_t*)plan_out;
    o[0] = p.tiles_m, o[1] = p.tiles_n, o[2] = p.split, o[3] = p.slice_steps;
  }
  return p.ok ? 1 : 0;
}

int tlq_debug_panel256_plan(int64_t M, int64_t N, int64_t K, int64_t group, int cus, void* plan_out) {
  if (!(M >= 1 && N >= 1 && K > 0 && group > 0 && M < kMaxDim && N < kMaxDim && K < kMaxDim)) return 0;
  const Panel2Plan p = w4a16_panel256_plan(M, N, K, group, cus);
  if (plan_out) {
    int64_t* o = (int64_t*)plan_out;
    o[0] = p.tiles_m, o[1] = p.tiles_n, o[2] = p.split, o[3] = p.slice_steps;
  }
  return p.ok ? 1 : 0;
}

int tlq_debug_panelm_plan(int64_t M, int64_t N, int64_t K, int64_t group, int cus, void* plan_out) {
  if (!(M >= 1 && N >= 1 && K > 0 && group > 0 && M < kMaxDim && N < kMaxDim && K < kMaxDim)) return 0;
  const PanelMPlan p = w4a16_panelm_plan(M, N, K, group, cus);
  if (plan_out) {
    int64_t* o = (int64_t*)plan_out;
    o[0] = p.tiles_m, o[1] = p.tiles_n, o[2] = p.split, o[3] = p.slice_steps, o[4] = 16 * p.tm;
  }
  return p.ok ? 1 : 0;
}

int tlq_debug_decode_plan(int64_t M, int64_t N, int64_t K, int64_t group, int cus, void* plan_out) {
  const DecodePlan p = w4a16_decode_plan(M, N, K, group, cus);
  if (plan_out) {
    int64_t* o = (int64_t*)plan_out;
    o[0] = p.mt, o[1] = p.chunks, o[2] = p.waves, o[3] = p.grid_x, o[4] = p.lds_bytes;
  }
  return p.ok ? 1 : 0;
}

// Activation rows from which the decode kernel is ahead of the GEMV kernels, whose time grows with every row: from three
// rows on, and with two rows once the weights are large enough for the second pass over them to show (measured: level at
// 4096 x 4096, 10.4 against 12.8 us (fp16) and 11.1 against 15.3 us (bf16, skinny kernel) at 11008 x 4096).
// Whether the skinny kernel's work-groups (one per 16 weight rows; one round of one per CU, or rounds of two per CU) leave a
// fifth or more of their last round's places empty.
static bool skinny_leaves_cus_idle(int64_t N) {
  if (tile_fill(1, 16, N, 16) < 0.8) return true;
  const int64_t wgs = ceil_div(N, (int64_t)16), places = 2 * cu_count_or_default();
  return wgs > places / 2 && (double)wgs / (double)(ceil_div(wgs, places) * places) < 0.8;
}
static bool decode_preferred(int64_t M, int64_t N, int64_t K) { return M > 2 || (M == 2 && N * K >= ((int64_t)1 << 24)); }

int tlq_gemm_w4a16(const void* A, const void* w_packed, const void* scales, const void* zeros, void* C, int64_t M,
                   int64_t N, int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, int algo,
                   void* stream) {
  TLQ_CHECK_DIMS("tlq_gemm_w4a16");
  TLQ_REQUIRE(in_dtype == TLQ_F16 || in_dtype == TLQ_BF16, "tlq_gemm_w4a16: in_dtype must be float16 or bfloat16 (got %d)",
              in_dtype);
  TLQ_REQUIRE(out_dtype == TLQ_F16 || out_dtype == TLQ_BF16 || out_dtype == TLQ_F32,
              "tlq_gemm_w4a16: out_dtype must be float16, bfloat16 or float32 (got %d)", out_dtype);
  TLQ_REQUIRE((algo >= TLQ_ALGO_AUTO && algo <= TLQ_ALGO_SKINNY) || algo == TLQ_ALGO_DECODE, "tlq_gemm_w4a16: bad algo %d", algo);
  if (M == 0 || N == 0) return 0;
  if (algo == TLQ_ALGO_AUTO) {
    // a tuned choice for this call signature (tlq_w4a16_choice_set) goes first; where that kernel refuses the call (its
    // shape or alignment rules: nothing launched), the rules below decide as if there were none
    const int chosen = w4a16_choice_lookup(M, N, K, group, in_dtype);
    if ((chosen >= TLQ_ALGO_GEMV && chosen <= TLQ_ALGO_SKINNY) || chosen == TLQ_ALGO_DECODE) {
      const uint64_t before = launch_count();
      const int rc = tlq_gemm_w4a16(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, chosen, stream);
      if (rc == 0 || launch_count() != before) return rc;
      set_error("%s", "");
    }
  }
  // More than 64 rows: the choice of the entry point with a workspace, called without one -- the streaming and panel kernels
  // need none where they do not cut K (4096 x 4096 x 4096 bf16: 105 us in the 256-row panel kernel against 146 us in the
  // tile kernel below, which is where that call comes back to whenever a kernel would need the workspace).
  static thread_local bool choosing_without_workspace = false;
  if (algo == TLQ_ALGO_AUTO && M > 64 && !choosing_without_workspace) {
    choosing_without_workspace = true;
    const int rc = tlq_gemm_w4a16_ws(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, TLQ_ALGO_AUTO, nullptr, 0, stream);
    choosing_without_workspace = false;
    return rc;
  }
  TLQ_REQUIRE(K > 0 && K % 64 == 0, "tlq_gemm_w4a16: K=%lld must be a positive multiple of 64", (long long)K);
  TLQ_REQUIRE(group > 0 && K % group == 0 && group % 32 == 0,
              "tlq_gemm_w4a16: group=%lld must divide K=%lld and be a multiple of 32", (long long)group, (long long)K);
  TLQ_REQUIRE(A && w_packed && C, "tlq_gemm_w4a16: null pointer");
  TLQ_REQUIRE(aligned16(A) && aligned16(w_packed) && aligned16(C), "tlq_gemm_w4a16: A, w_packed and C must be 16-byte aligned");
  TLQ_REQUIRE(((uintptr_t)scales & 1) == 0 && ((uintptr_t)zeros & 1) == 0, "tlq_gemm_w4a16: scales / zeros misaligned");
  hipStream_t st = (hipStream_t)stream;
  // The decode kernel (M <= 32): without a workspace only rows of up to 4096 values (one chunk of K).  Its scale / zero
  // gathers read aligned dwords: the tensors must start on a dword boundary (their length is checked by the plan).
  const DecodePlan dp = M <= 32 ? w4a16_decode_plan(M, N, K, group, cu_count_or_default()) : DecodePlan{false, 0, 0, 0, 0, 0};
  const bool decode_ok = dp.ok && dp.chunks == 1 && (((uintptr_t)scales | (uintptr_t)zeros) & 3) == 0;
  if (algo == TLQ_ALGO_DECODE) {
    TLQ_REQUIRE(decode_ok, "tlq_gemm_w4a16: the decode kernel needs 1 <= M <= 32, K %% 256 == 0, K <= 4096 without a workspace, a power-of-two "
                "group and dword-aligned scale / zero tensors (M=%lld N=%lld K=%lld group=%lld)", (long long)M, (long long)N, (long long)K,
                (long long)group);
    return gemm_w4a16_decode(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, TLQ_W_PLAIN, dp, nullptr, st);
  }
  if (algo == TLQ_ALGO_AUTO) {
    // The skinny kernel takes the same time for every M up to 16 (the weights bound it); the GEMV kernels grow with
    // M.  Measured crossovers: fp16 GEMV wins at M = 1, and at M = 2 while K <= 4096; the bf16 GEMV dequantises
    // element by element and wins only at M = 1 in its register-resident form (rows of up to 16384 values: level with the
    // skinny kernel on 4096 weight rows, 15 against 25 us on 5120 rows of 13824 values).
    const bool skinny_ok = M <= 64 && K % 128 == 0 && fits32(M, K * 2) && fits32(N, K / 2);
    // two fp16 activation rows on many weight rows: the ring GEMV (8.9 against 10.3 us for the decode kernel at
    // 11008 x 4096, 5.2 against 6.2 us at 8192 x 2048; with 4096 rows, one per wavefront, the decode kernel is 5 % ahead)
    if (M == 2 && N >= 8192 && gemv_ring_applies(M, N, K, group, in_dtype, scales, zeros))
      return gemv_w4a16(A, w_packed, scales, zeros, C, 1, M, N, K, group, zero_scalar, in_dtype, out_dtype, st);
    if (decode_preferred(M, N, K) && decode_ok && g_w4a16_decode)
      return gemm_w4a16_decode(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, TLQ_W_PLAIN, dp, nullptr, st);
    if (M > 4)
      algo = skinny_ok ? TLQ_ALGO_SKINNY : TLQ_ALGO_MFMA;
    else if (!skinny_ok)
      algo = TLQ_ALGO_GEMV;
    else if (in_dtype == TLQ_BF16)
      algo = (M == 1 && K <= 16384 && (group & (group - 1)) == 0) ? TLQ_ALGO_GEMV : TLQ_ALGO_SKINNY;
    else
      algo = ((M == 1 && K <= 16384) || (M == 2 && K <= 4096)) ? TLQ_ALGO_GEMV : TLQ_ALGO_SKINNY;  // (longer rows: no register-resident GEMV)
  }
  if (algo == TLQ_ALGO_SKINNY) {
    TLQ_REQUIRE(M <= 64, "tlq_gemm_w4a16: the skinny kernel handles M <= 64 (got %lld)", (long long)M);
    TLQ_REQUIRE(K % 128 == 0, "tlq_gemm_w4a16: the skinny kernel needs K %% 128 == 0 (got %lld)", (long long)K);
    TLQ_REQUIRE(fits32(M, K * 2) && fits32(N, K / 2), "tlq_gemm_w4a16: a matrix spans 4 GiB or more");
    return gemm_w4a16_skinny(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, st);
  }
  if (algo == TLQ_ALGO_GEMV) {
    TLQ_REQUIRE(M <= 16, "tlq_gemm_w4a16: the GEMV kernel handles M <= 16 (got %lld)", (long long)M);
    return gemv_w4a16(A, w_packed, scales, zeros, C, 1, M, N, K, group, zero_scalar, in_dtype, out_dtype, st);
  }
  TLQ_REQUIRE(N % 4 == 0, "tlq_gemm_w4a16: the MFMA kernel needs N %% 4 == 0 (got %lld)", (long long)N);
  TLQ_REQUIRE(fits32(M, K * 2) && fits32(N, K / 2), "tlq_gemm_w4a16: a matrix spans 4 GiB or more");
  return gemm_w4a16_mfma(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, st);
}

// M from which dequantising the whole matrix once and running the plain GEMM on it beats converting the
// weights again in every row block of the fused kernel (measured on the MLP shapes: level at M = 256 for
// N = 14336, K = 4096 and 20-40 % ahead from there on and for N = 4096, K = 14336)
static const int64_t kTwoPassMinM = 256;

// most K slices the streaming kernel may cut for any group size (the smallest group allows the shortest slices)
static int64_t stream_max_split(int64_t M, int64_t N, int64_t K) {
  int64_t most = 0;
  for (int64_t group = 32; group <= K; group *= 2) {
    if (K % group) continue;
    const StreamPlan p = w4a16_stream_plan(M, N, K, group, cu_count_or_default());  // (the count the launch plans with)
    if (p.ok && p.split > most) most = p.split;
  }
  return most;
}

// Second of the two passes: the plain GEMM on the dequantised matrix at the head of the workspace.  What the workspace
// holds beyond that matrix is room for fp32 matrices of K slices (few output tiles: tlq_gemm_f16_ws).
static int plain_gemm_on_workspace(const void* A, void* workspace, int64_t workspace_bytes, void* C, int64_t M, int64_t N,
                                   int64_t K, int in_dtype, int out_dtype, void* stream) {
  const int64_t head = (N * K * 2 + 15) / 16 * 16;
  return tlq_gemm_f16_ws(A, workspace, C, (uint8_t*)workspace + head, workspace_bytes - head, 1, M, N, K, in_dtype, out_dtype,
                         TLQ_B_NK, stream);
}

// fp32 partial sums of the K slices of the kernels for small and middle M (sized for the smallest group, which allows the
// most slices); 0 when none of them cuts K
static int64_t w4a16_partial_sum_bytes(int64_t M, int64_t N, int64_t K) {
  int64_t split = w4a16_mid_split(M, N, K, 32);
  const int64_t ssplit = stream_max_split(M, N, K);
  if (ssplit > split) split = ssplit;
  if (M <= 32) {  // the decode kernel cuts rows longer than 4096 values into chunks
    const DecodePlan dp = w4a16_decode_plan(M, N, K, 32, cu_count_or_default());
    if (dp.ok && dp.chunks > split) split = dp.chunks;
  }
  return split > 1 ? split * M * N * 4 : 0;
}

// what the panel kernel may ask of the workspace for any group size: the partial tiles of its K slices and the flag word
static int64_t panel_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (!(M >= 1 && N >= 1 && K > 0 && M < kMaxDim && N < kMaxDim && K < kMaxDim)) return 0;
  int64_t need = 0;
  for (int64_t group = 32; group <= 1024; group *= 2) {
    if (K % group != 0) continue;
    const PanelPlan pp = w4a16_panel_plan(M, N, K, group, cu_count_or_default());
    if (pp.ok) {
      const int64_t b = (pp.split > 1 ? (int64_t)pp.split * M * N * 4 : 0) + 16;
      if (b > need) need = b;
    }
    const Panel2Plan p2 = w4a16_panel256_plan(M, N, K, group, cu_count_or_default());
    if (p2.ok) {
      const int64_t b = (p2.split > 1 ? (int64_t)p2.split * M * N * 4 : 0) + 16;
      if (b > need) need = b;
    }
  }
  return need;
}

// the same for the middle-M panel kernel
static int64_t panelm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (!(M >= 1 && N >= 1 && K > 0 && M < kMaxDim && N < kMaxDim && K < kMaxDim)) return 0;
  int64_t need = 0;
  for (int64_t group = 32; group <= 1024; group *= 2) {
    if (K % group != 0) continue;
    const PanelMPlan pm = w4a16_panelm_plan(M, N, K, group, cu_count_or_default());
    if (pm.ok && pm.split > 1 && (int64_t)pm.split * M * N * 4 > need) need = (int64_t)pm.split * M * N * 4;
  }
  return need;
}

// The automatic choice takes the middle-M panel kernel from 257 to 512 activation rows on matrices of 2^25 weights or more
// (measured against the streaming kernel on five (N, K) pairs, groups of 128 and 64, fp16 with a zero-point tensor:
// 14336 x 4096 and 4096 x 14336: 43.5 - 43.9 against 45.8 - 47.0 us at 256 rows, 56 - 59 against 65 - 71 us at 384, 62 - 76 against
// 70 - 80 us at 512; 8192 x 8192: 47 / 66 / 77 against 49 / 74 / 82 us; below 256 rows and on 4096 x 4096 or 5120 x 5120 the
// streaming kernel is level or ahead by up to 15 %).  From 196 to 256 rows (two tiles of 128 rows, the second more than half
// full) the matrix has to be larger: 44 million weights with 10240 outputs or more, 56 million with fewer (10240 x 4096 at
// 196 - 252 rows: 36 - 41 us for the streaming kernel against 40 - 43 us; at 256 rows the streaming kernel takes
// 36 - 41 against 41 - 45 us on 6144 x 6144, 5120 x 8192 and 8192 x 5120 and 44 - 48 against 46 - 51 us on 7168 x 7168; at
// 200 - 248 rows the middle-M kernel takes 112 - 125 against 130 - 145 us on 28672 x 8192, 59 - 67 against 67 - 79 us on
// 28672 x 4096 and is 2 - 7 % ahead on 11008 x 4096, 12288 x 4096, 14336 x 4096, 4096 x 14336 and 8192 x 8192).
static bool panelm_preferred(int64_t M, int64_t N, int64_t K) {
  if (M < 196 || M > 512 || N * K < ((int64_t)1 << 25)) return false;
  return M > 256 || N * K >= (N >= 10240 ? 44000000 : 56000000);
}

// One tile of 128 rows (97 .. 128 activation rows) on matrices of 2^27 weights or more: the middle-M kernel is 9 - 18 % ahead of
// the streaming kernel (N = 50304, K = 4096, M = 128: 64.5 against 76.1 us; N = 65536, K = 8192: 144 against 154 us;
// N = 28672, K = 8192, M = 112: 74 against 82 us; N = 8192, K = 28672: 76 against 81 us; level at 64 and 96 rows).
static bool panelm_one_tile(int64_t M, int64_t N, int64_t K) { return M > 96 && M <= 128 && N * K >= ((int64_t)1 << 27); }

// 65 .. 128 rows on output-layer widths: the 128-row panel kernel, whose work-groups own 512 weight rows, where they fill more
// than five eighths of the machine in ONE round -- the streaming kernel's work-groups (256 weight rows) then need two, the second
// one partly empty (N = 102400, K = 4096, M = 96: 106 against 124 us; K = 5120: 133 against 159 us; N = 128256, K = 4096: 123
// against 136 us; N = 81920: 100 against 111 us).  Not with longer rows (N = 81920, K = 8192: 208 against 204 us).
static bool panel_one_round(int64_t M, int64_t N, int64_t K) {
  const int64_t cus_now = cu_count_or_default();
  const int64_t tiles = ceil_div(N, (int64_t)512);
  return M > 64 && M <= 128 && K <= 5120 && tiles <= cus_now && tiles * 8 >= cus_now * 5;
}

// What an explicitly named kernel family may ask of the workspace for any group size.
int64_t tlq_w4a16_workspace_bytes_for(int64_t M, int64_t N, int64_t K, int algo) {
  if (M <= 0 || N <= 0 || K <= 0 || M >= kMaxDim || N >= kMaxDim || K >= kMaxDim) return 0;
  switch (algo) {
    case TLQ_ALGO_AUTO: return tlq_w4a16_workspace_bytes(M, N, K);
    case TLQ_ALGO_TWO_PASS: return (N * K * 2 + 15) / 16 * 16 + tlq_f16_workspace_bytes(1, M, N, K);
    case TLQ_ALGO_STREAM: {
      const int64_t split = stream_max_split(M, N, K);
      return split > 1 ? split * M * N * 4 : 0;
    }
    case TLQ_ALGO_DECODE: {
      if (M > 32) return 0;
      const DecodePlan dp = w4a16_decode_plan(M, N, K, 32, cu_count_or_default());
      return dp.ok && dp.chunks > 1 ? (int64_t)dp.chunks * M * N * 4 : 0;
    }
    case TLQ_ALGO_MFMA: {  // with a workspace the tile kernel runs over K slices where it has few output tiles
      const int64_t split = w4a16_mid_split(M, N, K, 32);
      return split > 1 ? split * M * N * 4 : 0;
    }
    case TLQ_ALGO_PANEL:
    case TLQ_ALGO_PANEL256: return panel_workspace_bytes(M, N, K);
    case TLQ_ALGO_PANELM: return panelm_workspace_bytes(M, N, K);
    default: return 0;  // GEMV, skinny: no workspace
  }
}

static int64_t w4a16_kernel_workspace_bytes(int64_t M, int64_t N, int64_t K);
int64_t tlq_w4a16_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (N <= 0 || K <= 0) return 0;
  int64_t need = w4a16_kernel_workspace_bytes(M, N, K);
  // (a weight-row count that is no multiple of four: what the multiple of 16 below asks for, then its packed result, sized for fp32)
  if (ragged_rows_apply(M, N)) need = ragged_head(N) == 0 ? 0 : (w4a16_kernel_workspace_bytes(M, ragged_head(N), K) + 15) / 16 * 16 + ragged_result_bytes(M, N, 4);
  // (rows whose length is no power of two with one group per row: room behind everything else for the scales and zero points
  // written out per power-of-two group)
  if ((K & (K - 1)) != 0 && K % 64 == 0) return (need + 15) / 16 * 16 + 2 * row_group_tensor_bytes(N, K) + 16;
  return need;
}
// what the kernels themselves may ask for
static int64_t w4a16_kernel_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  int64_t need = w4a16_partial_sum_bytes(M, N, K);
  // (above 512 rows a row count that is no multiple of four runs as the multiple below plus a tail: room for that call)
  if (M > 512 && (M & 3) != 0) {
    const int64_t head = w4a16_kernel_workspace_bytes(M & ~(int64_t)3, N, K);
    if (head > need) need = head;
  }
  // tuned choices for this shape (any group, any type): room for the chosen family as well
  int64_t tuned[4] = {0, M, N, K};
  w4a16_choice_for_shape(M, N, K, [](int algo, void* ctx) {
    int64_t* const n = (int64_t*)ctx;
    if (algo == TLQ_ALGO_AUTO) return;
    const int64_t b = tlq_w4a16_workspace_bytes_for(n[1], n[2], n[3], algo);
    if (b > n[0]) n[0] = b;
  }, tuned);
  if (tuned[0] > need) need = tuned[0];
  if (panelm_preferred(M, N, K) || panelm_one_tile(M, N, K) || M > 512) {  // (above 512 rows: where its estimate beats the 256-row kernel's)
    const int64_t pm = panelm_workspace_bytes(M, N, K);
    if (pm > need) need = pm;
  }
  if (M > 128 || panelm_preferred(M, N, K) || panel_one_round(M, N, K)) {  // (129 .. 512 rows: where the 256-row kernel's estimate beats the middle-M or the streaming kernel's)
    const int64_t pn = panel_workspace_bytes(M, N, K);
    if (pn > need) need = pn;
  }
  // two passes (which of the two is taken depends on the group size, so the size covers both): the dequantised matrix,
  // then room for the K slices of the plain GEMM where it has few output tiles
  if (M >= kTwoPassMinM) {
    const int64_t two = (N * K * 2 + 15) / 16 * 16 + tlq_f16_workspace_bytes(1, M, N, K);
    if (two > need) need = two;
  }
  return need;
}

int64_t tlq_w4a16_workspace_bytes_min(int64_t M, int64_t N, int64_t K) {
  if (N <= 0 || K <= 0) return 0;
  const int64_t partial = w4a16_partial_sum_bytes(M, N, K);
  if (partial > 0) return partial;
  return M >= kTwoPassMinM ? N * K * 2 : 0;
}

// Estimated time of a panel kernel's launch (us): rounds of work-groups x (steps per K slice x step time + fixed part), plus
// the pass that adds the slices' partial tiles (a launch, their write and their read) where K is cut.
static double panel_estimate_us(int tiles_m, int tiles_n, int split, int slice_steps, double step_us, double fixed_us, int64_t M,
                                int64_t N, int64_t cus) {
  const int64_t wgs = (int64_t)tiles_m * tiles_n * split;
  const double rounds = (double)ceil_div(wgs, cus);
  return rounds * ((double)slice_steps * step_us + fixed_us) + (split > 1 ? 3.0 + (double)(split + 1) * (double)M * (double)N * 4.0 / 4e6 : 0.0);
}
// Above 512 rows: does the middle-M kernel (128-row tiles) beat the 256-row kernel by estimate?
static bool panelm_estimate_wins(int64_t M, int64_t N, int64_t K, int64_t group) {
  const int64_t cus_now = cu_count_or_default();
  const PanelMPlan pm = w4a16_panelm_plan(M, N, K, group, (int)cus_now);
  const Panel2Plan p2 = w4a16_panel256_plan(M, N, K, group, (int)cus_now);
  if (!pm.ok || !p2.ok || pm.tm != 8) return false;
  const double est_m = panel_estimate_us(pm.tiles_m, pm.tiles_n, pm.split, pm.slice_steps, 2.2, 6.0, M, N, cus_now);
  const double est_2 = panel_estimate_us(p2.tiles_m, p2.tiles_n, p2.split, p2.slice_steps, 3.3, 8.0, M, N, cus_now);
  return est_m < 0.94 * est_2;
}
// 256 .. 512 rows: does the 256-row kernel beat the middle-M kernel by the same estimate?
static bool panel256_estimate_wins(int64_t M, int64_t N, int64_t K, int64_t group) {
  const int64_t cus_now = cu_count_or_default();
  const PanelMPlan pm = w4a16_panelm_plan(M, N, K, group, (int)cus_now);
  const Panel2Plan p2 = w4a16_panel256_plan(M, N, K, group, (int)cus_now);
  if (!pm.ok || !p2.ok) return false;
  const double est_m = panel_estimate_us(pm.tiles_m, pm.tiles_n, pm.split, pm.slice_steps, pm.tm == 8 ? 2.2 : 1.8, 6.0, M, N, cus_now);
  const double est_2 = panel_estimate_us(p2.tiles_m, p2.tiles_n, p2.split, p2.slice_steps, 3.3, 8.0, M, N, cus_now);
  return est_2 < 0.9 * est_m;
}

// 257 .. 512 rows: does the 256-row kernel beat the streaming kernel's blocks of 128 rows by the same estimate (a streaming
// step of a 128-row block: 2.2 us, fixed part 8 us)?  It matters where the middle-M kernel does not take K (group counts
// that are no multiple of eight) and four blocks of 128 rows meet two tiles of 256: N = 5120, K = 13824, M = 448 - 512:
// 82 - 85 against 102 us; N = 3584, K = 18944: 81 - 85 against 102 - 106 us; N = 18944, K = 3584: 82 against 118 - 128 us;
// on 30 measured cases the estimated ratio is 4 - 25 % above the measured one, hence the bar of 0.95 (N = 8192, K = 6912,
// where the 256-row kernel is 2 - 5 % ahead, stays with the streaming kernel; N = 4096, K = 11008, where it is 6 % behind, too).
static bool panel256_beats_stream(int64_t M, int64_t N, int64_t K, int64_t group, const StreamPlan& sp) {
  // (256 rows: one tile against two blocks -- N = 151936, K = 3584: 278 against 333 us; 129 .. 192 rows in two blocks of 96
  // rows, 1.75 us a step, on very wide matrices: N = 50304 .. 128256, K = 4096 .. 8192, M = 160: 100 - 238 against 128 - 277 us)
  if (M <= 128 || !sp.ok || (sp.tm != 8 && sp.tm != 6)) return false;
  const int64_t cus_now = cu_count_or_default();
  const Panel2Plan p2 = w4a16_panel256_plan(M, N, K, group, (int)cus_now);
  if (!p2.ok) return false;
  const double est_s = panel_estimate_us(sp.m_blocks, sp.n_blocks, sp.split, sp.slice_steps, sp.tm == 8 ? 2.2 : 1.75, 8.0, M, N, cus_now);
  const double est_2 = panel_estimate_us(p2.tiles_m, p2.tiles_n, p2.split, p2.slice_steps, 3.3, 8.0, M, N, cus_now);
  return est_2 < 0.95 * est_s;
}

// The automatic choice takes the 256-row panel kernel where the last round of its work-groups fills more than half of the CUs
// (measured: 2 - 21 % behind the two passes at 0.375 -- 96 work-groups --, 3 % behind at exactly one half, ahead from there on:
// N = 11008, K = 4096, M = 768, 129 work-groups: 92 against 107 us).
static const double kPanel256Fill = 0.502;
static bool panel256_fills(int64_t M, int64_t N, int64_t K, int64_t group) {
  const int64_t cus_now = cu_count_or_default();
  const Panel2Plan pp = w4a16_panel256_plan(M, N, K, group, (int)cus_now);
  if (!pp.ok) return false;
  const int64_t wgs = (int64_t)pp.tiles_m * pp.tiles_n * pp.split;
  return (double)wgs / (double)(ceil_div(wgs, cus_now) * cus_now) >= kPanel256Fill;
}

// The panel kernel (large M, one launch, weights dequantised on the operand read).  Returns -1 when it does not take the
// problem (nothing launched, no error set), else the launch's return code.
static int try_panel(const void* A, const void* w_packed, const void* scales, const void* zeros, void* C, int64_t M, int64_t N,
                     int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, int w_layout, void* workspace,
                     int64_t workspace_bytes, void* stream) {
  if (!(M >= 1 && N >= 1 && K > 0 && group > 0 && M < kMaxDim && N < kMaxDim && K < kMaxDim)) return -1;
  const PanelPlan pp = w4a16_panel_plan(M, N, K, group, cu_count_or_default());
  if (!pp.ok) return -1;
  const bool args_ok = A && w_packed && C && aligned16(A) && aligned16(w_packed) && aligned16(C) && aligned16(scales) &&
                       aligned16(zeros) && (in_dtype == TLQ_F16 || in_dtype == TLQ_BF16) &&
                       (out_dtype == TLQ_F16 || out_dtype == TLQ_BF16 || out_dtype == TLQ_F32) && (M * N) % 4 == 0 &&
                       fits32(M, K * 2) && fits32(N, K / 2) && fits32(N, (K / group) * 2);
  if (!args_ok) return -1;
  // workspace: the partial tiles of the K slices, then (with a zero-point tensor) one word for the kernel's flag
  const int64_t part_bytes = pp.split > 1 ? (int64_t)pp.split * M * N * 4 : 0;
  const int64_t need = part_bytes + (zeros ? 16 : 0);
  if (need > 0 && !(workspace && aligned16(workspace) && workspace_bytes >= need)) return -1;
  return gemm_w4a16_panel(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, w_layout, pp,
                          (float*)workspace, zeros ? (uint32_t*)((uint8_t*)workspace + part_bytes) : nullptr, (hipStream_t)stream);
}

// The 256-row panel kernel: the same contract.
static int try_panel256(const void* A, const void* w_packed, const void* scales, const void* zeros, void* C, int64_t M, int64_t N,
                        int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, int w_layout, void* workspace,
                        int64_t workspace_bytes, void* stream) {
  if (!(M >= 1 && N >= 1 && K > 0 && group > 0 && M < kMaxDim && N < kMaxDim && K < kMaxDim)) return -1;
  const Panel2Plan pp = w4a16_panel256_plan(M, N, K, group, cu_count_or_default());
  if (!pp.ok) return -1;
  const bool args_ok = A && w_packed && C && aligned16(A) && aligned16(w_packed) && aligned16(C) && ((uintptr_t)scales & 1) == 0 &&
                       ((uintptr_t)zeros & 1) == 0 && (in_dtype == TLQ_F16 || in_dtype == TLQ_BF16) &&
                       (out_dtype == TLQ_F16 || out_dtype == TLQ_BF16 || out_dtype == TLQ_F32) && (M * N) % 4 == 0 &&
                       fits32(M, K * 2) && fits32(N, K / 2) && fits32(N, (K / group) * 2);
  if (!args_ok) return -1;
  const int64_t need = pp.split > 1 ? (int64_t)pp.split * M * N * 4 : 0;
  if (need > 0 && !(workspace && aligned16(workspace) && workspace_bytes >= need)) return -1;
  return gemm_w4a16_panel256(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, w_layout, pp,
                             (float*)workspace, (hipStream_t)stream);
}

// The middle-M panel kernel.  Returns -1 when it does not take the problem (nothing launched, no error set).
static int try_panelm(const void* A, const void* w_packed, const void* scales, const void* zeros, void* C, int64_t M, int64_t N,
                      int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, void* workspace,
                      int64_t workspace_bytes, void* stream) {
  if (!(M >= 1 && N >= 1 && K > 0 && group > 0 && M < kMaxDim && N < kMaxDim && K < kMaxDim)) return -1;
  const PanelMPlan pp = w4a16_panelm_plan(M, N, K, group, cu_count_or_default());
  if (!pp.ok) return -1;
  const bool args_ok = A && w_packed && C && aligned16(A) && aligned16(w_packed) && aligned16(C) && aligned16(scales) &&
                       aligned16(zeros) && (in_dtype == TLQ_F16 || in_dtype == TLQ_BF16) &&
                       (out_dtype == TLQ_F16 || out_dtype == TLQ_BF16 || out_dtype == TLQ_F32) && (M * N) % 4 == 0 &&
                       fits32(M, K * 2) && fits32(N, K / 2) && fits32(N, (K / group) * 2);
  if (!args_ok) return -1;
  const int64_t need = pp.split > 1 ? (int64_t)pp.split * M * N * 4 : 0;
  if (need > 0 && !(workspace && aligned16(workspace) && workspace_bytes >= need)) return -1;
  return gemm_w4a16_panelm(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, pp, (float*)workspace,
                           (hipStream_t)stream);
}

// One group per weight row on rows whose length is no power of two (K = 11008, 5120, 3584 ...): only the oldest kernels take
// such a group (M = 64, N = 4096, K = 11008: 59 us against 23 us with groups of 128).  The row's scale / zero point is
// written out per power-of-two group into the tail of the workspace (one small launch per tensor) and the call goes on with
// that group and the workspace in front of the tail.  Returns 0 where that does not apply (no such group, no room: the call
// goes on as it is), 1 with `out` filled in, -1 after a failed launch.
struct RowValues {
  const void* scales;
  const void* zeros;
  int64_t group, workspace_bytes;
};
static int write_out_row_values(const void* scales, const void* zeros, int64_t M, int64_t N, int64_t K, int64_t group, int in_dtype,
                                void* workspace, int64_t workspace_bytes, void* stream, RowValues& out) {
  if (!(M >= 1 && N >= 1 && N < kMaxDim && K >= 64 && K < kMaxDim && group == K && (K & (K - 1)) != 0 && K % 64 == 0 &&
        (in_dtype == TLQ_F16 || in_dtype == TLQ_BF16)))
    return 0;
  const int64_t g_eff = row_group_for(K), groups = K / g_eff, tensor_bytes = row_group_tensor_bytes(N, K);
  out = RowValues{scales, zeros, g_eff, workspace_bytes};
  if (!scales && !zeros) return 1;  // no tensors: any group size says the same
  const int64_t tail = ((scales ? 1 : 0) + (zeros ? 1 : 0)) * tensor_bytes;
  const int64_t head_bytes = (workspace_bytes - tail) & ~(int64_t)15;
  if (!(workspace && aligned16(workspace) && workspace_bytes >= tail + 16 && ((uintptr_t)scales & 1) == 0 && ((uintptr_t)zeros & 1) == 0)) return 0;
  uint8_t* const base = (uint8_t*)workspace + head_bytes;
  const int64_t n_out = N * groups;
  const int grid = (int)((n_out + 255) / 256 > 4096 ? 4096 : (n_out + 255) / 256);
  if (scales) {
    expand_row_values_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const uint16_t*)scales, (uint16_t*)base, n_out, (int)groups);
    if (!check_launch("tlq_gemm_w4a16 (one scale per row, written out per group)", "expand_row_values_kernel")) return -1;
    out.scales = base;
  }
  if (zeros) {
    uint8_t* const zb = base + (scales ? tensor_bytes : 0);
    expand_row_values_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const uint16_t*)zeros, (uint16_t*)zb, n_out, (int)groups);
    if (!check_launch("tlq_gemm_w4a16 (one zero point per row, written out per group)", "expand_row_values_kernel")) return -1;
    out.zeros = zb;
  }
  out.workspace_bytes = head_bytes;
  return 1;
}

// A weight-row count that is no multiple of four, more than 32 activation rows: only the skinny kernel (up to 64 rows) takes it as
// it is (N = 32001, K = 4096, M = 64: 88 us against 42 us for N = 32000; more rows were refused).  With room behind the workspace
// for the packed result of the first N - N % 16 rows: those through the usual choice, a copy into C, the last rows straight into C.
// `taken` says whether the call was answered here (the return value is then its result).
static int run_ragged_rows(const void* A, const void* w_packed, const void* scales, const void* zeros, void* C, int64_t M, int64_t N, int64_t K,
                           int64_t group, float zero_scalar, int in_dtype, int out_dtype, int w_layout, void* workspace, int64_t workspace_bytes,
                           void* stream, bool& taken) {
  taken = false;
  if (!(ragged_rows_apply(M, N) && K > 0 && K % 64 == 0 && group > 0 && K % group == 0 && group % 32 == 0 && A && w_packed && C &&
        (in_dtype == TLQ_F16 || in_dtype == TLQ_BF16) && (out_dtype == TLQ_F16 || out_dtype == TLQ_BF16 || out_dtype == TLQ_F32) &&
        ((uintptr_t)scales & 1) == 0 && ((uintptr_t)zeros & 1) == 0 && aligned16(A) && aligned16(w_packed) && aligned16(C)))
    return 0;
  const int out_bytes = out_dtype == TLQ_F32 ? 4 : 2;
  const int64_t head = ragged_head(N), result_bytes = ragged_result_bytes(M, N, out_bytes);
  if (!(head == 0 || (workspace && aligned16(workspace) && workspace_bytes >= result_bytes))) return 0;
  taken = true;
  const int64_t front = head == 0 ? 0 : (workspace_bytes - result_bytes) & ~(int64_t)15;
  uint8_t* const packed = (uint8_t*)workspace + front;
  const int64_t groups = K / group;
  if (head > 0) {
    if (int rc = tlq_gemm_w4a16_layout_ws(A, w_packed, scales, zeros, packed, M, head, K, group, zero_scalar, in_dtype, out_dtype, TLQ_ALGO_AUTO, w_layout,
                                          workspace, front, stream))
      return rc;
    const dim3 grid((unsigned)ceil_div(head, (int64_t)256), (unsigned)(M > 4096 ? 4096 : M));
    if (out_bytes == 4)
      copy_into_wider_rows_kernel<uint32_t><<<grid, 256, 0, (hipStream_t)stream>>>((const uint32_t*)packed, (uint32_t*)C, M, head, N);
    else
      copy_pairs_into_wider_rows_kernel<<<dim3((unsigned)ceil_div(head / 2 + 1, (int64_t)256), grid.y), 256, 0, (hipStream_t)stream>>>(
          (const uint16_t*)packed, (uint16_t*)C, M, head, N);
    if (!check_launch("tlq_gemm_w4a16 (packed result into C)", out_bytes == 4 ? "copy_into_wider_rows_kernel" : "copy_pairs_into_wider_rows_kernel")) return 1;
  }
  const int eb = 2;  // scales and zero points: 16-bit values
  return w4a16_tail_rows(A, (const uint8_t*)w_packed + head * (K / 2), scales ? (const uint8_t*)scales + head * groups * eb : nullptr,
                         zeros ? (const uint8_t*)zeros + head * groups * eb : nullptr, C, M, N - head, K, group, zero_scalar, in_dtype, out_dtype, w_layout, N,
                         head, (hipStream_t)stream);
}

int tlq_gemm_w4a16_ws(const void* A, const void* w_packed, const void* scales, const void* zeros, void* C, int64_t M,
                      int64_t N, int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, int algo,
                      void* workspace, int64_t workspace_bytes, void* stream) {
  TLQ_REQUIRE(algo >= TLQ_ALGO_AUTO && algo <= TLQ_ALGO_PANELM, "tlq_gemm_w4a16_ws: bad algo %d", algo);
  if (algo != TLQ_ALGO_TWO_PASS) {  // (not for the two passes by name: their dequantisation pass takes any group as it is)
    RowValues rv;
    const int wrote = write_out_row_values(scales, zeros, M, N, K, group, in_dtype, workspace, workspace_bytes, stream, rv);
    if (wrote < 0) return 1;
    if (wrote > 0)
      return tlq_gemm_w4a16_ws(A, w_packed, rv.scales, rv.zeros, C, M, N, K, rv.group, zero_scalar, in_dtype, out_dtype, algo, workspace, rv.workspace_bytes, stream);
  }
  if (algo == TLQ_ALGO_AUTO) {
    bool taken = false;
    const int rc = run_ragged_rows(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, TLQ_W_PLAIN, workspace, workspace_bytes, stream, taken);
    if (taken) return rc;
  }
  if (algo == TLQ_ALGO_AUTO && M >= 1 && N >= 1) {
    // a tuned choice for this call signature goes first (as in tlq_gemm_w4a16); a kernel that refuses the call -- its shape
    // rules, the alignment of an operand, a workspace smaller than it needs -- has launched nothing, and the rules decide
    const int chosen = w4a16_choice_lookup(M, N, K, group, in_dtype);
    if (chosen != TLQ_ALGO_AUTO) {
      const uint64_t before = launch_count();
      const int rc = tlq_gemm_w4a16_ws(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, chosen, workspace,
                                       workspace_bytes, stream);
      if (rc == 0 || launch_count() != before) return rc;
      set_error("%s", "");
    }
  }
  // Above 512 rows the panel kernels are the fast path, and they take row counts that are multiples of four (their direct
  // loads move four activation rows).  Any other count -- prompt lengths are what they are -- runs as its multiple of four
  // below through the same choice plus the last one to three rows through the small-M kernels, which is one short launch
  // more instead of the two passes for everything (measured: M = 1001, N = 14336, K = 4096: 147 us in one piece, 128 us for
  // 1000 rows; M = 2049, N = K = 8192: 392 against 249 us; M = 601, N = K = 8192: 164 against 120 us; the tail takes 6 - 15 us).
  if (algo == TLQ_ALGO_AUTO && !g_w4a16_panel && M > 512 && (M & 3) != 0 && M < kMaxDim && N >= 16 && N % 16 == 0 && N < kMaxDim && K > 0 &&
      K < kMaxDim && group > 0 && A && C && (in_dtype == TLQ_F16 || in_dtype == TLQ_BF16) &&
      (out_dtype == TLQ_F16 || out_dtype == TLQ_BF16 || out_dtype == TLQ_F32)) {
    const int64_t head = M & ~(int64_t)3;
    if (w4a16_panel256_plan(head, N, K, group, cu_count_or_default()).ok) {
      const int rc = tlq_gemm_w4a16_ws(A, w_packed, scales, zeros, C, head, N, K, group, zero_scalar, in_dtype, out_dtype, TLQ_ALGO_AUTO, workspace,
                                       workspace_bytes, stream);
      if (rc != 0) return rc;
      const int64_t out_bytes = out_dtype == TLQ_F32 ? 4 : 2;
      return tlq_gemm_w4a16((const uint8_t*)A + head * K * 2, w_packed, scales, zeros, (uint8_t*)C + head * N * out_bytes, M - head, N, K, group,
                            zero_scalar, in_dtype, out_dtype, TLQ_ALGO_AUTO, stream);
    }
  }
  if (algo == TLQ_ALGO_PANELM) {
    const int rc = try_panelm(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, workspace, workspace_bytes, stream);
    TLQ_REQUIRE(rc >= 0, "tlq_gemm_w4a16_ws: the middle-M panel kernel needs K %% 128 == 0, M %% 4 == 0, N %% 16 == 0, a power-of-two group "
                ">= 64 with (K / group) %% 8 == 0, 16-byte aligned operands, scale and zero tensors, and a workspace for its K slices (M=%lld "
                "N=%lld K=%lld group=%lld, workspace %lld)", (long long)M, (long long)N, (long long)K, (long long)group, (long long)workspace_bytes);
    return rc;
  }
  if (algo == TLQ_ALGO_PANEL256) {
    const int rc = try_panel256(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, TLQ_W_PLAIN, workspace,
                                workspace_bytes, stream);
    TLQ_REQUIRE(rc >= 0, "tlq_gemm_w4a16_ws: the 256-row panel kernel needs K %% 128 == 0, M %% 4 == 0, N %% 16 == 0, a power-of-two group "
                ">= 32, 16-byte aligned operands and a workspace for its K slices (M=%lld "
                "N=%lld K=%lld group=%lld, workspace %lld)", (long long)M, (long long)N, (long long)K, (long long)group, (long long)workspace_bytes);
    return rc;
  }
  if (algo == TLQ_ALGO_PANEL) {
    const int rc = try_panel(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, TLQ_W_PLAIN, workspace,
                             workspace_bytes, stream);
    TLQ_REQUIRE(rc >= 0, "tlq_gemm_w4a16_ws: the panel kernel needs K %% 128 == 0, M %% 4 == 0, N %% 16 == 0, a power-of-two group >= 32 "
                "with (K / group) %% 8 == 0, 16-byte aligned operands, scale and zero tensors, and a workspace for its K slices and (with a "
                "zero-point tensor) 16 bytes more (M=%lld N=%lld K=%lld group=%lld, workspace %lld)", (long long)M, (long long)N, (long long)K, (long long)group, (long long)workspace_bytes);
    return rc;
  }
  // decode batches: rows longer than 4096 values run as chunks of K whose fp32 partial sums live in the workspace
  if (((algo == TLQ_ALGO_AUTO && g_w4a16_decode && (decode_preferred(M, N, K) || K > 16384)) || algo == TLQ_ALGO_DECODE) && M <= 32 && M >= 1 && N >= 1 && K > 0 && group > 0 &&
      N < kMaxDim && K < kMaxDim) {
    const DecodePlan dp = w4a16_decode_plan(M, N, K, group, cu_count_or_default());
    const bool args_ok = A && w_packed && C && aligned16(A) && aligned16(w_packed) && aligned16(C) &&
                         (in_dtype == TLQ_F16 || in_dtype == TLQ_BF16) &&
                         (out_dtype == TLQ_F16 || out_dtype == TLQ_BF16 || out_dtype == TLQ_F32) &&
                         (((uintptr_t)scales | (uintptr_t)zeros) & 3) == 0;
    // measured on rows of 14336 values: with up to 16 activation rows the skinny kernel is level or ahead (no second
    // launch for the partial sums), from 17 rows on the decode kernel is 10 - 15 % ahead of the streaming kernel
    // (also for rows of more than 16384 values, which the register-resident GEMV does not take: M = 1, N = 8192,
    // K = 28672: 32 against 49 us for the generic GEMV;
    // from 64 MB of weights on -- N = 28672, K = 8192, M = 16: 31.6 against 45.6 us -- and where the skinny kernel's
    // work-groups, one per 16 weight rows, would leave a fifth of the machine or more idle in their last round:
    // N = 5120, K = 13824: 15.8 against 23.6 us; with 8192 or 13824 weight rows the skinny kernel is level or ahead.
    // Two of its work-groups share a CU, so that holds for rounds of twice the CU count as well: N = 10240, K = 8192
    // (640 work-groups on 512 places): 15 against 20 - 26 us; N = 12288, K = 6144 (768): 14 - 15 against 17 - 21 us;
    // N = 17408, K = 5120 (1088): 17 - 19 against 20 - 24 us; with 512 or 960 work-groups the skinny kernel is ahead)
    if (dp.ok && dp.chunks > 1 && (algo == TLQ_ALGO_DECODE || M > 16 || K > 16384 || N * (K / 2) >= ((int64_t)64 << 20) || skinny_leaves_cus_idle(N)) && args_ok && (M * N) % 4 == 0 && workspace && aligned16(workspace) &&
        workspace_bytes >= (int64_t)dp.chunks * M * N * 4)
      return gemm_w4a16_decode(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, TLQ_W_PLAIN, dp,
                               (float*)workspace, (hipStream_t)stream);
    if (algo == TLQ_ALGO_DECODE && !(dp.ok && dp.chunks == 1)) {
      set_error("tlq_gemm_w4a16_ws: the decode kernel needs 1 <= M <= 32, K %% 256 == 0, a power-of-two group, dword-aligned scale / zero "
                "tensors, M * N %% 4 == 0 and a workspace of %lld bytes (M=%lld N=%lld K=%lld group=%lld, workspace %lld)",
                (long long)(dp.ok ? (int64_t)dp.chunks * M * N * 4 : 0), (long long)M, (long long)N, (long long)K, (long long)group,
                (long long)workspace_bytes);
      return 1;
    }
  }
  if (algo == TLQ_ALGO_AUTO && M >= 1 && N >= 1 && K > 0 && N < kMaxDim && K < kMaxDim) {
    // Small problems are launch-bound: a second launch (for the partial sums of K slices, or for the dequantisation
    // pass) costs more than it saves.  Measured: 256^3 6.5 against 9.5 us, M = 128 on 1024 x 512 9.7 against 12.4 us,
    // M = 64 on 1024^2 6.7 against 11.4 us and on 2048^2 11.0 against 13.0 us; the streaming kernel with its K slices is
    // ahead from M = 256 on 1024^2 (15.5 against 20.8 us) and for M = 40 on 1024 rows of 4096 values (13.0 against 16.5 us).
    // Short rows (K <= 2048) on up to 2^24 weights, 33 .. 64 activation rows: the skinny kernel's single launch is ahead of the
    // streaming kernel, whose launch has 8 us that do not depend on K (N = 8192, K = 1024: 7.9 / 8.4 against 12.5 / 13.4 us at
    // 40 / 64 rows; N = 16384, K = 1024: 10.7 / 12.4 against 13.8 / 15.6 us; N = 8192, K = 2048: 12.0 / 14.9 against 14.7 / 16.4 us;
    // behind from 2^25 weights on and with rows of 3072 values).
    const int64_t nk = N * K;
    // (rows of more than 1280 values only where the skinny kernel's work-groups, one per 16 weight rows, run in one round or
    // fill their last round: N = 6144, K = 2048, 384 work-groups: 16 - 22 against 14 - 15 us)
    const bool skinny_fills = ceil_div(N, (int64_t)16) <= cu_count_or_default() || tile_fill(1, 16, N, 16) >= 0.8;
    if ((M <= 64 && (nk <= ((int64_t)1 << 21) || (nk <= ((int64_t)1 << 24) && (K <= 1280 || (K <= 2048 && skinny_fills))))) || nk <= ((int64_t)1 << 19))
      return tlq_gemm_w4a16(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, TLQ_ALGO_AUTO, stream);
    // Short rows, 96 .. 512 activation rows, one round of 128 x 128 tiles: the tile kernel in one launch takes 4.5 us + 1.45 us
    // per 128 values of K whatever M and N, the streaming kernel 11 - 15 us at K = 512 and 19 - 30 us at K = 1024 .. 1536.
    // Measured on five values of N from 2048 to 32768 x six of M: ahead by 1.1 - 1.4 x on all 23 cases at K = 512, by
    // 1.07 - 1.4 x at K = 1024 from 96 tiles on (level or behind with 64 tiles and fewer), by 1.1 - 1.27 x at K = 1536 from 128
    // tiles and 128 rows on; behind at K = 2048.  (Groups of 32 values at K = 1024: from 192 tiles on; fp16 with a zero-point
    // tensor is 3 - 16 % behind on 96 - 128 tiles.)  Out of sample (eight values of K from 384 to 2560 x seven of N x seven of M, both
    // types, against the build before): 1.1 - 1.5 x on the cases that change, none more than 3 % slower.
    const int64_t tiles128 = ceil_div(M, (int64_t)128) * ceil_div(N, (int64_t)128);
    if (M >= 96 && M <= 512 && N % 4 == 0 && tiles128 <= cu_count_or_default() &&
        (K <= 512 || (K <= 768 && tiles128 >= 96) || (K <= 1024 && tiles128 >= (group < 64 ? 192 : 96)) || (K <= 1536 && tiles128 >= 128 && (M == 128 || M > 192))))  // (129 .. 192 rows: the streaming kernel's blocks of 96 rows are level there)
      return tlq_gemm_w4a16(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, TLQ_ALGO_MFMA, stream);
    // 17 .. 32 activation rows whose K is one chunk of the decode kernel: that kernel, which needs no workspace
    // (M = 32, N = 14336, K = 4096: 16.8 against 20 us for the streaming kernel)
    if (M > 16 && M <= 32 && g_w4a16_decode && group > 0) {
      const DecodePlan dp = w4a16_decode_plan(M, N, K, group, cu_count_or_default());
      if (dp.ok && dp.chunks == 1 && (((uintptr_t)scales | (uintptr_t)zeros) & 3) == 0)
        return tlq_gemm_w4a16(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, TLQ_ALGO_AUTO, stream);
    }
  }
  const int64_t need = (N > 0 && K > 0) ? N * K * 2 : 0;
  const bool have = workspace != nullptr && workspace_bytes >= need && aligned16(workspace);
  if (algo == TLQ_ALGO_TWO_PASS)
    TLQ_REQUIRE(have, "tlq_gemm_w4a16_ws: the two-pass path needs a 16-byte aligned workspace of %lld bytes (got %lld)",
                (long long)need, (long long)workspace_bytes);
  // 256 .. 512 activation rows on large matrices: the middle-M panel kernel
  // (not up to 256 rows with groups of 512 values or more: the panel kernels cut K into windows of eight groups -- 32 steps and
  // more -- and run uncut or nearly so, the streaming kernel cuts inside a group: N = 14336, K = 4096, M = 256: 50 against 59 us;
  // N = 11008: 47 against 58 us; N = K = 8192: 52 against 61 us; from 384 rows on the panel kernels are ahead again)
  if (algo == TLQ_ALGO_AUTO && !g_w4a16_panel && panelm_preferred(M, N, K) && group > 0 && !(M <= 256 && group >= 512)) {
    // (very wide matrices: where the 128-row tiles need a second round of work-groups and the 256-row tiles do not, the
    // 256-row kernel by the same estimate -- N = 28672, K = 4096, M = 512: 104 against 129 us)
    if (panel256_estimate_wins(M, N, K, group)) {
      const int rc = try_panel256(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, TLQ_W_PLAIN, workspace,
                                  workspace_bytes, stream);
      if (rc >= 0) return rc;
    }
    const int rc = try_panelm(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, workspace, workspace_bytes, stream);
    if (rc >= 0) return rc;
  }
  if (algo == TLQ_ALGO_AUTO && !g_w4a16_panel && panel_one_round(M, N, K) && group > 0) {
    const int rc = try_panel(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, TLQ_W_PLAIN, workspace, workspace_bytes, stream);
    if (rc >= 0) return rc;
  }
  if (algo == TLQ_ALGO_AUTO && !g_w4a16_panel && panelm_one_tile(M, N, K) && group > 0) {
    const int rc = try_panelm(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, workspace, workspace_bytes, stream);
    if (rc >= 0) return rc;
  }
  // 17 .. 512 activation rows: the streaming kernel (weights once per 128 rows, deep ring of direct loads)
  if ((algo == TLQ_ALGO_AUTO && g_w4a16_stream) || algo == TLQ_ALGO_STREAM) {
    const StreamPlan sp = (K > 0 && group > 0 && M < kMaxDim && N < kMaxDim && K < kMaxDim)
                              ? w4a16_stream_plan(M, N, K, group, cu_count_or_default())
                              : StreamPlan{false, 0, 0, 0, 0, 0};
    const bool args_ok = A && w_packed && C && aligned16(A) && aligned16(w_packed) && aligned16(C) &&
                         (in_dtype == TLQ_F16 || in_dtype == TLQ_BF16) &&
                         (out_dtype == TLQ_F16 || out_dtype == TLQ_BF16 || out_dtype == TLQ_F32) && (M * N) % 4 == 0 &&
                         ((uintptr_t)scales & 1) == 0 && ((uintptr_t)zeros & 1) == 0 && K > 0 && fits32(M, K * 2) && fits32(N, K / 2);
    const bool ws_ok = sp.ok && (sp.split == 1 || (workspace && aligned16(workspace) && workspace_bytes >= (int64_t)sp.split * M * N * 4));
    if (algo == TLQ_ALGO_AUTO && !g_w4a16_panel && group > 0 && panel256_beats_stream(M, N, K, group, sp)) {
      const int rc = try_panel256(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, TLQ_W_PLAIN, workspace,
                                  workspace_bytes, stream);
      if (rc >= 0) return rc;
    }
    // measured on the MLP shapes: 20 - 35 % ahead of the tile kernel up to 256 rows, level with it at 512 -- unless the
    // tile kernels cannot fill the machine there (M = 512 on 4096 weight rows: 128 tiles of 128 x 128; K = 11008: 89
    // against 137 us for the two passes, K = 4096: 34 against 43 us)
    // (rows of more than 8192 values that the tile kernel can cut into enough K slices stay with it: N = 5120, K = 13824:
    // 101 against 127 us)
    // When the partial sums of many short K slices (split x M x N x 4 bytes, written and read back) outweigh the packed
    // weights, the tile kernel, which cuts K as it likes, is ahead.  (Since a slice of the streaming kernel may run over
    // several windows of 16 groups its plan seldom cuts that short.)
    // (Only where the partial sums are tens of MB: on 4096 weight rows, or below, the streaming kernel stays ahead.)
    // And only where the tile kernel finds a K cut that fills the machine: rows of 11008 = 2 x 43 x 128 values can only be halved.
    // Up to three blocks of 128 activation rows the streaming kernel is level with or ahead of the tile kernel over K
    // slices on 18 of 20 (N, K) pairs (N = 10240, K = 8192, M = 384: 93 against 155 us; the other two are 4 % behind);
    // with four blocks only while its work-groups fit the machine at once (N = 8192, K = 4096, M = 512: 51 against 59 us;
    // N = 13824, K = 5120, 432 work-groups: 114 against 99 us).
    // Its weak spot: somewhat more work-groups than CUs (one work-group per CU: the second round runs half empty).  Where
    // K has no cut for the tile kernel either, the two passes, whose plain GEMM cuts K unevenly, are ahead then:
    // N = 4096, K = 11008 (86 steps: 288 work-groups at M = 384, 384 at M = 512): 69 against 82 us, 78 against 87 us.
    const int64_t stream_wgs = (int64_t)sp.m_blocks * sp.n_blocks * sp.split;
    const int64_t cus_now = cu_count_or_default();
    const bool thin_second_round = M > 256 && have && N % 8 == 0 && stream_wgs > cus_now && stream_wgs * 2 <= cus_now * 3 &&
                                   w4a16_mid_split(M, N, K, group) <= 1;
    // A K cut of the tile kernel into long slices -- 3072 values or more per work-group -- does not pay between 192 and 256 rows
    // either: N = 28672, K = 8192, M = 192: 154 against 122 us for the streaming kernel; N = 8192, K = 28672: 156 against 121 us.
    // With groups of 32 values, where neither the middle-M kernel nor long windows are to be had, it does (N = 8192, K = 28672,
    // bf16, M = 196 - 252: 139 - 147 against 153 - 156 us).
    const int64_t tile_split = group < 64 && M >= 192 && M <= 256 ? w4a16_mid_split(M, N, K, group) : 1;
    const bool long_tile_slices = tile_split > 1 && K / tile_split >= 3072 && w4a16_mid_fill(M, N, K, group) >= 0.85 &&
                                  workspace != nullptr && workspace_bytes >= tile_split * M * N * 4;
    // Groups of 32 values give the streaming kernel windows of four steps, each with a round trip to memory of its own:
    // from 320 rows on, the tile kernel over K slices is 2 - 11 % ahead wherever its cut fills the machine (N = 4096,
    // K = 14336, M = 384: 77 against 84 us; N = 5120, K = 13824: 89 against 97 us); where it cannot cut K (rows of 11008
    // values) the streaming kernel is far ahead (64 against 160 us) and stays.
    const bool short_windows = group < 64 && M > 256 && sp.ok && (int64_t)sp.slice_steps * 128 > 2 * 16 * group &&
                               w4a16_mid_split(M, N, K, group) > 1 && w4a16_mid_fill(M, N, K, group) >= 0.8;
    const bool stream_first = ((M <= 384 && !thin_second_round) || stream_wgs <= cus_now) && !long_tile_slices && !short_windows;
    const bool slices_too_short = group < 128 && (int64_t)sp.split * M * 4 >= K && (int64_t)sp.split * M * N * 4 > ((int64_t)40 << 20) &&
                                  w4a16_mid_fill(M, N, K, group) >= 0.66;
    // One full tile height of the tile kernel (97 .. 128 rows) on up to 2^23 weights: the tile kernel over K slices is ahead of the
    // streaming kernel (128 rows, seven (N, K) pairs, fp16 and bf16: 13.6 - 18.2 against 15.3 - 18.8 us; level at 96 rows and
    // at 4096 x 4096, a third behind from 160 rows on).
    const bool tile_band = algo == TLQ_ALGO_AUTO && M > 96 && M <= 128 && N * K <= ((int64_t)1 << 23) && w4a16_mid_split(M, N, K, group) > 1 &&
                           workspace != nullptr && workspace_bytes >= w4a16_mid_split(M, N, K, group) * M * N * 4;
    if (sp.ok && args_ok && ws_ok && !tile_band &&
        (algo == TLQ_ALGO_STREAM || (stream_first && !slices_too_short) || (!slices_too_short && !thin_second_round && !long_tile_slices && !short_windows && tile_fill(1, M, N, 128) < 0.65 && (K <= 8192 || w4a16_mid_split(M, N, K, group) <= 1))))
      return gemm_w4a16_stream(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, TLQ_W_PLAIN, sp, (float*)workspace,
                               (hipStream_t)stream);
    if (algo == TLQ_ALGO_STREAM) {
      set_error("tlq_gemm_w4a16_ws: the streaming kernel needs 17 <= M <= 512, K %% 128 == 0, a power-of-two group >= 32, N %% 4 == 0, "
                "16-byte aligned operands and a workspace of %lld bytes (M=%lld N=%lld K=%lld group=%lld, workspace %lld)",
                (long long)(sp.ok ? (int64_t)sp.split * M * N * 4 : 0), (long long)M, (long long)N, (long long)K, (long long)group,
                (long long)workspace_bytes);
      return 1;
    }
  }
  // Above 512 rows: the 256-row panel kernel (one launch, no dequantised matrix) where its work-groups fill the machine.
  // Measured against the choice without it (two passes, tile kernel over K slices) and against the 128-row panel kernel
  // on ten (N, K) pairs x eleven values of M from 576 to 8192, fp16 with a zero-point tensor and bf16 with a scalar one,
  // groups of 128: wherever its last round of work-groups fills more than half of the CUs it is level or ahead -- by 3 - 16 %
  // from 3072 rows on (4096 x 4096 x 4096 bf16: 104 against 113 - 119 us; 8192 x 8192 x 8192: 1.11 x), by 10 - 56 % between
  // 576 and 2048 rows on wide or long matrices (N = 28672, K = 4096, M = 768: 1.40 - 1.54 x; N = 4096, K = 14336, M = 1280:
  // 1.50 - 1.56 x), 0.98 - 0.99 on a few of the largest fp16 problems -- and 2 - 21 % behind below that fill (N = K = 4096,
  // M <= 1024: 96 work-groups).  The 128-row kernel is ahead of it nowhere by more than 4 % and stays an explicit choice.
  if (algo == TLQ_ALGO_AUTO && !g_w4a16_panel && M > 512 && K > 0 && group > 0 && N >= 1 && N < kMaxDim && K < kMaxDim && M < kMaxDim) {
    // The middle-M kernel's 128-row tiles first where an estimate of both kernels' times says so: rounds of work-groups x
    // (steps per K slice x the time of a step + a fixed part) + the pass over the slices' partial tiles, with the step
    // times measured at a full machine (2.2 us on 128 rows, 3.3 us on 256) and fixed parts of 6 / 8 us.  On ten (N, K)
    // pairs x M = 576 .. 3072, fp16 with a zero-point tensor and bf16 with a scalar one (144 cases where both kernels
    // apply), taking the 128-row kernel where its estimate is below 0.94 of the other's never lost against the choice
    // without it and gains 4 % on average: N = 11008, K = 4096, M = 576 - 640 (5 x 43 tiles fill the machine once, 3 x 43
    // half of it) 69 against 102 - 106 us; N = 8192, K = 2048, M <= 1024 35 - 43 against 50 - 54 us; N = K = 4096, M = 1024
    // 50 against 62 us; N = 2048, K = 8192, M <= 1024 42 - 51 against 47 - 59 us.
    if (panelm_estimate_wins(M, N, K, group)) {
      const int rc = try_panelm(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, workspace, workspace_bytes, stream);
      if (rc >= 0) return rc;
    }
    if (panel256_fills(M, N, K, group)) {
      const int rc = try_panel256(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, TLQ_W_PLAIN, workspace,
                                  workspace_bytes, stream);
      if (rc >= 0) return rc;
    }
  }
  const bool split_region = w4a16_mid_split(M, N, K, group > 0 ? group : 32) > 1;
  const bool two_pass = algo == TLQ_ALGO_TWO_PASS ||
                        (algo == TLQ_ALGO_AUTO && have && M >= kTwoPassMinM && N % 8 == 0 && !split_region);
  if (!two_pass && (algo == TLQ_ALGO_AUTO || algo == TLQ_ALGO_MFMA) && M > 16 && workspace && aligned16(workspace) &&
      K > 0 && K % 64 == 0 && group > 0 && K % group == 0 && group % 32 == 0 && A && w_packed && C && aligned16(A) &&
      aligned16(w_packed) && aligned16(C) && N % 4 == 0 && (M * N) % 4 == 0 && M < kMaxDim && N < kMaxDim && K < kMaxDim &&
      (in_dtype == TLQ_F16 || in_dtype == TLQ_BF16) && (out_dtype == TLQ_F16 || out_dtype == TLQ_BF16 || out_dtype == TLQ_F32) &&
      fits32(M, K * 2) && fits32(N, K / 2) && ((uintptr_t)scales & 1) == 0 && ((uintptr_t)zeros & 1) == 0) {
    // small and middle M: the tile kernel over K slices, partial sums in the workspace, one pass to add them up
    const int64_t split = w4a16_mid_split(M, N, K, group);
    if (split > 1 && workspace_bytes >= split * M * N * 4)
      return gemm_w4a16_mfma_splitk(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, split,
                                    (float*)workspace, (hipStream_t)stream);
  }
  if (!two_pass)
    return tlq_gemm_w4a16(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype,
                          algo == TLQ_ALGO_TWO_PASS ? TLQ_ALGO_AUTO : algo, stream);
  TLQ_CHECK_DIMS("tlq_gemm_w4a16_ws");
  TLQ_REQUIRE(in_dtype == TLQ_F16 || in_dtype == TLQ_BF16, "tlq_gemm_w4a16_ws: in_dtype must be float16 or bfloat16 (got %d)",
              in_dtype);
  TLQ_REQUIRE(out_dtype == TLQ_F16 || out_dtype == TLQ_BF16 || out_dtype == TLQ_F32,
              "tlq_gemm_w4a16_ws: out_dtype must be float16, bfloat16 or float32 (got %d)", out_dtype);
  if (M == 0 || N == 0) return 0;
  TLQ_REQUIRE(K > 0 && K % 64 == 0, "tlq_gemm_w4a16_ws: K=%lld must be a positive multiple of 64", (long long)K);
  TLQ_REQUIRE(group > 0 && K % group == 0 && group % 32 == 0,
              "tlq_gemm_w4a16_ws: group=%lld must divide K=%lld and be a multiple of 32", (long long)group, (long long)K);
  TLQ_REQUIRE(((uintptr_t)scales & 1) == 0 && ((uintptr_t)zeros & 1) == 0, "tlq_gemm_w4a16_ws: scales / zeros misaligned");
  if (int rc = tlq_dequant_w4(w_packed, scales, zeros, workspace, N, K, group, zero_scalar, in_dtype, stream)) return rc;
  return plain_gemm_on_workspace(A, workspace, workspace_bytes, C, M, N, K, in_dtype, out_dtype, stream);
}

int tlq_gemm_w4a16_layout_ws(const void* A, const void* w_packed, const void* scales, const void* zeros, void* C, int64_t M,
                             int64_t N, int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, int algo,
                             int w_layout, void* workspace, int64_t workspace_bytes, void* stream) {
  TLQ_REQUIRE(w_layout == TLQ_W_PLAIN || w_layout == TLQ_W_INTERLEAVED_F16, "tlq_gemm_w4a16_layout_ws: bad weight layout %d", w_layout);
  if (w_layout == TLQ_W_PLAIN)
    return tlq_gemm_w4a16_ws(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, algo, workspace,
                             workspace_bytes, stream);
  TLQ_CHECK_DIMS("tlq_gemm_w4a16_layout_ws");
  TLQ_REQUIRE(algo == TLQ_ALGO_AUTO || algo == TLQ_ALGO_GEMV || algo == TLQ_ALGO_STREAM || algo == TLQ_ALGO_TWO_PASS || algo == TLQ_ALGO_DECODE || algo == TLQ_ALGO_PANEL || algo == TLQ_ALGO_PANEL256,
              "tlq_gemm_w4a16_layout_ws: interleaved weights are read by the ring GEMV, the decode kernel, the streaming kernel, the panel kernels and the two passes (algo %d)", algo);
  TLQ_REQUIRE(in_dtype == TLQ_F16 || in_dtype == TLQ_BF16, "tlq_gemm_w4a16_layout_ws: in_dtype must be float16 or bfloat16 (got %d)", in_dtype);
  TLQ_REQUIRE(out_dtype == TLQ_F16 || out_dtype == TLQ_BF16 || out_dtype == TLQ_F32, "tlq_gemm_w4a16_layout_ws: bad out_dtype %d", out_dtype);
  if (M == 0 || N == 0) return 0;
  TLQ_REQUIRE(K > 0 && K % 64 == 0, "tlq_gemm_w4a16_layout_ws: K=%lld must be a positive multiple of 64", (long long)K);
  TLQ_REQUIRE(group > 0 && K % group == 0 && group % 32 == 0, "tlq_gemm_w4a16_layout_ws: group=%lld must divide K=%lld and be a multiple of 32",
              (long long)group, (long long)K);
  TLQ_REQUIRE(A && w_packed && C, "tlq_gemm_w4a16_layout_ws: null pointer");
  TLQ_REQUIRE(aligned16(A) && aligned16(w_packed) && aligned16(C), "tlq_gemm_w4a16_layout_ws: A, w_packed and C must be 16-byte aligned");
  TLQ_REQUIRE(((uintptr_t)scales & 1) == 0 && ((uintptr_t)zeros & 1) == 0, "tlq_gemm_w4a16_layout_ws: scales / zeros misaligned");
  TLQ_REQUIRE(fits32(M, K * 2) && fits32(N, K / 2), "tlq_gemm_w4a16_layout_ws: a matrix spans 4 GiB or more");
  if (algo != TLQ_ALGO_TWO_PASS) {  // one scale / zero point per row on rows that are no power of two: as for plain words
    RowValues rv;
    const int wrote = write_out_row_values(scales, zeros, M, N, K, group, in_dtype, workspace, workspace_bytes, stream, rv);
    if (wrote < 0) return 1;
    if (wrote > 0)
      return tlq_gemm_w4a16_layout_ws(A, w_packed, rv.scales, rv.zeros, C, M, N, K, rv.group, zero_scalar, in_dtype, out_dtype, algo, w_layout, workspace,
                                      rv.workspace_bytes, stream);
  }
  if (algo == TLQ_ALGO_AUTO) {  // ragged weight-row counts: as for plain words
    bool taken = false;
    const int rc = run_ragged_rows(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, w_layout, workspace, workspace_bytes, stream, taken);
    if (taken) return rc;
  }
  const bool ws_aligned = workspace && aligned16(workspace);
  // one or two activation rows: the ring GEMV where the plain layout takes it too (one row; two fp16 rows on 8192 weight
  // rows or more), or when asked for by name
  if (M <= 2 && (algo == TLQ_ALGO_GEMV || (algo == TLQ_ALGO_AUTO && (M == 1 || N >= 8192)))) {
    const int rc = gemv_w4a16_ring_interleaved(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype,
                                               (hipStream_t)stream);
    if (rc >= 0) return rc;
    TLQ_REQUIRE(algo != TLQ_ALGO_GEMV, "tlq_gemm_w4a16_layout_ws: the GEMV kernel reads interleaved weights for M <= 2 (fp16; bf16 M = 1), "
                "K <= 4096, a power-of-two group with (K / group) %% 8 == 0 and 16-byte aligned scale / zero tensors (M=%lld N=%lld K=%lld "
                "group=%lld)", (long long)M, (long long)N, (long long)K, (long long)group);
  }
  TLQ_REQUIRE(algo != TLQ_ALGO_GEMV, "tlq_gemm_w4a16_layout_ws: the GEMV kernel reads interleaved weights for M <= 2 only (got %lld)", (long long)M);
  if (M <= 32 && (algo == TLQ_ALGO_AUTO || algo == TLQ_ALGO_DECODE)) {
    const DecodePlan dp = w4a16_decode_plan(M, N, K, group, cu_count_or_default());
    const bool dec_ok = dp.ok && (((uintptr_t)scales | (uintptr_t)zeros) & 3) == 0 &&
                        (dp.chunks == 1 || ((M * N) % 4 == 0 && ws_aligned && workspace_bytes >= (int64_t)dp.chunks * M * N * 4));
    if (dec_ok)
      return gemm_w4a16_decode(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, w_layout, dp,
                               (float*)workspace, (hipStream_t)stream);
    TLQ_REQUIRE(algo != TLQ_ALGO_DECODE, "tlq_gemm_w4a16_layout_ws: the decode kernel does not take M=%lld N=%lld K=%lld group=%lld with a "
                "workspace of %lld bytes (K %% 256 == 0, a power-of-two group, dword-aligned scale / zero tensors)", (long long)M, (long long)N,
                (long long)K, (long long)group, (long long)workspace_bytes);
  }
  TLQ_REQUIRE(algo != TLQ_ALGO_DECODE, "tlq_gemm_w4a16_layout_ws: the decode kernel handles M <= 32 (got %lld)", (long long)M);
  if (algo == TLQ_ALGO_PANEL256 || (algo == TLQ_ALGO_AUTO && !g_w4a16_panel && M > 512)) {
    // (the same rule as for plain words: where the 256-row panel kernel's tiles fill the machine)
    if (algo == TLQ_ALGO_PANEL256 || panel256_fills(M, N, K, group)) {
      const int rc = try_panel256(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, w_layout, workspace,
                                  workspace_bytes, stream);
      if (rc >= 0) return rc;
    }
    TLQ_REQUIRE(algo != TLQ_ALGO_PANEL256, "tlq_gemm_w4a16_layout_ws: the 256-row panel kernel does not take M=%lld N=%lld K=%lld group=%lld "
                "with a workspace of %lld bytes (K %% 128 == 0, M %% 4 == 0, N %% 16 == 0, a power-of-two group >= 32)", (long long)M,
                (long long)N, (long long)K, (long long)group, (long long)workspace_bytes);
  }
  if (algo == TLQ_ALGO_PANEL) {
    const PanelPlan pp = w4a16_panel_plan(M, N, K, group, cu_count_or_default());
    if (pp.ok) {
      const int rc = try_panel(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, w_layout, workspace,
                               workspace_bytes, stream);
      if (rc >= 0) return rc;
    }
    TLQ_REQUIRE(false, "tlq_gemm_w4a16_layout_ws: the panel kernel does not take M=%lld N=%lld K=%lld group=%lld with a "
                "workspace of %lld bytes (K %% 128 == 0, M %% 4 == 0, N %% 16 == 0, a power-of-two group with (K / group) %% 8 == 0, 16-byte "
                "aligned scale / zero tensors)", (long long)M, (long long)N, (long long)K, (long long)group, (long long)workspace_bytes);
  }
  if (algo == TLQ_ALGO_AUTO && !g_w4a16_panel && panel_one_round(M, N, K)) {  // (65 .. 128 rows on output-layer widths, as for plain words)
    const int rc = try_panel(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, w_layout, workspace, workspace_bytes, stream);
    if (rc >= 0) return rc;
  }
  if (algo != TLQ_ALGO_TWO_PASS) {
    const StreamPlan sp = w4a16_stream_plan(M, N, K, group, cu_count_or_default());
    const bool ws_ok = sp.ok && (M * N) % 4 == 0 && (sp.split == 1 || (ws_aligned && workspace_bytes >= (int64_t)sp.split * M * N * 4));
    // (129 .. 512 rows: the 256-row kernel where its estimate beats the streaming kernel's, as for the plain layout)
    if (algo == TLQ_ALGO_AUTO && !g_w4a16_panel && group > 0 && panel256_beats_stream(M, N, K, group, sp)) {
      const int rc = try_panel256(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, w_layout, workspace,
                                  workspace_bytes, stream);
      if (rc >= 0) return rc;
    }
    if (ws_ok && (algo == TLQ_ALGO_STREAM || M <= 384 || (int64_t)sp.m_blocks * sp.n_blocks * sp.split <= cu_count_or_default() || tile_fill(1, M, N, 128) < 0.65 || !(ws_aligned && workspace_bytes >= N * K * 2)))  // (no tile kernel reads this layout: the alternative is the two passes)
      return gemm_w4a16_stream(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, w_layout, sp,
                               (float*)workspace, (hipStream_t)stream);
    TLQ_REQUIRE(algo != TLQ_ALGO_STREAM, "tlq_gemm_w4a16_layout_ws: the streaming kernel does not take M=%lld N=%lld K=%lld group=%lld "
                "with a workspace of %lld bytes", (long long)M, (long long)N, (long long)K, (long long)group, (long long)workspace_bytes);
  }
  TLQ_REQUIRE(M >= 17, "tlq_gemm_w4a16_layout_ws: with M=%lld interleaved weights need the decode kernel's shapes (K %% 256 == 0, power-of-two "
              "group, dword-aligned scale / zero tensors); other decode-sized problems read the plain layout", (long long)M);
  TLQ_REQUIRE(ws_aligned && workspace_bytes >= N * K * 2 && N % 8 == 0,
              "tlq_gemm_w4a16_layout_ws: M=%lld N=%lld K=%lld needs a 16-byte aligned workspace of %lld bytes (got %lld) and N %% 8 == 0",
              (long long)M, (long long)N, (long long)K, (long long)(N * K * 2), (long long)workspace_bytes);
  if (int rc = tlq_dequant_w4_layout(w_packed, scales, zeros, workspace, N, K, group, zero_scalar, in_dtype, w_layout, stream)) return rc;
  return plain_gemm_on_workspace(A, workspace, workspace_bytes, C, M, N, K, in_dtype, out_dtype, stream);
}

int tlq_gemv_w4a16_batched(const void* A, const void* w_packed, const void* scales, const void* zeros, void* C,
                           int64_t batch, int64_t M, int64_t N, int64_t K, int64_t group, float zero_scalar, int in_dtype,
                           int out_dtype, void* stream) {
  TLQ_CHECK_DIMS("tlq_gemv_w4a16_batched");
  TLQ_REQUIRE(batch >= 0 && batch <= 65535, "tlq_gemv_w4a16_batched: batch=%lld must be in 0..65535", (long long)batch);
  TLQ_REQUIRE(in_dtype == TLQ_F16 || in_dtype == TLQ_BF16, "tlq_gemv_w4a16_batched: bad in_dtype %d", in_dtype);
  TLQ_REQUIRE(out_dtype == TLQ_F16 || out_dtype == TLQ_BF16 || out_dtype == TLQ_F32, "tlq_gemv_w4a16_batched: bad out_dtype %d",
              out_dtype);
  if (batch == 0 || M == 0 || N == 0) return 0;
  TLQ_REQUIRE(M <= 16, "tlq_gemv_w4a16_batched: M=%lld must be <= 16", (long long)M);
  TLQ_REQUIRE(K > 0 && K % 64 == 0, "tlq_gemv_w4a16_batched: K=%lld must be a positive multiple of 64", (long long)K);
  TLQ_REQUIRE(group > 0 && K % group == 0 && group % 32 == 0,
              "tlq_gemv_w4a16_batched: group=%lld must divide K=%lld and be a multiple of 32", (long long)group, (long long)K);
  TLQ_REQUIRE(A && w_packed && C, "tlq_gemv_w4a16_batched: null pointer");
  TLQ_REQUIRE(aligned16(A) && aligned16(w_packed), "tlq_gemv_w4a16_batched: A and w_packed must be 16-byte aligned");
  return gemv_w4a16(A, w_packed, scales, zeros, C, batch, M, N, K, group, zero_scalar, in_dtype, out_dtype,
                    (hipStream_t)stream);
}

int tlq_gemm_f16_batched(const void* A, const void* B, void* C, int64_t batch, int64_t M, int64_t N, int64_t K, int in_dtype,
                         int out_dtype, int b_layout, void* stream) {
  TLQ_CHECK_DIMS("tlq_gemm_f16");
  TLQ_REQUIRE(batch >= 0 && batch < kMaxDim, "tlq_gemm_f16: bad batch %lld", (long long)batch);
  TLQ_REQUIRE(in_dtype == TLQ_F16 || in_dtype == TLQ_BF16, "tlq_gemm_f16: in_dtype must be float16 or bfloat16 (got %d)",
              in_dtype);
  TLQ_REQUIRE(out_dtype == TLQ_F16 || out_dtype == TLQ_BF16 || out_dtype == TLQ_F32, "tlq_gemm_f16: bad out_dtype %d",
              out_dtype);
  TLQ_REQUIRE(b_layout == TLQ_B_KN || b_layout == TLQ_B_NK, "tlq_gemm_f16: bad b_layout %d", b_layout);
  if (batch == 0 || M == 0 || N == 0) return 0;
  TLQ_REQUIRE(K > 0 && K % 8 == 0, "tlq_gemm_f16: K=%lld must be a positive multiple of 8", (long long)K);
  TLQ_REQUIRE(N % 8 == 0, "tlq_gemm_f16: N=%lld must be a multiple of 8", (long long)N);
  TLQ_REQUIRE(A && B && C, "tlq_gemm_f16: null pointer");
  TLQ_REQUIRE(aligned16(A) && aligned16(B) && aligned16(C), "tlq_gemm_f16: pointers must be 16-byte aligned");
  TLQ_REQUIRE(fits32(M, K * 2) && fits32(N, K * 2), "tlq_gemm_f16: a matrix spans 4 GiB or more");
  TLQ_REQUIRE(batch == 1 || (((M * K) % 8 == 0) && ((M * N) % 8 == 0)),
              "tlq_gemm_f16: every matrix of a batch must start on a 16-byte boundary (M*K and M*N multiples of 8)");
  return gemm_f16_plain(A, B, C, batch, M, N, K, in_dtype, out_dtype, b_layout, (hipStream_t)stream);
}

int tlq_gemm_f16(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int in_dtype, int out_dtype,
                 int b_layout, void* stream) {
  return tlq_gemm_f16_batched(A, B, C, 1, M, N, K, in_dtype, out_dtype, b_layout, stream);
}

int64_t tlq_f16_workspace_bytes(int64_t batch, int64_t M, int64_t N, int64_t K) {
  if (batch != 1 || M <= 0 || N <= 0 || K <= 0 || M >= kMaxDim || N >= kMaxDim || K >= kMaxDim || N % 8 != 0) return 0;
  const int split = f16_split_choice(batch, M, N, K);
  return split > 1 ? (int64_t)split * M * N * 4 : 0;
}

int tlq_gemm_f16_ws(const void* A, const void* B, void* C, void* workspace, int64_t workspace_bytes, int64_t batch, int64_t M,
                    int64_t N, int64_t K, int in_dtype, int out_dtype, int b_layout, void* stream) {
  // One batch, few activation rows: K slices write fp32 matrices into the workspace, a second pass adds them in slice
  // order and rounds once.  As many slices as the workspace holds; none, or a shape that is not cut: tlq_gemm_f16_batched.
  int split = 1;
  if (tlq_f16_workspace_bytes(batch, M, N, K) > 0 && workspace != nullptr && aligned16(workspace)) {
    split = f16_split_choice(batch, M, N, K);
    while (split > 1 && (int64_t)split * M * N * 4 > workspace_bytes) split /= 2;
  }
  if (split <= 1) return tlq_gemm_f16_batched(A, B, C, batch, M, N, K, in_dtype, out_dtype, b_layout, stream);
  TLQ_REQUIRE(in_dtype == TLQ_F16 || in_dtype == TLQ_BF16, "tlq_gemm_f16_ws: in_dtype must be float16 or bfloat16 (got %d)",
              in_dtype);
  TLQ_REQUIRE(out_dtype == TLQ_F16 || out_dtype == TLQ_BF16 || out_dtype == TLQ_F32, "tlq_gemm_f16_ws: bad out_dtype %d",
              out_dtype);
  TLQ_REQUIRE(b_layout == TLQ_B_KN || b_layout == TLQ_B_NK, "tlq_gemm_f16_ws: bad b_layout %d", b_layout);
  TLQ_REQUIRE(A && B && C, "tlq_gemm_f16_ws: null pointer");
  TLQ_REQUIRE(aligned16(A) && aligned16(B) && aligned16(C), "tlq_gemm_f16_ws: pointers must be 16-byte aligned");
  TLQ_REQUIRE(fits32(M, K * 2) && fits32(N, K * 2), "tlq_gemm_f16_ws: a matrix spans 4 GiB or more");
  return gemm_f16_slices(A, B, C, (float*)workspace, M, N, K, split, in_dtype, out_dtype, b_layout, (hipStream_t)stream);
}

void tlq_tune_f16_split(int slices) { g_f16_split = slices; }
int tlq_debug_f16_split(int64_t M, int64_t N, int64_t K) { return f16_split_choice(1, M, N, K); }

int tlq_gemm_f16_splitk(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t split_k,
                        int in_dtype, int b_layout, void* stream) {
  TLQ_CHECK_DIMS("tlq_gemm_f16_splitk");
  TLQ_REQUIRE(in_dtype == TLQ_F16 || in_dtype == TLQ_BF16,
              "tlq_gemm_f16_splitk: in_dtype must be float16 or bfloat16 (got %d)", in_dtype);
  TLQ_REQUIRE(b_layout == TLQ_B_KN || b_layout == TLQ_B_NK, "tlq_gemm_f16_splitk: bad b_layout %d", b_layout);
  TLQ_REQUIRE(split_k >= 1 && split_k <= 1024, "tlq_gemm_f16_splitk: split_k=%lld out of range 1..1024", (long long)split_k);
  if (M == 0 || N == 0) return 0;
  TLQ_REQUIRE(K > 0 && K % split_k == 0 && (K / split_k) % 8 == 0,
              "tlq_gemm_f16_splitk: K=%lld must split into %lld slices of a multiple of 8", (long long)K, (long long)split_k);
  TLQ_REQUIRE(N % 8 == 0, "tlq_gemm_f16_splitk: N=%lld must be a multiple of 8", (long long)N);
  TLQ_REQUIRE(A && B && C, "tlq_gemm_f16_splitk: null pointer");
  TLQ_REQUIRE(aligned16(A) && aligned16(B) && aligned16(C), "tlq_gemm_f16_splitk: pointers must be 16-byte aligned");
  TLQ_REQUIRE(fits32(M, K * 2) && fits32(N, K * 2), "tlq_gemm_f16_splitk: a matrix spans 4 GiB or more");
  return gemm_f16_splitk(A, B, (float*)C, M, N, K, split_k, in_dtype, b_layout, (hipStream_t)stream);
}

int tlq_gemm_i8(const void* A, const void* B, void* C, int64_t batch, int64_t M, int64_t N, int64_t K, int b_layout,
                void* stream) {
  TLQ_CHECK_DIMS("tlq_gemm_i8");
  TLQ_REQUIRE(batch >= 0 && batch < kMaxDim, "tlq_gemm_i8: bad batch %lld", (long long)batch);
  TLQ_REQUIRE(b_layout == TLQ_B_KN || b_layout == TLQ_B_NK, "tlq_gemm_i8: bad b_layout %d", b_layout);
  if (batch == 0 || M == 0 || N == 0) return 0;
  TLQ_REQUIRE(K > 0 && K % 16 == 0, "tlq_gemm_i8: K=%lld must be a positive multiple of 16", (long long)K);
  TLQ_REQUIRE(N % 16 == 0, "tlq_gemm_i8: N=%lld must be a multiple of 16", (long long)N);
  TLQ_REQUIRE(A && B && C, "tlq_gemm_i8: null pointer");
  TLQ_REQUIRE(aligned16(A) && aligned16(B) && aligned16(C), "tlq_gemm_i8: pointers must be 16-byte aligned");
  TLQ_REQUIRE(fits32(M, K) && fits32(N, K), "tlq_gemm_i8: a matrix spans 4 GiB or more");
  // few activation rows: K slices add into C itself (int32, exact in any order)
  if (const int split = i8_split_choice(batch, M, N, K, false); split > 1)
    return gemm_i8_i32_splitk(A, B, (int32_t*)C, M, N, K, split, b_layout, (hipStream_t)stream);
  return gemm_i8_i32(A, B, C, batch, M, N, K, b_layout, (hipStream_t)stream);
}

int tlq_gemm_w4a8(const void* A, const void* w_packed, void* C, int64_t M, int64_t N, int64_t K, int sign_mode,
                  void* stream) {
  TLQ_CHECK_DIMS("tlq_gemm_w4a8");
  TLQ_REQUIRE(sign_mode >= TLQ_U4 && sign_mode <= TLQ_S4_OFFSET7, "tlq_gemm_w4a8: bad sign_mode %d", sign_mode);
  if (M == 0 || N == 0) return 0;
  TLQ_REQUIRE(K > 0 && K % 32 == 0, "tlq_gemm_w4a8: K=%lld must be a positive multiple of 32", (long long)K);
  TLQ_REQUIRE(N % 4 == 0, "tlq_gemm_w4a8: N=%lld must be a multiple of 4", (long long)N);
  TLQ_REQUIRE(A && w_packed && C, "tlq_gemm_w4a8: null pointer");
  TLQ_REQUIRE(aligned16(A) && aligned16(w_packed) && aligned16(C), "tlq_gemm_w4a8: pointers must be 16-byte aligned");
  TLQ_REQUIRE(fits32(M, K) && fits32(N, K / 2), "tlq_gemm_w4a8: a matrix spans 4 GiB or more");
  // few activation rows: K slices add into C (int32, exact in any order)
  if (const int split = i8_split_choice(1, M, N, K, false, 2.5); split > 1)
    return gemm_w4a8_i32_splitk(A, w_packed, C, M, N, K, sign_mode, split, nullptr, (hipStream_t)stream);
  return gemm_w4a8_i32(A, w_packed, C, M, N, K, sign_mode, (hipStream_t)stream);
}

static thread_local int g_w4a8_ws_mode = 0;  // tlq_tune_w4a8_ws: 0 = automatic, 1 = K slices in the workspace, 2 = unpack + int8 GEMM

int tlq_gemm_w4a8_ws(const void* A, const void* w_packed, void* workspace, int64_t workspace_bytes, void* C, int64_t M,
                     int64_t N, int64_t K, int sign_mode, void* stream) {
  // The reference's int8 [N, K] workspace is used in one of two ways.  Many activation rows: the reference's own two
  // steps -- unpack into the workspace, int8 GEMM on it -- each at its own roofline (M = N = K = 4096: 6 + 66 us against
  // 98 us fused; M = 1024: 37 against 65 us).  Few rows (the unpack pass would cost more than the GEMM): the kernel that
  // unpacks on the way into LDS over K slices, the workspace holding one int32 [M, N] matrix per slice.
  const bool usable = workspace != nullptr && aligned16(workspace) && N > 0 && K > 0 && M > 0 && M < kMaxDim && N < kMaxDim &&
                      K < kMaxDim && fits32(N, K / 2) && fits32(M, K);
  if (usable && K % 32 == 0 && N % 4 == 0 && g_w4a8_ws_mode != 2 && (M <= 256 || g_w4a8_ws_mode == 1)) {
    int split = i8_split_choice(1, M, N, K, true, 2.5);
    while (split > 1 && (int64_t)split * M * N * 4 > workspace_bytes) split /= 2;
    if (split > 1) {
      TLQ_REQUIRE(sign_mode >= TLQ_U4 && sign_mode <= TLQ_S4_OFFSET7, "tlq_gemm_w4a8_ws: bad sign_mode %d", sign_mode);
      TLQ_REQUIRE(A && w_packed && C && aligned16(A) && aligned16(w_packed) && aligned16(C),
                  "tlq_gemm_w4a8_ws: null or misaligned pointer");
      return gemm_w4a8_i32_splitk(A, w_packed, C, M, N, K, sign_mode, split, (int32_t*)workspace, (hipStream_t)stream);
    }
  }
  const bool two_steps = usable && workspace_bytes >= N * K && K % 16 == 0 && N % 16 == 0 && fits32(N, K) &&
                         (M > 64 || g_w4a8_ws_mode == 2);
  if (!two_steps) return tlq_gemm_w4a8(A, w_packed, C, M, N, K, sign_mode, stream);
  TLQ_REQUIRE(sign_mode >= TLQ_U4 && sign_mode <= TLQ_S4_OFFSET7, "tlq_gemm_w4a8_ws: bad sign_mode %d", sign_mode);
  TLQ_REQUIRE(A && w_packed && C && aligned16(w_packed), "tlq_gemm_w4a8_ws: null or misaligned pointer");
  if (int rc = tlq_unpack_int4(w_packed, workspace, N, K, TLQ_I8, sign_mode, stream)) return rc;
  return tlq_gemm_i8(A, workspace, C, 1, M, N, K, TLQ_B_NK, stream);
}

void tlq_tune_w4a8_ws(int mode) { g_w4a8_ws_mode = mode; }

int tlq_gemm_w8a8(const void* A, const void* B, const void* scale_a, const void* scale_b, void* C, int64_t batch,
                  int64_t M, int64_t N, int64_t K, int64_t n_scale_b, int b_layout, int out_dtype, void* stream) {
  TLQ_CHECK_DIMS("tlq_gemm_w8a8");
  TLQ_REQUIRE(batch >= 0 && batch < kMaxDim, "tlq_gemm_w8a8: bad batch %lld", (long long)batch);
  TLQ_REQUIRE(b_layout == TLQ_B_KN || b_layout == TLQ_B_NK, "tlq_gemm_w8a8: bad b_layout %d", b_layout);
  TLQ_REQUIRE(out_dtype == TLQ_F16 || out_dtype == TLQ_BF16 || out_dtype == TLQ_F32, "tlq_gemm_w8a8: bad out_dtype %d",
              out_dtype);
  if (batch == 0 || M == 0 || N == 0) return 0;
  TLQ_REQUIRE(K > 0 && K % 16 == 0, "tlq_gemm_w8a8: K=%lld must be a positive multiple of 16", (long long)K);
  TLQ_REQUIRE(N % 16 == 0, "tlq_gemm_w8a8: N=%lld must be a multiple of 16", (long long)N);
  TLQ_REQUIRE(scale_b == nullptr || n_scale_b == 1 || n_scale_b == N,
              "tlq_gemm_w8a8: n_scale_b=%lld must be 1 or N=%lld", (long long)n_scale_b, (long long)N);
  TLQ_REQUIRE(A && B && C, "tlq_gemm_w8a8: null pointer");
  TLQ_REQUIRE(aligned16(A) && aligned16(B) && aligned16(C), "tlq_gemm_w8a8: pointers must be 16-byte aligned");
  TLQ_REQUIRE(((uintptr_t)scale_a & 3) == 0 && ((uintptr_t)scale_b & 3) == 0, "tlq_gemm_w8a8: scales misaligned");
  TLQ_REQUIRE(fits32(M, K) && fits32(N, K), "tlq_gemm_w8a8: a matrix spans 4 GiB or more");
  return gemm_w8a8_rescale(A, B, scale_a, scale_b, C, batch, M, N, K, n_scale_b, b_layout, out_dtype,
                           (hipStream_t)stream);
}

static bool w8a8_dims_split(int64_t batch, int64_t M, int64_t N, int64_t K) {
  return batch == 1 && M > 0 && N > 0 && K > 0 && M < kMaxDim && N < kMaxDim && K < kMaxDim && K % 16 == 0 && N % 16 == 0 &&
         fits32(M, K) && fits32(N, K);
}

int64_t tlq_w8a8_workspace_bytes(int64_t batch, int64_t M, int64_t N, int64_t K) {
  if (!w8a8_dims_split(batch, M, N, K)) return 0;
  const int split = i8_split_choice(batch, M, N, K, true);
  return split > 1 ? (int64_t)split * M * N * 4 : 0;
}

int tlq_gemm_w8a8_ws(const void* A, const void* B, const void* scale_a, const void* scale_b, void* C, void* workspace,
                     int64_t workspace_bytes, int64_t batch, int64_t M, int64_t N, int64_t K, int64_t n_scale_b,
                     int b_layout, int out_dtype, void* stream) {
  // One batch, few activation rows: K slices write their int32 tiles into the workspace, a second pass sums and
  // rescales them into C (the reference's own two steps, example_quant_batch_matmul.py:42,66-68, with a matrix per slice).
  int split = 1;
  if (w8a8_dims_split(batch, M, N, K) && workspace != nullptr && aligned16(workspace)) {
    split = i8_split_choice(batch, M, N, K, true);
    while (split > 1 && (int64_t)split * M * N * 4 > workspace_bytes) split /= 2;  // as many slices as the workspace holds
  }
  if (split <= 1)
    return tlq_gemm_w8a8(A, B, scale_a, scale_b, C, batch, M, N, K, n_scale_b, b_layout, out_dtype, stream);
  TLQ_REQUIRE(b_layout == TLQ_B_KN || b_layout == TLQ_B_NK, "tlq_gemm_w8a8_ws: bad b_layout %d", b_layout);
  TLQ_REQUIRE(out_dtype == TLQ_F16 || out_dtype == TLQ_BF16 || out_dtype == TLQ_F32, "tlq_gemm_w8a8_ws: bad out_dtype %d",
              out_dtype);
  TLQ_REQUIRE(scale_b == nullptr || n_scale_b == 1 || n_scale_b == N,
              "tlq_gemm_w8a8_ws: n_scale_b=%lld must be 1 or N=%lld", (long long)n_scale_b, (long long)N);
  TLQ_REQUIRE(A && B && C, "tlq_gemm_w8a8_ws: null pointer");
  TLQ_REQUIRE(aligned16(A) && aligned16(B) && aligned16(C), "tlq_gemm_w8a8_ws: pointers must be 16-byte aligned");
  TLQ_REQUIRE(((uintptr_t)scale_a & 3) == 0 && ((uintptr_t)scale_b & 3) == 0, "tlq_gemm_w8a8_ws: scales misaligned");
  return gemm_w8a8_rescale_splitk(A, B, scale_a, scale_b, C, (int32_t*)workspace, M, N, K, n_scale_b, split, b_layout,
                                  out_dtype, (hipStream_t)stream);
}

}  // extern "C"
