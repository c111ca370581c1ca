/*
 * tlq.h -- C ABI of libtlq.so: MI355X (gfx950) quantized-matmul kernels.
 *
 * Drop-in boundary for the quantized-matmul hot path of tile-ai/tilelang-ascend.  The
 * reference compiles one shared object per kernel exposing
 *     extern "C" void call(uint8_t* p0, ..., uint8_t* pn, [int64_t dyn...], aclrtStream stream)
 * (emitter: src/target/codegen_ascend.cc:1061-1112; ctypes caller:
 * tilelang/jit/adapter/cython/cython_wrapper.pyx:189-197).  The entry points below keep
 * that ordering rule -- raw device pointers first, then sizes, then option codes, the
 * stream last -- with one named symbol per operator instead of one anonymous `call` per
 * specialisation.
 *
 * Conventions
 *   * all pointers are DEVICE pointers owned by the caller; the library borrows them for
 *     the duration of the (asynchronous) launch and never allocates or frees memory;
 *   * `stream` is a hipStream_t passed as void* (NULL = the legacy default stream);
 *   * return value 0 = launched; non-zero = rejected before launch, with the reason
 *     available from tlq_last_error() (thread local).  This is the
 *     `int init()/const char* get_last_error()` protocol the reference declares in
 *     tilelang/jit/adapter/wrapper.py:30-50 but leaves unwired for its NPU backend
 *     (tilelang/jit/adapter/cython/adapter.py:269-275);
 *   * packed int4 weights are uint8 [N, K/2]: element k of row n is nibble (k % 2) of byte
 *     k / 2, low nibble first (examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:27-29,
 *     tilelang/quantize/utils.py:64-67);
 *   * per-group scales / zeros are [N, K/group] in the activation dtype.
 */
#ifndef TLQ_H_
#define TLQ_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TLQ_ABI_VERSION 1

/* element type codes */
enum {
  TLQ_F16 = 0,
  TLQ_BF16 = 1,
  TLQ_F32 = 2,
  TLQ_I8 = 3,
  TLQ_I32 = 4
};

/* int4 sign conventions (how a nibble u in 0..15 becomes an integer) */
enum {
  TLQ_U4 = 0,        /* u            tilelang/quantize/quantization.py:198-206; fine_grained.py:10-57 */
  TLQ_S4_TWOS = 1,   /* u>=8 ? u-16 : u   quantization.py:221-231; example_dequant_gemm_w4a8.py:124-145 */
  TLQ_S4_OFFSET8 = 2,/* u - 8        quantization.py:186-195; lop3.py:14 (isSigned) */
  TLQ_S4_OFFSET7 = 3 /* u - 7        quantization.py:56-65 */
};

/* layout of the second GEMM operand */
enum {
  TLQ_B_KN = 0, /* B[K, N] row-major (example_quant_batch_matmul.py:39, fine_grained.py:85) */
  TLQ_B_NK = 1  /* B[N, K] row-major, i.e. transpose_B (examples/deepseek_v4/int8_gemm.py:58,77) */
};

/* arrangement of the eight 4-bit fields inside each 32-bit word of packed weights */
enum {
  TLQ_W_PLAIN = 0,           /* field k = element k: general_compress (tilelang/quantize/utils.py:53-69) */
  TLQ_W_INTERLEAVED_F16 = 1  /* fields hold elements 0, 2, 4, 6, 1, 3, 5, 7: interleave_weight for the fp16 target
                              * (utils.py:73-101), the layout the reference's fast decoders read (lop3.py:17-24) */
};

/* kernel selection for tlq_gemm_w4a16 */
enum {
  TLQ_ALGO_AUTO = 0,
  TLQ_ALGO_GEMV = 1, /* split-K wavefront GEMV (M <= 16) */
  TLQ_ALGO_MFMA = 2, /* LDS-staged MFMA dequant-GEMM */
  TLQ_ALGO_SKINNY = 3, /* M <= 64: weights stream from HBM through the dequantiser into MFMA operands, no LDS tile */
  TLQ_ALGO_TWO_PASS = 4, /* tlq_gemm_w4a16_ws only: dequantise into the workspace, then the plain GEMM */
  TLQ_ALGO_STREAM = 5, /* tlq_gemm_w4a16_ws only: 17 <= M <= 512, weights streamed once per 128 activation rows through a deep
                       * ring of direct loads, dequantised in registers; K slices add up through the workspace */
  TLQ_ALGO_DECODE = 6, /* 1 <= M <= 32, K % 256 == 0, power-of-two group: persistent work-groups, activations resident in registers, every
                       * weight read once through deep wavefront-private rings (rows longer than 4096 values need the workspace) */
  TLQ_ALGO_PANEL = 7 /* tlq_gemm_w4a16_ws / tlq_gemm_w4a16_layout_ws only: large M in one launch, 128 activation rows x 512 weight rows
                      * per work-group, packed weights copied global -> LDS as they are and dequantised on the MFMA operand read;
                      * K % 128 == 0, M % 4 == 0, N % 16 == 0, power-of-two group >= 32, (K / group) % 8 == 0, 16-byte aligned scale /
                      * zero tensors.  Workspace: the fp32 partial tiles where K is cut into slices, plus 16 bytes with a zero-point
                      * tensor (a flag word: a second launch redoes the product with the unfolded dequantiser when a zero point
                      * turns out not to be a small integer) */
  ,
  TLQ_ALGO_PANEL256 = 8 /* the same with 256 activation rows x 256 weight rows per work-group on four wavefronts that each own a
                         * full register file: per MFMA half the dequantiser arithmetic and half the LDS operand traffic; scales
                         * and zero points are gathered into registers, so any number of groups per row and 2-byte aligned
                         * scale / zero tensors will do; a zero-point tensor is handled inside the one launch (folded while the
                         * zero points are small integers, unfolded from the first step whose are not).  K % 128 == 0, M % 4 == 0,
                         * N % 16 == 0, power-of-two group >= 32.  Workspace: the fp32 partial tiles where K is cut into slices */
  ,
  TLQ_ALGO_PANELM = 9 /* middle M (tens to hundreds of activation rows): the four-wavefront panel structure on 64 or 128
                       * activation rows x 256 weight rows per work-group, a ring of four / three LDS slots, scales and zero
                       * points through LDS windows; a zero-point tensor is handled inside the one launch (folded while the
                       * zero points are small integers, unfolded from the first window that is not).  K % 128 == 0, M % 4 == 0,
                       * N % 16 == 0, power-of-two group >= 64 with (K / group) % 8 == 0, 16-byte aligned scale / zero tensors;
                       * plain word layout.  Workspace: the fp32 partial tiles where K is cut into slices */
};

int tlq_abi_version(void);
const char* tlq_last_error(void);

/* Number of compute units of the current device (0 on failure). */
int tlq_device_cu_count(void);

/* Nibble unpack, replaces torch_unpack_uint4_to_fp16 / torch_unpack_uint4_to_int8
 * (example_dequant_gemm_fine_grained.py:10-57), torch_convert (example_dequant_gemm_w4a8.py:124-145)
 * and the vector-core unpack of w4a8_gemm_cv (:69-106).
 * out[n, k] = convert(sign_mode, nibble) as out_dtype (TLQ_F16 / TLQ_BF16 / TLQ_I8).  K even. */
int tlq_unpack_int4(const void* w_packed, void* out, int64_t N, int64_t K, int out_dtype, int sign_mode, void* stream);

/* Per-group dequantisation W[n,k] = rn_T( rn_T(T(u) - T(z)) * s ), T = dtype (TLQ_F16 / TLQ_BF16):
 * the "original" zeros mode of tilelang/quantize/lop3.py:135-175 and gen_quant4's
 * ref = (q - 8).half() * s (tilelang/quantize/utils.py:33).
 * scales: [N, K/group] or NULL (=1).  zeros: [N, K/group] or NULL (then zero_scalar is used).
 * group must divide K and be even. */
int tlq_dequant_w4(const void* w_packed, const void* scales, const void* zeros, void* out, int64_t N, int64_t K,
                   int64_t group, float zero_scalar, int dtype, void* stream);

/* tlq_dequant_w4 for either arrangement of the packed words (w_layout: TLQ_W_PLAIN | TLQ_W_INTERLEAVED_F16).  Interleaved
 * words need K % 8 == 0 and group % 8 == 0. */
int tlq_dequant_w4_layout(const void* w_packed, const void* scales, const void* zeros, void* out, int64_t N, int64_t K,
                          int64_t group, float zero_scalar, int dtype, int w_layout, void* stream);

/* Fast decode of INTERLEAVED 4-bit weights, the gfx950 counterpart of the CUDA decoders that
 * get_lop3_intrin_group returns (tilelang/quantize/lop3.py:5-421, 998-1046, 1090-1202).  `words` are
 * 32-bit words whose nibbles were permuted by interleave_weight (tilelang/quantize/utils.py:73-126)
 * for the fp16 target (out_dtype TLQ_F16: 8 fp16 per word) or the int8 target (TLQ_I8: 16 int8 per
 * word pair).  is_signed subtracts 8 (fp16) / 7 (int8), as the reference's decoders do.
 * scales (fp16, one per `words_per_group` words) or NULL; zeros_mode 0 none | 1 original (u - z) * s |
 * 2 rescale fma(u, s, -|z|) | 3 quantized (u - qz) * s with zeros an int16 array; zeros fp16 otherwise.
 * The device functions themselves are in tilelang_ascend_amd/csrc/decode_i4.h. */
int tlq_decode_i4_interleaved(const void* words, const void* scales, const void* zeros, void* out, int64_t n_words,
                              int64_t words_per_group, int out_dtype, int is_signed, int zeros_mode, void* stream);

/* The "_offset" decoders of the same family (tilelang/quantize/lop3.py:82-131, 177-230, 272-322, 364-421; chosen by
 * get_lop3_intrin_group for storage_scope "warp" with scaling, :1178-1180): the eight weights of a word belong to two
 * groups.  Word i has group g = i / words_per_group; outputs 0..3 use scales[g] / zeros[g], outputs 4..7 use
 * scales[g + offset] / zeros[g + offset].  fp16 output only.  zeros_mode as above, except 3 (quantized): zeros are
 * 32-bit words of eight 4-bit zero points, the first half takes field group_offset of zeros[g], the second field
 * group_offset of zeros[g + zero_offset].  n_scales / n_zeros are the lengths of the two arrays (elements / words);
 * every index is checked against them before the launch. */
int tlq_decode_i4_interleaved_offset(const void* words, const void* scales, const void* zeros, void* out, int64_t n_words,
                                     int64_t words_per_group, int64_t n_scales, int64_t n_zeros, int offset, int zero_offset,
                                     int group_offset, int is_signed, int zeros_mode, void* stream);

/* The fast decoders for interleaved 2-bit and 1-bit weights (tilelang/quantize/lop3.py:423-890 fp16 targets, :892-996 int8
 * targets, :1048-1087 2-bit -> packed 4-bit; the device functions are in csrc/decode_lowbit.h under the reference's names).
 * A unit is what one call of a decoder handles: out_bits 16 (fp16): 8 outputs from 16 (source_bit 2) or 8 (source_bit 1)
 * source bits, out = f0 f4 f1 f5 f2 f6 f3 f7 of the source's fields f_j; out_bits 8 (int8): 16 outputs from 32 or 16 source
 * bits; out_bits 4 (source_bit 2 only): 16 nibbles in two 32-bit words from 32 source bits.  src holds n_units source
 * units back to back, out n_units x 16 bytes (8 bytes for out_bits 4).  scales / zeros (fp16 targets only): fp16, one per
 * units_per_group consecutive units; zeros_mode 0 none | 1 original rn(rn(u - z) s) | 2 rescale (2-bit: rn(rn(u s) - z),
 * 1-bit: fma(u, s, -|z|)) | 3 quantized (2-bit only; zeros are 16-bit integers) -- zeros with unsigned sources only.
 * is_signed: 2-bit u - 2, 1-bit 2 u - 1 (the 2-bit -> 4-bit form ignores it, as the reference's does). */
int tlq_decode_lowbit_interleaved(const void* src, const void* scales, const void* zeros, void* out, int64_t n_units,
                                  int64_t units_per_group, int source_bit, int out_bits, int is_signed, int zeros_mode,
                                  void* stream);

/* Fused weight-only GEMM / GEMV, replaces dequant_gemm_fp16_wrapper + fp16_gemm
 * (example_dequant_gemm_fine_grained.py:60-115,176-223) extended with per-group scale / zero:
 *   C[M,N] = rn_out( sum_k f32(A[m,k]) * f32(W[n,k]) ),  W as in tlq_dequant_w4, fp32 accumulate.
 * A: [M,K] in_dtype (TLQ_F16 / TLQ_BF16); C: [M,N] out_dtype (TLQ_F16 / TLQ_BF16 / TLQ_F32).
 * Requires K % 64 == 0 and group % 32 == 0 (group divides K).  The MFMA kernel additionally needs
 * N % 4 == 0 and a power-of-two group (32, 64, 128, ...); the GEMV kernel (M <= 16) takes any such group;
 * the skinny kernel (M <= 64) needs K % 128 == 0.  TLQ_ALGO_AUTO: M = 1 GEMV (fp16; bf16 up to K = 8192; fp16 also M = 2 with
 * K <= 4096), otherwise the decode kernel (TLQ_ALGO_DECODE) where M <= 32, K % 256 == 0, K <= 4096, the group is a power of two and the
 * scale / zero tensors are dword aligned, else M <= 64 skinny where its conditions hold (else GEMV up to M = 4), else -- more than
 * 64 rows -- what tlq_gemm_w4a16_ws takes when it is given no workspace: the streaming and panel kernels where they do not cut K, else MFMA. */
int tlq_gemm_w4a16(const void* A, const void* w_packed, const void* scales, const void* zeros, void* C, int64_t M,
                   int64_t N, int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, int algo,
                   void* stream);

/* The same operator with a caller-owned workspace of tlq_w4a16_workspace_bytes(M, N, K) bytes (0 when a
 * workspace would not be used).  With it, 16 < M <= 384 runs the streaming kernel (TLQ_ALGO_STREAM; K % 128 == 0,
 * power-of-two group, N % 4 == 0; up to M = 512 while its work-groups fit the machine at once) or, where that does not
 * apply and up to M = 2048 while there are few output tiles, the tile kernel, both over slices of K whose fp32 partial sums
 * live in the workspace and are added in slice order, and larger problems take two passes -- tlq_dequant_w4 into the
 * workspace, then the plain GEMM on it (itself over K slices, kept behind the dequantised matrix, where it has few output
 * tiles) -- which is the structure of the reference's own wrapper (example_dequant_gemm_fine_grained.py:176-223 unpacks,
 * then calls fp16_gemm) and is faster than converting the weights again in every row block of the fused kernel.  The
 * workspace holds nothing between calls.
 * algo: as tlq_gemm_w4a16, or TLQ_ALGO_TWO_PASS to force the two passes (workspace required).
 * With TLQ_ALGO_AUTO and more than 512 rows, a row count that is no multiple of four runs as two calls on the stream: the
 * multiple of four below (the large-M kernels take such counts only), then the last one to three rows.
 * One scale / zero point per weight row (group == K) on rows whose length is no power of two: the kernels over K slices take
 * power-of-two groups, so the per-row values are first written out per group of min(K & -K, 1024) values into the last
 * 2 * align16(N * K / group * 2) + 16 bytes of the workspace (tlq_w4a16_workspace_bytes counts them) and the call runs with
 * that group: bit for bit what a caller gets who replicates the values.  A smaller workspace: the call runs with group == K.
 * A weight-row count N that is no multiple of four (vocabularies of 50257 or 32001 rows) with more than 32 activation rows, or a
 * multiple of four that is no multiple of eight with more than 512 (while the packed result stays below 1 GiB): the
 * first N - N % 16 weight rows run through the usual choice into a packed [M, N - N % 16] result kept in the last
 * align16(M * (N - N % 16) * sizeof(out)) bytes of the workspace, one launch copies it into C and one more computes the last
 * weight rows straight into C (tlq_w4a16_workspace_bytes counts that room, sized for fp32 outputs).  Without it such a count
 * is taken up to 64 rows (skinny kernel) and refused above, as by tlq_gemm_w4a16. */
int64_t tlq_w4a16_workspace_bytes(int64_t M, int64_t N, int64_t K);
/* The least workspace with which tlq_gemm_w4a16_ws still takes a workspace-based kernel for this shape (the partial sums
 * of the K-slice kernels where they apply, else the dequantised matrix of the two passes); for callers short of memory. */
int64_t tlq_w4a16_workspace_bytes_min(int64_t M, int64_t N, int64_t K);
/* What the explicitly named family `algo` may ask of the workspace for this shape (any group size); 0 for the families that
 * use none.  TLQ_ALGO_AUTO: tlq_w4a16_workspace_bytes. */
int64_t tlq_w4a16_workspace_bytes_for(int64_t M, int64_t N, int64_t K, int algo);
int tlq_gemm_w4a16_ws(const void* A, const void* w_packed, const void* scales, const void* zeros, void* C, int64_t M,
                      int64_t N, int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, int algo,
                      void* workspace, int64_t workspace_bytes, void* stream);

/* tlq_gemm_w4a16_ws for weights whose words were repacked by interleave_weight (w_layout TLQ_W_INTERLEAVED_F16, e.g. by
 * tlq_pack_int4(interleave = 1)); TLQ_W_PLAIN is tlq_gemm_w4a16_ws itself.  Consumers of the repacked layout: the ring GEMV
 * (one activation row, or two fp16 rows; K <= 4096, (K / group) % 8 == 0; TLQ_ALGO_GEMV or the automatic choice), the
 * decode kernel (M <= 32, K % 256 == 0), the streaming kernel (17 <= M <= 512; the fp16 decode saves the four byte permutes
 * per word that only undo the plain layout), the panel kernels and the two passes (M >= 256 with a workspace of N * K
 * 16-bit values).  Other shapes are rejected.  Results are bit-identical to the plain layout on the same logical weights,
 * except for the GEMV, whose dot products pair neighbouring elements instead of elements four apart: there the two
 * layouts agree to the rounding of the fp32 sums (and bit for bit on one-hot activations).  One scale / zero point per row on
 * rows whose length is no power of two is written out per group into the workspace's tail as in tlq_gemm_w4a16_ws, and ragged
 * weight-row counts run as the multiple of 16 below plus the last rows in the same way. */
int tlq_gemm_w4a16_layout_ws(const void* A, const void* w_packed, const void* scales, const void* zeros, void* C, int64_t M,
                             int64_t N, int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, int algo,
                             int w_layout, void* workspace, int64_t workspace_bytes, void* stream);

/* Tuned kernel choice.  The reference searches its configurations per call signature and keeps the winner, in memory and
 * on disk (tilelang/autotuner/tuner.py:102-760 AutoTuner.run, tilelang/cache/tuner_cache.py).  The kernels here are pre-built,
 * so what a search finds is WHICH family runs: a process-wide table (M, N, K, group, in_dtype) -> TLQ_ALGO_* that
 * tlq_gemm_w4a16, tlq_gemm_w4a16_ws (and through it tlq_gemm_w4a16_noalloc and tlq_gemm_w4a16_layout_ws with TLQ_W_PLAIN)
 * consult before their own rules when called with TLQ_ALGO_AUTO.  A chosen family that refuses the call -- its shape rules,
 * the alignment of an operand, a workspace smaller than tlq_w4a16_workspace_bytes_for asks -- launches nothing and the
 * call proceeds by the rules, without an error.  tlq_w4a16_workspace_bytes covers the choices present for (M, N, K).
 * choice_set with TLQ_ALGO_AUTO removes an entry.  choice_save / choice_load: one entry per text line,
 * "M N K group in_dtype algo" in the codes of this header, '#' comments; load adds to (and overrides) what the table holds
 * and changes nothing when a line is malformed.  All six are thread safe; a choice made on one GPU model is not meant for
 * another (keep one file per device).  tilelang_ascend_amd.autotuner.tune_w4a16_choice fills the table by measurement. */
int tlq_w4a16_choice_set(int64_t M, int64_t N, int64_t K, int64_t group, int in_dtype, int algo);
int tlq_w4a16_choice_get(int64_t M, int64_t N, int64_t K, int64_t group, int in_dtype);
void tlq_w4a16_choice_clear(void);
int64_t tlq_w4a16_choice_count(void);
int tlq_w4a16_choice_save(const char* path);
int tlq_w4a16_choice_load(const char* path);

/* The same operator for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference, whose wrapper allocates its
 * workspace anew on every call (tilelang/jit/adapter/cython/cython_wrapper.pyx:128-129).  The workspace is
 * a device array built into the library, TLQ_NOALLOC_SCRATCH_BYTES per GPU, held until the process ends.  The
 * call allocates and frees nothing; results are those of tlq_gemm_w4a16_ws with a workspace of
 * TLQ_NOALLOC_SCRATCH_BYTES bytes (the preferred kernel where tlq_w4a16_workspace_bytes(M, N, K) fits), bit for bit;
 * problems whose tlq_w4a16_workspace_bytes_min(M, N, K) exceeds the array run as tlq_gemm_w4a16_ws runs them without a
 * workspace (the kernels that need no scratch), never with an error for lack of room.  All
 * calls on one GPU share the array: calls that overlap there (other streams, other threads) race.
 * tlq_gemm_w4a16_noalloc_init looks the array's address up for the current device (otherwise the first call on a
 * device does it); it allocates nothing either. */
#define TLQ_NOALLOC_SCRATCH_BYTES (64 << 20)
int tlq_gemm_w4a16_noalloc_init(void);
int tlq_gemm_w4a16_noalloc(const void* A, const void* w_packed, const void* scales, const void* zeros, void* C, int64_t M,
                           int64_t N, int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, int algo,
                           void* stream);

/* `batch` independent decode GEMVs in one launch (one grid row per problem): A [batch,M,K],
 * w_packed [batch,N,K/2], scales / zeros [batch,N,K/group], C [batch,M,N], all contiguous.
 * Same arithmetic as tlq_gemm_w4a16 with TLQ_ALGO_GEMV; M <= 16.  This is the shape of a decode
 * step that applies many weight-only-quantized projections (layers, experts) of one size; the
 * reference has no batched form of its GEMV (examples/gemv/example_gemv_c.py:27-46 is one
 * vector x one matrix), its batched operators are examples/batch_gemm/batch_gemm.py:28-60 and
 * quant_batch_matmul. */
int tlq_gemv_w4a16_batched(const void* A, const void* w_packed, const void* scales, const void* zeros, void* C,
                           int64_t batch, int64_t M, int64_t N, int64_t K, int64_t group, float zero_scalar, int in_dtype,
                           int out_dtype, void* stream);

/* Plain fp16 / bf16 GEMM with fp32 accumulate, replaces fp16_gemm
 * (example_dequant_gemm_fine_grained.py:60-115): C[M,N] = A[M,K] . B, B laid out per b_layout. */
int tlq_gemm_f16(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int in_dtype, int out_dtype,
                 int b_layout, void* stream);

/* Batched form, replaces batch_matmul (examples/batch_gemm/batch_gemm.py:28-60): C[b] = A[b] . B[b] for b < batch,
 * A [batch, M, K], B [batch, K, N] (or [batch, N, K] per b_layout), C [batch, M, N], dense.  One launch covers the
 * batch (the reference flattens batch x row tiles x column tiles into one grid the same way, :38-43). */
int tlq_gemm_f16_batched(const void* A, const void* B, void* C, int64_t batch, int64_t M, int64_t N, int64_t K, int in_dtype,
                         int out_dtype, int b_layout, void* stream);

/* tlq_gemm_f16_batched with a workspace for one batch with few activation rows (too few output tiles to fill the machine):
 * K is cut into slices of whole 128-byte stages that write fp32 [M,N] matrices into the workspace, and a second pass adds
 * them in slice order and rounds once (deterministic).  tlq_f16_workspace_bytes gives the size for the preferred number
 * of slices (0: this shape is not cut); a smaller workspace (16-byte aligned) means fewer slices, none means
 * tlq_gemm_f16_batched.  No counterpart in the reference: its fp16_gemm (example_dequant_gemm_fine_grained.py:60-115)
 * has one kernel for every M. */
int64_t tlq_f16_workspace_bytes(int64_t batch, int64_t M, int64_t N, int64_t K);
int tlq_gemm_f16_ws(const void* A, const void* B, void* C, void* workspace, int64_t workspace_bytes, int64_t batch, int64_t M,
                    int64_t N, int64_t K, int in_dtype, int out_dtype, int b_layout, void* stream);

/* Split-K form of the same GEMM, replaces gemm_splitk (examples/gemm_splitk/example_tilelang_gemm_splitk.py:16-48):
 * C (fp32 [M,N], accumulated IN PLACE, the caller zeroes it as the example does) += A[M,K] . B.  K is cut into
 * split_k slices handled by different work-groups that add their partial tiles with atomic adds, so small-M /
 * large-K problems fill the chip.  K % split_k == 0 and (K / split_k) % 8 == 0.  The order of the atomic adds is
 * not fixed: results can differ between runs in the last bits. */
int tlq_gemm_f16_splitk(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t split_k,
                        int in_dtype, int b_layout, void* stream);

/* Plain GEMV y[N] = A[N,K] . x[K] with fp32 accumulate, replaces simple_gemv (examples/gemv/example_gemv_v.py:17-80 on
 * the vector cores, example_gemv_c.py:16-46 on the cube cores; both y = x @ A.T).  dtype (of x and A): TLQ_F16,
 * TLQ_BF16 or TLQ_F32; a row must be a multiple of 16 bytes; y in out_dtype. */
int tlq_gemv(const void* x, const void* A, void* y, int64_t N, int64_t K, int dtype, int out_dtype, void* stream);

/* int8 x int8 -> int32 GEMM (bit exact), replaces int8_gemm
 * (example_dequant_gemm_fine_grained.py:118-173); batched when batch > 1 (A [B,M,K], B [B,K,N] or
 * [B,N,K], C [B,M,N]). */
int tlq_gemm_i8(const void* A, const void* B, void* C, int64_t batch, int64_t M, int64_t N, int64_t K, int b_layout,
                void* stream);

/* int8 activations x packed int4 weights -> int32, replaces w4a8_gemm_cv
 * (example_dequant_gemm_w4a8.py:25-121) and dequant_gemm_int8_wrapper
 * (example_dequant_gemm_fine_grained.py:226-266): C[M,N] = A[M,K] . convert(sign_mode, Wp)[N,K]^T.
 * The reference's caller-supplied int8 [N,K] workspace is not needed here (unpack is fused); tlq_gemm_w4a8_ws takes it. */
int tlq_gemm_w4a8(const void* A, const void* w_packed, void* C, int64_t M, int64_t N, int64_t K, int sign_mode,
                  void* stream);
/* The same with the reference kernel's third positional, the caller's int8 [N, K] workspace
 * (example_dequant_gemm_w4a8.py:27,69-106 unpacks into it on the vector cores, :108-120 multiplies from it).  With many
 * activation rows (M > 256) and a usable workspace (N * K bytes, 16-byte aligned, K and N multiples of 16) the weights
 * are unpacked into it and the int8 GEMM runs on it, as in the reference; the workspace then holds the unpacked
 * weights.  With few rows the unpack stays fused and K is cut into slices, the workspace holding one int32 [M, N] matrix
 * per slice (as many slices as fit).  Otherwise this is tlq_gemm_w4a8.  The result is the same in every case. */
int tlq_gemm_w4a8_ws(const void* A, const void* w_packed, void* workspace, int64_t workspace_bytes, void* C, int64_t M,
                     int64_t N, int64_t K, int sign_mode, void* stream);

/* W8A8 matmul with fused rescale epilogue, replaces simple_quant_batch_matmul
 * (examples/quant_batch_matmul/example_quant_batch_matmul.py:8-91), simple_quant_matmul
 * (example_quant_matmul.py:8-90) and int8_gemm_kernel_corrected
 * (examples/deepseek_v4/int8_gemm.py:25-104):
 *   acc = A[b] . B[b]            (int32, exact)
 *   C   = rn_out( rn_f32( rn_f32(f32(acc) * scale_a[b,m]) * scale_b[n] ) )
 * scale_a: fp32 [batch*M] or NULL (skipped).  scale_b: fp32 [n_scale_b], n_scale_b = 1 (per
 * tensor) or N (per channel), or NULL.  The reference's int32 [B,M,N] workspace round trip
 * (:42,66-68) is fused away. */
int tlq_gemm_w8a8(const void* A, const void* B, const void* scale_a, const void* scale_b, void* C, int64_t batch,
                  int64_t M, int64_t N, int64_t K, int64_t n_scale_b, int b_layout, int out_dtype, void* stream);

/* The same with an int32 workspace in the place of the reference kernels' workspace_1 [B,M,N]
 * (example_quant_batch_matmul.py:28,42,66-68; example_quant_matmul.py:27,41; deepseek_v4/int8_gemm.py workspace_idx=[5]):
 * with one batch and few activation rows (too few output tiles to fill the machine) K is cut into slices that write
 * their int32 tiles into the workspace, one [M,N] matrix per slice, and a second pass sums and rescales them into C --
 * the same value bit for bit (integer sums are exact in any order).  tlq_w8a8_workspace_bytes gives the size that
 * allows the preferred number of slices (0: this shape is not split); a smaller workspace (16-byte aligned) means fewer
 * slices, none or too small a one means tlq_gemm_w8a8. */
int64_t tlq_w8a8_workspace_bytes(int64_t batch, int64_t M, int64_t N, int64_t K);
int tlq_gemm_w8a8_ws(const void* A, const void* B, const void* scale_a, const void* scale_b, void* C, void* workspace,
                     int64_t workspace_bytes, int64_t batch, int64_t M, int64_t N, int64_t K, int64_t n_scale_b,
                     int b_layout, int out_dtype, void* stream);

/* Offline weight preparation on the GPU.
 * tlq_pack_int4 replaces general_compress (tilelang/quantize/utils.py:53-69, 4-bit source) and, with
 * interleave = 1 (fp16 target) or 2 (int8 target), the interleave_weight that follows it (:73-101):
 * values int8 [N,K] -> packed bytes [N,K/2], value k of a byte pair at bits 4k (not masked, like the
 * reference: out-of-range values spill into their neighbours), then the field permutation within each
 * 32-bit word.  K % 8 == 0.
 * tlq_quantize_sym4 is the quantiser of gen_quant4 (:5-50) for weights stored [N,K] with groups along K:
 * s = max|w| / 8 per group, q = clamp(round(w / s) + 8, 0, 16); writes q - 8 (int8 [N,K]) and s
 * ([N,K/group], dtype of W: TLQ_F16 or TLQ_BF16).  group % 8 == 0. */
int tlq_pack_int4(const void* values, void* packed, int64_t N, int64_t K, int interleave, void* stream);
int tlq_quantize_sym4(const void* W, void* q_minus8, void* scales, int64_t N, int64_t K, int64_t group, int dtype,
                      void* stream);

/* Per-token int8 activation quantiser, replaces act_quant_kernel_int8_optimized
 * (examples/deepseek_v4/act_quant.py:25-92) with the arithmetic of its golden function (:112-142):
 *   amax = max(max_n |x[m,n]|, 1e-4);  scale[m] = amax / 127  (round_scale: 2^ceil(log2(amax / 127)), :95-109)
 *   y[m,n] = int8( rint( clamp(x[m,n] / scale[m], -127, 127) ) ),  all in fp32, round half to even.
 * X: [M,N] in_dtype (TLQ_BF16 like the reference, TLQ_F16 or TLQ_F32), Y: int8 [M,N], S: fp32 [M].
 * Its outputs are the A / scale_a operands of tlq_gemm_w8a8. */
int tlq_act_quant_i8(const void* X, void* Y, void* S, int64_t M, int64_t N, int in_dtype, int round_scale, void* stream);

/* The host-side self-checks of the kernels' address arithmetic (tlq_debug_*) and the tuning hooks that benchmark sweeps and
 * the autotuner use (tlq_tune_*) are exported by the same library and declared in tlq_debug.h: they are not part of the
 * operator boundary above. */

#ifdef __cplusplus
}
#endif
#endif /* TLQ_H_ */
