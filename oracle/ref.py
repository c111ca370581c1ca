"""TEST INFRASTRUCTURE ONLY -- numpy / torch-CPU restatement of the reference arithmetic.

Every function cites the reference lines it follows (paths relative to the reference
checkout).  The restatement is written from the reference's source text; the
reference itself cannot be imported (it needs TVM and torch_npu).

What pins each function (so that a dropped term, wrong nibble order or transposed
operand fails a test):

* unpack_uint4 / torch_unpack_uint4_to_{fp16,int8}: the reference's own known-answer
  vector [[0x12, 0x34]] -> [2, 1, 4, 3]; the literal per-element loop on small shapes;
  an exhaustive 256-byte x 2-position table; the independent C restatement (oracle.c).
* torch_convert (two's-complement int4): exhaustive table; round trip with
  generate_quantized_weight; C restatement.
* general_compress: inverse of the unpackers; brute force on tiny shapes.
* interleave_weight (nbits=4): explicit permutation tables e0,e2,e4,e6,e1,e3,e5,e7
  (fp16) and e0,e4,e1,e5,e2,e6,e3,e7 (int8); the general placement formula bit by bit for
  2-bit sources with the int8 target.  The 1-bit and the 2-bit/float16 special branches call
  ``torch.int32(...)`` in the reference, which raises TypeError; so does this restatement
  (the reference's behaviour is the exception, and a test pins it).
* gen_quant4: invariants only (ref == (q-8).half()*s, shapes, ranges, seed
  reproducibility) -- the random stream itself is torch's.
* dequant_w4 (per-group scale / zero): float64 evaluation followed by one correctly
  rounded conversion per operation (C restatement uses a different rounding routine).
* int8 matmuls: exact int64 brute force on small shapes, float64 matmul (exact below
  2**53) on large ones, the closed form for constant inputs.
* rescale epilogues: pure functions of (acc, scale) -- compared with a float64
  evaluation rounded once.
* lop3 decoders: closed forms (u-8 for signed, (u-z)*s, fma(u,s,-z), (u-qz)*s).
* lop3 decoders for 2-bit and 1-bit sources (lop3_decode_lowbit_to_f16 / _to_i8, lop3_decode_i2_to_i4): the reference
  holds no vectors for them and its own interleave_weight cannot produce their fp16 layouts (see above), so they are
  pinned by what the arithmetic fixes: every one of the 2^16 / 2^8 sources against field-by-field closed forms that index
  the fields by division instead of the decoders' shifts and masks (order f0 f4 f1 f5 f2 f6 f3 f7; u - 2 and 2u - 1 for
  signed; two roundings against one for the 2-bit rescale form, told apart by constants chosen for that), and, for the
  2-bit int8 target, decode(interleave_weight(q, 2, "int8")) == the plain unpack, the one low-bit layout the reference's
  interleave_weight does produce.
* act_quant_torch (per-token int8 quantiser): hand-built rows with known answers (ties at
  .5 fix round-half-to-even, the row maximum maps to +-127, all-zero rows give the 1e-4 / 127
  scale), invariants (odd symmetry, exact invariance under power-of-two rescaling,
  |y * s - x| <= s / 2), and a per-element float32 loop.  pow2_ceil is pinned by a search over
  all powers of two.
"""
from __future__ import annotations

import numpy as np
import torch

TORCH_DTYPE = {
    "float16": torch.float16,
    "bfloat16": torch.bfloat16,
    "float32": torch.float32,
    "int8": torch.int8,
    "int32": torch.int32,
}


def _np_u8(t) -> np.ndarray:
    if isinstance(t, torch.Tensor):
        t = t.cpu()
        if t.dtype == torch.int8:
            t = t.view(torch.uint8)
        return t.numpy()
    a = np.asarray(t)
    return a.view(np.uint8) if a.dtype == np.int8 else a


# --------------------------------------------------------------------------------------
# U1 / U2: unsigned nibble unpack
# --------------------------------------------------------------------------------------
def unpack_uint4_loop(packed, out_dtype=torch.float16) -> torch.Tensor:
    """Literal per-element loop of examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:10-32
    (fp16) and :35-57 (int8).  N*K Python iterations: small inputs only."""
    assert packed.dtype == torch.uint8
    N, K_packed = packed.shape
    K = K_packed * 2
    result = torch.empty(N, K, dtype=out_dtype)
    for i in range(N):
        for j in range(K):
            val = packed[i, j // 2].item()
            pos = j % 2
            u4 = (val >> (pos * 4)) & 0xF
            result[i, j] = float(u4) if out_dtype.is_floating_point else u4
    return result


def unpack_uint4(packed) -> np.ndarray:
    """Vectorised form of the same loop: element k of row n is nibble (k % 2) of byte k // 2,
    low nibble first.  Returns uint8 values 0..15, shape [..., 2*K_packed]."""
    p = _np_u8(packed)
    out = np.empty(p.shape[:-1] + (p.shape[-1] * 2,), dtype=np.uint8)
    out[..., 0::2] = p & 0xF
    out[..., 1::2] = p >> 4
    return out


def torch_unpack_uint4_to_fp16(tensor: torch.Tensor) -> torch.Tensor:
    """example_dequant_gemm_fine_grained.py:10-32, vectorised."""
    assert tensor.dtype == torch.uint8
    return torch.from_numpy(unpack_uint4(tensor).astype(np.float16))


def torch_unpack_uint4_to_int8(tensor: torch.Tensor) -> torch.Tensor:
    """example_dequant_gemm_fine_grained.py:35-57, vectorised."""
    assert tensor.dtype == torch.uint8
    return torch.from_numpy(unpack_uint4(tensor).astype(np.int8))


# --------------------------------------------------------------------------------------
# U3 / P4: two's-complement signed int4
# --------------------------------------------------------------------------------------
def torch_convert_loop(tensor: torch.Tensor) -> torch.Tensor:
    """Literal loop of examples/dequantize_gemm/example_dequant_gemm_w4a8.py:124-145."""

    def _convert(val, pos):
        assert val.dtype == torch.uint8
        val = val.view(torch.int8)
        mask = (1 << 4) - 1
        i4_shifted = (val >> (pos * 4)) & mask
        i4 = (i4_shifted << 4) >> 4
        return i4.view(torch.int8)

    N, K = tensor.shape
    new_tensor = torch.empty(N, K * 2, dtype=torch.int8)
    for i in range(N):
        for j in range(K * 2):
            new_tensor[i][j] = _convert(tensor[i][j // 2], j % 2)
    return new_tensor


def torch_convert(tensor) -> torch.Tensor:
    """Vectorised example_dequant_gemm_w4a8.py:124-145: nibble -> sign-extended int8 (-8..7)."""
    u = unpack_uint4(tensor).astype(np.int16)
    return torch.from_numpy(np.where(u >= 8, u - 16, u).astype(np.int8))


def generate_quantized_weight(N: int, K: int, generator: torch.Generator | None = None):
    """example_dequant_gemm_w4a8.py:156-165 with the loop vectorised:
    qB[n, j] = (B[n, 2j+1] & 15) << 4 | (B[n, 2j] & 15)."""
    B_int8 = torch.randint(-8, 8, (N, K), dtype=torch.int8, generator=generator)
    b = B_int8.numpy().view(np.uint8)
    qB = ((b[:, 1::2] & 0xF) << 4) | (b[:, 0::2] & 0xF)
    return torch.from_numpy(qB.astype(np.uint8)), B_int8


# --------------------------------------------------------------------------------------
# Q1..Q5: tilelang.quantize element converters, restated on integer arrays
# --------------------------------------------------------------------------------------
def _field(val, pos, nbit):
    v = np.asarray(val).astype(np.int64) & 0xFFFFFFFF
    return (v >> (np.asarray(pos).astype(np.int64) * nbit)) & ((1 << nbit) - 1)


def packed_to_unsigned(val, pos, nbit=4):
    """tilelang/quantize/quantization.py:198-206: (val >> pos*nbit) & mask."""
    return _field(val, pos, nbit)


def packed_to_unsigned_with_zeros(val, pos, zero, nbit=4):
    """quantization.py:209-218: ((val >> pos*nbit) & mask) - zero, exact integer subtraction."""
    return _field(val, pos, nbit) - np.asarray(zero).astype(np.int64)


def packed_to_signed_offset(val, pos, nbit=4):
    """quantization.py:186-195: offset-binary, u - 2**(nbit-1)."""
    return _field(val, pos, nbit) - (1 << (nbit - 1))


def packed_int_to_int(val, pos, nbit=4):
    """quantization.py:221-231 (and :68-78): two's-complement sign extension of the field."""
    u = _field(val, pos, nbit)
    return np.where(u >= (1 << (nbit - 1)), u - (1 << nbit), u)


def packed_uint_to_uint_to_float(val, pos, nbit=4):
    """quantization.py:56-65: u - (2**(nbit-1) - 1)."""
    return _field(val, pos, nbit) - ((1 << (nbit - 1)) - 1)


# --------------------------------------------------------------------------------------
# P1..P3: tilelang/quantize/utils.py
# --------------------------------------------------------------------------------------
def general_compress(lowprecision_weight: torch.Tensor, source_bits=4, storage_dtype=None) -> torch.Tensor:
    """tilelang/quantize/utils.py:53-69.  out[..., j] |= (w[..., j*epb+k] << bits*k) truncated to
    8 bits, accumulated in int8, then cast to storage_dtype."""
    if storage_dtype is None:
        storage_dtype = torch.int8
    epb = 8 // source_bits
    w = lowprecision_weight
    if w.dtype == torch.float16:
        w = w.to(torch.int8)
    a = w.cpu().numpy().astype(np.int64)
    out = np.zeros(a.shape[:-1] + (a.shape[-1] // epb,), dtype=np.int64)
    for k in range(epb):
        out |= (a[..., k::epb][..., : out.shape[-1]] << (source_bits * k)) & 0xFF
    return torch.from_numpy(out.astype(np.uint8).view(np.int8).copy()).to(storage_dtype)


def interleave_weight(qweight: torch.Tensor, nbits=4, target_dtype="float16") -> torch.Tensor:
    """tilelang/quantize/utils.py:73-126.  Per 32-bit word, field i moves to bit
    (i % G) * stride + (i // G) * nbits with stride 16 (fp16) / 8 (int8), G = 32 // stride."""
    assert target_dtype in ["float16", "int8"]
    q = qweight.cpu().contiguous().view(torch.int32).numpy().view(np.uint32)
    new = np.zeros_like(q)
    stride = 8 if target_dtype == "int8" else 16
    mask = np.uint32((1 << nbits) - 1)
    G = 32 // stride
    per = stride // nbits
    for i in range(G):
        for j in range(per):
            off = i * per + j
            shift = (off % G) * stride + (off // G) * nbits
            new |= ((q >> np.uint32(nbits * off)) & mask) << np.uint32(shift)

    # For 1-bit sources and for 2-bit sources with the float16 target the reference goes on to regroup nibbles /
    # bytes with masks written torch.int32(0x...) (utils.py:103-124); torch.int32 is a dtype object and calling it
    # raises TypeError, so those three branches never return a value in the reference.  Same behaviour here.
    if nbits == 1 or (nbits == 2 and target_dtype == "float16"):
        raise TypeError("'torch.dtype' object is not callable (interleave_weight of %d-bit weights for %s: the reference "
                        "raises here, tilelang/quantize/utils.py:103-124)" % (nbits, target_dtype))
    return torch.from_numpy(new.view(np.int32).copy()).view(torch.int8)


def gen_quant4(k, n, groupsize=-1):
    """tilelang/quantize/utils.py:5-50, same torch calls in the same order (so the same seed
    gives the same stream).  Note maxq = 16 and the clamp to [0, 16] (sic)."""
    import torch.nn as nn

    maxq = 2**4
    w = torch.randn((k, n), dtype=torch.half, device="cpu")
    original_w = w.clone()
    if groupsize == -1:
        groupsize = k
    w = w.reshape((-1, groupsize, n)).permute(1, 0, 2).reshape((groupsize, -1))
    s = torch.max(torch.abs(w), 0, keepdim=True)[0]
    s *= 2 / maxq
    w = torch.round(w / s).int()
    w += maxq // 2
    w = torch.clamp(w, 0, maxq)
    ref = (w - maxq // 2).half() * s

    def reshape(x):
        return x.reshape((groupsize, -1, n)).permute(1, 0, 2).reshape((k, n)).contiguous()

    ref = reshape(ref)
    w = reshape(w)
    s = s.reshape((-1, n)).contiguous()
    linear = nn.Linear(k, n, bias=False)
    linear.weight.data = ref.t()
    return original_w, linear, s, (w - maxq // 2)


# --------------------------------------------------------------------------------------
# Per-group dequantisation: W[n,k] = rn_T( rn_T(T(u) - T(z[n,k//g])) * s[n,k//g] )
# ("original" zeros mode of tilelang/quantize/lop3.py:135-175: sub.f16x2 then fma.rn.f16x2
#  with a zero addend; gen_quant4's ref = (q-8).half()*s, utils.py:33)
# --------------------------------------------------------------------------------------
def dequant_w4(B_packed, scales=None, zeros=None, group_size=128, dtype=torch.float16) -> torch.Tensor:
    """scales: [N, K/g] tensor of dtype T or None (=1).  zeros: None (=0), a python number, or a
    [N, K/g] tensor of dtype T.  Each arithmetic step rounds to T (torch CPU half/bfloat16
    arithmetic computes in fp32 and rounds once per operation, which equals native rounding)."""
    u = torch.from_numpy(unpack_uint4(B_packed).astype(np.float32)).to(dtype)
    N, K = u.shape
    if zeros is not None:
        if isinstance(zeros, torch.Tensor):
            z = zeros.cpu().to(dtype).repeat_interleave(group_size, dim=1)
            assert z.shape == (N, K)
        else:
            z = torch.tensor(float(zeros), dtype=dtype)
        u = u - z
    if scales is not None:
        s = scales.cpu().to(dtype).repeat_interleave(group_size, dim=1)
        assert s.shape == (N, K)
        u = u * s
    return u


def ref_program_w4a16(A, B_packed, scales=None, zeros=None, group_size=128, output_dtype="float16"):
    """ref_program_fp16 (example_dequant_gemm_fine_grained.py:269-289) extended with the group
    dequant above: (A.f32 @ W.f32.T).to(out).  A is NOT down-cast (line :283)."""
    W = dequant_w4(B_packed, scales, zeros, group_size, A.dtype)
    C = torch.matmul(A.cpu().to(torch.float32), W.to(torch.float32).T)
    return C.to(TORCH_DTYPE[output_dtype])


def ref_program_fp16(A, B_packed, output_dtype):
    """example_dequant_gemm_fine_grained.py:269-289 (vectorised unpack)."""
    B_fp16 = torch_unpack_uint4_to_fp16(B_packed)
    C = torch.matmul(A.to(torch.float32), B_fp16.to(torch.float32).T)
    return C.to(TORCH_DTYPE[output_dtype])


def ref_program_fp16_loop(A, B_packed, output_dtype):
    """Same, with the literal per-element unpack loop (small shapes only)."""
    B_fp16 = unpack_uint4_loop(B_packed, torch.float16)
    C = torch.matmul(A.to(torch.float32), B_fp16.to(torch.float32).T)
    return C.to(TORCH_DTYPE[output_dtype])


# --------------------------------------------------------------------------------------
# Integer matmuls
# --------------------------------------------------------------------------------------
def int_matmul_exact(A, B) -> torch.Tensor:
    """Exact integer A @ B through float64 (every partial sum is an integer < 2**53).
    Batched when the inputs are 3-D.  Returns int64."""
    return torch.matmul(A.cpu().to(torch.float64), B.cpu().to(torch.float64)).to(torch.int64)


def ref_program_int8(A, B_packed, output_dtype):
    """example_dequant_gemm_fine_grained.py:292-312: (A.i32 @ U2(Wp).i32.T).to(out)."""
    B_int8 = torch_unpack_uint4_to_int8(B_packed)
    C = int_matmul_exact(A, B_int8.T).to(torch.int32)
    return C.to(TORCH_DTYPE[output_dtype])


def ref_program_w4a8(A, qB):
    """example_dequant_gemm_w4a8.py:148-153: returns the TRANSPOSE [N, M] (int32)."""
    B = torch_convert(qB)
    C = torch.matmul(A.cpu().to(torch.float), B.T.to(torch.float)).to(torch.int32)
    return C.transpose(0, 1)


def ref_program_quant(A, B, scale, out_dtype, accum_dtype=torch.int32, literal=False):
    """examples/quant_batch_matmul/example_quant_batch_matmul.py:93-95 and
    example_quant_matmul.py:92-94: ((A.acc @ B.acc).to(scale.dtype) * scale).to(out).
    literal=True runs torch's own integer matmul (slow); otherwise the exact float64 route."""
    if literal:
        C = A.cpu().to(accum_dtype) @ B.cpu().to(accum_dtype)
    else:
        C = int_matmul_exact(A, B).to(accum_dtype)
    return (C.to(scale.dtype) * scale.cpu()).to(out_dtype)


def ref_int8_gemm_sequential(A, B_nk, scale_a, scale_b, out_dtype):
    """Kernel order of examples/deepseek_v4/int8_gemm.py:95-102: cast acc to fp32 (RINT),
    multiply by scale_a[m], then by scale_b[n] (two fp32 roundings), cast to out (RINT)."""
    acc = int_matmul_exact(A, B_nk.transpose(-1, -2)).to(torch.int32)
    c = acc.to(torch.float32)
    c = c * scale_a.cpu().reshape(*scale_a.shape[: A.dim() - 1], 1).to(torch.float32)
    c = c * scale_b.cpu().reshape(-1).to(torch.float32)
    return c.to(out_dtype)


def int8_gemm_torch_optimized(a_int8, a_scales, b_int8, b_scales, out_dtype=torch.float32):
    """Golden of examples/deepseek_v4/int8_gemm.py:108-139: fp32 matmul times outer(a_s, b_s).
    The fp32 matmul is inexact for full-range int8 at large K -- a tolerance oracle only."""
    shape = a_int8.shape
    a2 = a_int8.reshape(-1, shape[-1]).to(torch.float32)
    out = torch.matmul(a2, b_int8.to(torch.float32).T)
    out = out * torch.outer(a_scales.reshape(-1), b_scales.reshape(-1))
    if out_dtype == torch.bfloat16:
        out = out.bfloat16()
    return out.view(*shape[:-1], b_int8.shape[0])


# --------------------------------------------------------------------------------------
# Q6: closed forms of the lop3 decoders (tilelang/quantize/lop3.py:5-421), 4-bit -> fp16
# --------------------------------------------------------------------------------------
LOP3_F16_ORDER = (0, 4, 1, 5, 2, 6, 3, 7)  # output slot j holds field LOP3_F16_ORDER[j] of the u32


def lop3_decode_i4_to_f16(words_u32, signed=False, scale=None, zeros=None, zeros_mode=None, scale_r=None, zeros_r=None):
    """One u32 -> 8 fp16.  h[i] (a half2) = fields (i, i+4) of the word (lop3.py:17-24), so the
    flat output order is field 0,4,1,5,2,6,3,7: the weights must have been passed through
    interleave_weight for the flat order to be the logical one.  signed subtracts 8 (:14).
    zeros_mode: None | 'original' (u - z) * s (:165-166) | 'rescale' fma(u, s, -|z|) (:247,260: the addend is the
    zero point with its sign bit forced) | 'quantized' (u - qz) * s with integer qz (:340,351-353).
    scale_r / zeros_r: the "_offset" forms (:82-131, 177-230, 272-322, 364-421) -- h[0], h[1] (flat outputs 0..3) use
    scale / zeros, h[2], h[3] (flat outputs 4..7) use scale_r / zeros_r."""
    w = np.asarray(words_u32, dtype=np.uint32).reshape(-1)
    f = np.stack([(w >> np.uint32(4 * i)) & np.uint32(0xF) for i in LOP3_F16_ORDER], axis=1)
    h = f.astype(np.float16)
    if signed:
        h = h - np.float16(8)

    def half(a):  # one value per output column: first four from the left parameter, last four from the right one
        l, r = a
        return np.array([l] * 4 + [l if r is None else r] * 4)

    if zeros_mode in ("original", "quantized"):
        h = (h - half((zeros, zeros_r)).astype(np.float16)).astype(np.float16)
    if scale is not None:
        sc = half((scale, scale_r)).astype(np.float16)
        if zeros_mode == "rescale":
            z = np.abs(half((zeros, zeros_r)).astype(np.float16))
            h = (h.astype(np.float64) * sc.astype(np.float64) - z.astype(np.float64)).astype(np.float16)
        else:
            h = (h * sc).astype(np.float16)
    return h


# --------------------------------------------------------------------------------------
# The 2-bit and 1-bit lop3 decoders (tilelang/quantize/lop3.py:423-996, 1048-1087), restated step by step: the spread of
# the source bits, the shift + mask + OR of the magic number per output pair, then the packed fp16 arithmetic in the
# reference's order (every operation rounds to fp16).  tests/test_oracle.py pins them on all 2^16 / 2^8 sources against
# field-by-field closed forms written independently of the shifts used here.
# --------------------------------------------------------------------------------------
def _f16_from_bits(u16):
    return np.asarray(u16, dtype=np.uint16).view(np.float16)


def lop3_decode_lowbit_to_f16(src, source_bit, signed=False, scale=None, zeros=None, zeros_mode=None):
    """src: uint16 array (2-bit: 8 fields per element) or uint8 array (1-bit: 8 bits per element) -> [n, 8] fp16.
    2-bit (lop3.py:423-676): i2s = (w & 0xff) | ((w & 0xff00) << 8); h[i] = ((i2s >> 2i) & 0x00030003) | 0x64006400,
    minus 0x6400 (unsigned) or 0x6402 (signed: u - 2); then scale: fma(h, s, 0); original: (h - z) then fma(., s, 0);
    rescale: fma(h, s, 0) then - z (two roundings, :626-627); quantized: h + (0xe400 | qz) then fma(., s, 0) (:656,668-669).
    1-bit (lop3.py:678-890): i1s = (b & 0x0f) | ((b & 0xf0) << 12); h[i] = ((i1s >> i) & 0x00010001) | 0x64006400, minus
    0x6400; signed: h + h, then + 0xbc00 (-1) (:712-716); scale: fma(h, s, 0); original: (h - z) then fma(., s, 0);
    rescale: fma(h, s, 0x8000 | z) -- one rounding, the addend with its sign bit forced (:870,880)."""
    assert source_bit in (2, 1)
    f16 = np.float16
    if source_bit == 2:
        w = np.asarray(src, dtype=np.uint16).reshape(-1).astype(np.uint32)
        spread = (w & np.uint32(0x00FF)) | ((w & np.uint32(0xFF00)) << np.uint32(8))
        mask, step = np.uint32(0x00030003), 2
    else:
        w = np.asarray(src, dtype=np.uint8).reshape(-1).astype(np.uint32)
        spread = (w & np.uint32(0x0F)) | ((w & np.uint32(0xF0)) << np.uint32(12))
        mask, step = np.uint32(0x00010001), 1
    out = np.empty((w.size, 8), dtype=f16)
    for i in range(4):
        h = ((spread >> np.uint32(step * i)) & mask) | np.uint32(0x64006400)
        for half, col in ((h & np.uint32(0xFFFF), 2 * i), (h >> np.uint32(16), 2 * i + 1)):
            x = _f16_from_bits(half.astype(np.uint16))
            if zeros_mode == "quantized":
                assert source_bit == 2
                qz = np.uint16(np.int16(zeros)) if np.ndim(zeros) == 0 else np.asarray(zeros, dtype=np.int16).view(np.uint16)
                x = (x + _f16_from_bits(np.uint16(0xE400) | qz)).astype(f16)
            else:
                median = 0x6402 if (source_bit == 2 and signed) else 0x6400
                x = (x - _f16_from_bits(np.uint16(median))).astype(f16)
                if source_bit == 1 and signed:
                    x = (x + x).astype(f16)
                    x = (x + _f16_from_bits(np.uint16(0xBC00))).astype(f16)
            if zeros_mode == "original":
                x = (x - f16(zeros)).astype(f16)
            if scale is not None:
                if zeros_mode == "rescale" and source_bit == 1:
                    nz = _f16_from_bits(np.asarray(f16(zeros)).view(np.uint16) | np.uint16(0x8000))
                    x = (x.astype(np.float64) * np.float64(f16(scale)) + nz.astype(np.float64)).astype(f16)
                else:
                    x = (x.astype(np.float64) * np.float64(f16(scale))).astype(f16)  # fma with a zero addend: one rounding
                    if zeros_mode == "rescale":
                        x = (x - f16(zeros)).astype(f16)
            out[:, col] = x
    return out


def lop3_decode_lowbit_to_i8(src, source_bit, signed=False):
    """2-bit (lop3.py:949-996): src uint32, word i of the output = (w >> 2i) & 0x03030303, signed: minus 2 per byte.
    1-bit (lop3.py:892-947): src uint16, i1b = (w & 0x0f0f) | ((w & 0xf0f0) << 12), word i = (i1b >> i) & 0x01010101,
    signed: per byte x + x, then + 0xff (:916-917).  Returns [n, 16] int8 in memory order (word i, byte lane b at 4i + b)."""
    assert source_bit in (2, 1)
    if source_bit == 2:
        w = np.asarray(src, dtype=np.uint32).reshape(-1)
        words = [(w >> np.uint32(2 * i)) & np.uint32(0x03030303) for i in range(4)]
    else:
        w16 = np.asarray(src, dtype=np.uint16).reshape(-1).astype(np.uint32)
        i1b = (w16 & np.uint32(0x0F0F)) | ((w16 & np.uint32(0xF0F0)) << np.uint32(12))
        words = [(i1b >> np.uint32(i)) & np.uint32(0x01010101) for i in range(4)]
    by = np.stack(words, axis=1).astype("<u4").view(np.uint8).reshape(-1, 16)
    if signed:
        by = (by - np.uint8(2)) if source_bit == 2 else ((by + by) + np.uint8(0xFF))  # uint8 arithmetic wraps per byte
    return by.astype(np.uint8).view(np.int8)


def lop3_decode_i2_to_i4(src):
    """lop3.py:1048-1087 (N = 16): word i of the output = (w >> 2 (i % 2)) & 0x33333333 for i = 0, 1 (i / 2 = 0: the one
    source word); the signed form's body is a comment, so signed and unsigned agree.  Returns [n, 2] uint32."""
    w = np.asarray(src, dtype=np.uint32).reshape(-1)
    return np.stack([(w >> np.uint32(2 * (i % 2))) & np.uint32(0x33333333) for i in range(2)], axis=1)


# --------------------------------------------------------------------------------------
# A1: per-token int8 activation quantiser (examples/deepseek_v4/act_quant.py)
# --------------------------------------------------------------------------------------
def pow2_ceil(s):
    """Smallest power of two >= s for positive normal float32 s: the bit arithmetic of
    fast_log2_ceil / fast_pow2 (examples/deepseek_v4/act_quant.py:93-105) -- the exponent field,
    plus one when any mantissa bit is set."""
    s = np.asarray(s, dtype=np.float32)
    bits = s.view(np.uint32)
    e = ((bits >> 23) & 0xFF).astype(np.int64) + (bits & 0x7FFFFF != 0)
    return (e.astype(np.uint32) << 23).view(np.float32)


def act_quant_torch(x: torch.Tensor, round_scale: bool = False, exact_log2: bool = False):
    """Golden of examples/deepseek_v4/act_quant.py:112-142, all in float32 on the CPU.
    Returns (int8 tensor of x's shape, float32 scales [..., 1]).

    ``exact_log2`` replaces ``2 ** ceil(log2(.))`` by pow2_ceil: torch.log2 rounds its result,
    so a scale within a few ulp above a power of two 2**k (|k| >= 2) has log2 == k exactly and
    the literal form returns 2**k instead of 2**(k+1)."""
    shape = x.shape
    x2 = x.reshape(-1, shape[-1]).float()
    abs_max = torch.max(torch.abs(x2), dim=1, keepdim=True)[0]
    abs_max = torch.clamp(abs_max, min=1e-4)
    if round_scale:
        if exact_log2:
            scales = torch.from_numpy(pow2_ceil((abs_max / 127.0).numpy()))
        else:
            scales = 2 ** torch.ceil(torch.log2(abs_max / 127.0))
    else:
        scales = abs_max / 127.0
    clipped = torch.clamp(x2 / scales, -127, 127)
    y = torch.round(clipped).to(torch.float16).to(torch.int8)
    return y.view(shape), scales.view(*shape[:-1], 1)


def act_quant_loop(x: torch.Tensor):
    """Per-element float32 loop of the same definition (small inputs only)."""
    x2 = x.float().numpy()
    M, N = x2.shape
    y = np.zeros((M, N), dtype=np.int8)
    s = np.zeros(M, dtype=np.float32)
    for m in range(M):
        amax = np.float32(1e-4)
        for n in range(N):
            amax = max(amax, np.float32(abs(x2[m, n])))
        s[m] = np.float32(amax) / np.float32(127.0)
        for n in range(N):
            q = np.float32(x2[m, n]) / s[m]
            q = min(max(q, np.float32(-127.0)), np.float32(127.0))
            y[m, n] = int(np.rint(q))
    return y, s


# --------------------------------------------------------------------------------------
# N1: non-quantised twins (examples/gemv, examples/gemm_splitk)
# --------------------------------------------------------------------------------------
def ref_program_gemv(x: torch.Tensor, A: torch.Tensor) -> torch.Tensor:
    """examples/gemv/example_gemv_v.py:83-84 (``x @ A.T``), evaluated in float64 and rounded once to
    x's dtype: the kernels accumulate in float32, so this is a tolerance oracle (pinned by the
    one-hot and constant-row closed forms in the tests)."""
    return (A.double() @ x.double()).to(x.dtype)


def ref_program_splitk(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """examples/gemm_splitk/example_tilelang_gemm_splitk.py:66 (``a @ b`` compared in float32), in float64."""
    return (a.double() @ b.double()).float()


# --------------------------------------------------------------------------------------
# P5: the quantiser inside gen_quant4 for weights stored [N, K], groups along K
# --------------------------------------------------------------------------------------
def quantize_sym4(W: torch.Tensor, group: int):
    """tilelang/quantize/utils.py:20-31 on W [N, K] (the reference holds w [k, n] and groups along k:
    the same numbers, transposed): s = max|w| * (2 / 16) in W's dtype, q = clamp(round(w / s).int() + 8, 0, 16).
    Returns (q - 8 as int8, s [N, K/group]).  A group of zeros divides 0 by 0; the int conversion of the
    NaN is the most negative integer on x86, so q = 0 there (q - 8 = -8)."""
    N, K = W.shape
    wg = W.reshape(N, K // group, group)
    s = wg.abs().amax(dim=2, keepdim=True) * (2 / 16)
    quot = torch.round(wg / s).float()                      # w / s is rounded to W's dtype before the round
    quot = torch.where(torch.isnan(quot), torch.full_like(quot, -1e9), quot)
    q = torch.clamp(quot.to(torch.int64) + 8, 0, 16)
    return (q - 8).to(torch.int8).reshape(N, K), s.reshape(N, K // group).contiguous()
