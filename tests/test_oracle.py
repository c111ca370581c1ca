"""Pins of the CPU oracle (oracle/ref.py, oracle/oracle.c).

The oracle is only useful as a checker if it is itself checked by something other than a copy
of its own formula.  Each test below uses one of: the reference's own known-answer vector, the
literal per-element loops of the reference's examples, exhaustive tables computed with plain
Python integers, inverse/round-trip relations between independent functions, closed forms for
constant inputs, or the independent C restatement (its own rounding routine, its own loops).
"""
import json
import os

import numpy as np
import pytest
import torch

from oracle import cref, ref

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _rng(seed):
    return torch.Generator().manual_seed(seed)


# ------------------------------------------------------------------------------------------------
# unsigned nibble unpack
# ------------------------------------------------------------------------------------------------
def test_reference_known_answer_vector():
    # examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:384-401
    kat = json.load(open(os.path.join(GOLDEN, "kat_unpack_uint4.json")))
    packed = torch.tensor(kat["packed"], dtype=torch.uint8)
    for fn, dt in ((ref.torch_unpack_uint4_to_fp16, torch.float16), (ref.torch_unpack_uint4_to_int8, torch.int8)):
        out = fn(packed)
        assert out.dtype == dt and list(out.shape) == kat["shape"]
        assert out.tolist() == [[float(v) if dt.is_floating_point else v for v in row] for row in kat["expected"]]
    assert ref.unpack_uint4_loop(packed, torch.int8).tolist() == kat["expected"]
    assert cref.unpack_u4(packed.numpy()).tolist() == kat["expected"]


def test_unpack_exhaustive_table_plain_python():
    packed = torch.arange(256, dtype=torch.uint8).reshape(256, 1)
    want = [[b & 15, b >> 4] for b in range(256)]
    assert ref.unpack_uint4(packed).tolist() == want
    assert cref.unpack_u4(packed.numpy()).tolist() == want


def test_unpack_vectorised_equals_literal_loop():
    packed = torch.randint(0, 256, (7, 9), dtype=torch.uint8, generator=_rng(1))
    assert torch.equal(ref.torch_unpack_uint4_to_fp16(packed), ref.unpack_uint4_loop(packed, torch.float16))
    assert torch.equal(ref.torch_unpack_uint4_to_int8(packed), ref.unpack_uint4_loop(packed, torch.int8))


# ------------------------------------------------------------------------------------------------
# two's-complement int4
# ------------------------------------------------------------------------------------------------
def test_signed_convert_exhaustive_and_loop():
    packed = torch.arange(256, dtype=torch.uint8).reshape(256, 1)

    def s4(v):
        return v - 16 if v >= 8 else v

    want = [[s4(b & 15), s4(b >> 4)] for b in range(256)]
    assert ref.torch_convert(packed).tolist() == want
    assert cref.convert_s4(packed.numpy()).tolist() == want
    small = torch.randint(0, 256, (5, 6), dtype=torch.uint8, generator=_rng(2))
    assert torch.equal(ref.torch_convert(small), ref.torch_convert_loop(small))


def test_signed_round_trip_with_weight_generator():
    # example_dequant_gemm_w4a8.py:156-165 packs, :124-145 unpacks; the example asserts equality (:182)
    qB, B = ref.generate_quantized_weight(33, 64, generator=_rng(3))
    assert qB.dtype == torch.uint8 and qB.shape == (33, 32)
    assert B.min() >= -8 and B.max() <= 7
    assert torch.equal(ref.torch_convert(qB), B)
    # literal packing loop of the reference on the same values
    lit = torch.empty_like(qB)
    for i in range(33):
        for j in range(32):
            lit[i, j] = ((int(B[i, 2 * j + 1]) & 0xF) << 4) | (int(B[i, 2 * j]) & 0xF)
    assert torch.equal(lit, qB)


# ------------------------------------------------------------------------------------------------
# tilelang.quantize element converters: 16-entry tables
# ------------------------------------------------------------------------------------------------
def test_converter_tables():
    word = 0xFEDCBA98_76543210 & 0xFFFFFFFF  # nibbles 0..7 in positions 0..7
    word_hi = 0xFEDCBA98
    pos = np.arange(8)
    u_lo = ref.packed_to_unsigned(word, pos).tolist()
    u_hi = ref.packed_to_unsigned(word_hi, pos).tolist()
    assert u_lo == list(range(8)) and u_hi == list(range(8, 16))
    u = np.arange(16)
    words = np.array([word] * 8 + [word_hi] * 8)
    posn = np.concatenate([pos, pos])
    assert ref.packed_to_signed_offset(words, posn).tolist() == (u - 8).tolist()
    assert ref.packed_uint_to_uint_to_float(words, posn).tolist() == (u - 7).tolist()
    assert ref.packed_int_to_int(words, posn).tolist() == [v - 16 if v >= 8 else v for v in range(16)]
    for z in (0, 6, 8, 9, 15):
        assert ref.packed_to_unsigned_with_zeros(words, posn, z).tolist() == (u - z).tolist()
    # int8 storage (negative python ints) must give the same fields as the uint8 view
    assert ref.packed_to_unsigned(np.int8(-1), 1).item() == 15
    # 2-bit fields
    assert ref.packed_to_unsigned(0b11100100, np.arange(4), nbit=2).tolist() == [0, 1, 2, 3]
    assert ref.packed_int_to_int(0b11100100, np.arange(4), nbit=2).tolist() == [0, 1, -2, -1]


# ------------------------------------------------------------------------------------------------
# general_compress / interleave_weight / gen_quant4
# ------------------------------------------------------------------------------------------------
def test_general_compress_inverts_the_unpackers():
    w = torch.randint(0, 16, (6, 32), dtype=torch.int8, generator=_rng(4))
    packed = ref.general_compress(w, 4, torch.int8)
    assert packed.dtype == torch.int8 and packed.shape == (6, 16)
    assert np.array_equal(ref.unpack_uint4(packed), w.numpy())
    ws = torch.randint(-8, 8, (6, 32), dtype=torch.int8, generator=_rng(5))
    assert torch.equal(ref.torch_convert(ref.general_compress(ws & 15, 4, torch.int8).view(torch.uint8)), ws)
    # the reference does not mask its operands (tilelang/quantize/utils.py:64-67): the sign bits of a
    # negative low element smear into the high nibble, so callers must pass values 0..15
    smear = ref.general_compress(torch.tensor([[-1, 0]], dtype=torch.int8), 4, torch.int8)
    assert smear.view(torch.uint8).tolist() == [[0xFF]]
    # fp16 input takes the .to(int8) route (tilelang/quantize/utils.py:58-59)
    assert torch.equal(ref.general_compress(w.half(), 4, torch.int8), packed)
    # brute force on a tiny case with plain integers, 4-bit and 2-bit
    for bits in (4, 2):
        epb = 8 // bits
        t = torch.randint(0, 1 << bits, (2, 2 * epb), dtype=torch.int8, generator=_rng(6))
        want = [[sum(int(t[r, j * epb + k]) << (bits * k) for k in range(epb)) for j in range(2)] for r in range(2)]
        got = ref.general_compress(t, bits, torch.int8).view(torch.uint8).tolist()
        assert got == want


def test_interleave_weight_permutation_tables():
    # one word whose nibble i holds the value i
    base = torch.tensor([[0x10, 0x32, 0x54, 0x76]], dtype=torch.uint8).view(torch.int8)
    f16 = ref.unpack_uint4(ref.interleave_weight(base, 4, "float16")).tolist()[0]
    i8 = ref.unpack_uint4(ref.interleave_weight(base, 4, "int8")).tolist()[0]
    assert f16 == [0, 2, 4, 6, 1, 3, 5, 7]
    assert i8 == [0, 4, 1, 5, 2, 6, 3, 7]
    # the general formula: field i lands at bit (i % G) * stride + (i // G) * nbits
    for nbits, target, stride in ((4, "float16", 16), (4, "int8", 8), (2, "int8", 8)):
        G, nf = 32 // stride, 32 // nbits
        for i in range(nf):
            word = ((1 << nbits) - 1) << (nbits * i)
            src = torch.tensor([word], dtype=torch.int64).to(torch.int32).view(torch.int8).reshape(1, 4)
            got = ref.interleave_weight(src, nbits, target).reshape(-1).view(torch.int32).item() & 0xFFFFFFFF
            assert got == ((1 << nbits) - 1) << ((i % G) * stride + (i // G) * nbits), (nbits, target, i)
    # nibble permutation of random data: multiset of nibbles per word unchanged
    q = torch.randint(-128, 128, (3, 16), dtype=torch.int8, generator=_rng(7))
    a = np.sort(ref.unpack_uint4(q).reshape(3, 4, 8), axis=-1)
    b = np.sort(ref.unpack_uint4(ref.interleave_weight(q, 4, "float16")).reshape(3, 4, 8), axis=-1)
    assert np.array_equal(a, b)


def test_lop3_decode_of_interleaved_weights_is_the_plain_unpack():
    q = torch.randint(0, 256, (4, 8), dtype=torch.uint8, generator=_rng(8))
    inter = ref.interleave_weight(q.view(torch.int8), 4, "float16")
    words = inter.contiguous().view(torch.int32).numpy().view(np.uint32).reshape(-1)
    plain = ref.unpack_uint4(q).reshape(-1, 8).astype(np.float16)
    assert np.array_equal(ref.lop3_decode_i4_to_f16(words), plain)
    assert np.array_equal(ref.lop3_decode_i4_to_f16(words, signed=True), plain - np.float16(8))
    s, z = 0.0123, 7.0
    s16, z16 = np.float16(s), np.float16(z)
    orig = ref.lop3_decode_i4_to_f16(words, scale=s, zeros=z, zeros_mode="original")
    assert np.array_equal(orig, ((plain - z16).astype(np.float16) * s16).astype(np.float16))
    resc = ref.lop3_decode_i4_to_f16(words, scale=s, zeros=z, zeros_mode="rescale")
    exact = plain.astype(np.float64) * float(s16) - float(z16)  # single rounding (fma)
    assert np.array_equal(resc, exact.astype(np.float16))
    # a negative zero point enters the fused form with its sign bit forced (0x80008000 | zeros, lop3.py:247): -|z| again
    assert np.array_equal(ref.lop3_decode_i4_to_f16(words, scale=s, zeros=-z, zeros_mode="rescale"), resc)


def test_lop3_offset_forms_use_one_group_per_half():
    """The "_offset" decoders (lop3.py:82-131, 177-230, 272-322, 364-421): outputs 0..3 of a word take the first
    scale / zero point, outputs 4..7 the one `offset` further on.  Checked element by element with scalar arithmetic,
    and against the one-group forms when both halves get the same parameters."""
    q = torch.randint(0, 256, (6, 4), dtype=torch.uint8, generator=_rng(18))
    words = ref.interleave_weight(q.view(torch.int8), 4, "float16").contiguous().view(torch.int32).numpy().view(np.uint32).reshape(-1)
    plain = ref.unpack_uint4(q).reshape(-1, 8)
    sl, sr, zl, zr = 0.011, 0.019, 6.5, 9.0
    for mode in (None, "original", "rescale", "quantized"):
        zl_, zr_ = (7, 12) if mode == "quantized" else (zl, zr)
        kw = {} if mode is None else dict(zeros=zl_, zeros_r=zr_, zeros_mode=mode)
        got = ref.lop3_decode_i4_to_f16(words, scale=sl, scale_r=sr, **kw)
        same = ref.lop3_decode_i4_to_f16(words, scale=sl, scale_r=sl, **dict(kw, zeros_r=zl_) if kw else {})
        one = ref.lop3_decode_i4_to_f16(words, scale=sl, **({} if mode is None else dict(zeros=zl_, zeros_mode=mode)))
        assert np.array_equal(same, one), mode
        for w in range(plain.shape[0]):
            for j in range(8):
                s16 = np.float16(sl if j < 4 else sr)
                z16 = np.float16(zl_ if j < 4 else zr_)
                u = np.float16(plain[w, j])
                if mode is None:
                    want = np.float16(u * s16)
                elif mode == "rescale":
                    want = np.float16(float(u) * float(s16) - float(z16))
                else:
                    want = np.float16(np.float16(u - z16) * s16)
                assert got[w, j] == want, (mode, w, j)
    signed = ref.lop3_decode_i4_to_f16(words, signed=True, scale=sl, scale_r=sr)
    assert np.array_equal(signed[:, :4], ((plain[:, :4].astype(np.float16) - np.float16(8)) * np.float16(sl)).astype(np.float16))
    assert np.array_equal(signed[:, 4:], ((plain[:, 4:].astype(np.float16) - np.float16(8)) * np.float16(sr)).astype(np.float16))


def test_gen_quant4_invariants():
    torch.manual_seed(0)
    k, n, g = 256, 24, 64
    w0, linear, s, q = ref.gen_quant4(k, n, g)
    assert w0.shape == (k, n) and s.shape == (k // g, n) and q.shape == (k, n)
    assert linear.weight.shape == (n, k)
    assert int(q.min()) >= -8 and int(q.max()) <= 8  # the clamp is [0, 16] before the -8 shift
    s_full = s.repeat_interleave(g, dim=0)
    assert torch.equal(linear.weight.data.t(), q.half() * s_full)
    # s = max|w| / 8 per (group, column)
    want_s = w0.reshape(k // g, g, n).abs().amax(dim=1) * (2 / 16)
    assert torch.equal(s, want_s)
    # round(w / s) + 8 with ties to even, before clamping
    want_q = torch.clamp(torch.round(w0 / s_full).int() + 8, 0, 16) - 8
    assert torch.equal(q, want_q)
    torch.manual_seed(0)
    again = ref.gen_quant4(k, n, g)
    assert torch.equal(again[0], w0) and torch.equal(again[3], q)
    torch.manual_seed(0)
    whole = ref.gen_quant4(k, n)  # groupsize=-1: one group over all of K
    assert whole[2].shape == (1, n)


# ------------------------------------------------------------------------------------------------
# per-group dequantisation
# ------------------------------------------------------------------------------------------------
def _bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("dtype,kind", [(torch.float16, 0), (torch.bfloat16, 1)])
def test_dequant_matches_float64_with_explicit_rounding_and_c(dtype, kind):
    N, K, g = 12, 128, 32
    gen = _rng(9)
    wp = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=gen)
    s = (torch.rand(N, K // g, generator=gen) * 0.015 + 0.005).to(dtype)
    z = torch.randint(0, 16, (N, K // g), generator=gen).to(dtype)
    got = ref.dequant_w4(wp, s, z, g, dtype)
    # float64 route: u - z is exact for small integers, so only the product rounds
    u = ref.unpack_uint4(wp).astype(np.float64)
    zf = z.double().numpy().repeat(g, axis=1)
    sf = s.double().numpy().repeat(g, axis=1)
    want = torch.from_numpy((u - zf) * sf).to(dtype)  # one correctly rounded conversion
    assert torch.equal(got, want)
    c = cref.dequant_w4(wp.numpy(), _bits(s), _bits(z), 0.0, g, kind)
    assert np.array_equal(c, _bits(got))
    # scalar zero point and absent scale / zero
    got8 = ref.dequant_w4(wp, s, 8, g, dtype)
    assert torch.equal(got8, torch.from_numpy((u - 8.0) * sf).to(dtype))
    assert np.array_equal(cref.dequant_w4(wp.numpy(), _bits(s), None, 8.0, g, kind), _bits(got8))
    plain = ref.dequant_w4(wp, None, None, g, dtype)
    assert torch.equal(plain, torch.from_numpy(u).to(dtype))


def test_dequant_fractional_zero_rounds_twice():
    # a non-integer zero point makes (u - z) inexact in fp16: the difference is rounded, then the product
    wp = torch.tensor([[0xF0]], dtype=torch.uint8)
    s = torch.tensor([[0.3333]], dtype=torch.float16)
    z = torch.tensor([[0.0999]], dtype=torch.float16)
    got = ref.dequant_w4(wp, s, z, 2, torch.float16)
    d = (np.float16(15) - z.numpy()[0, 0]).astype(np.float16)
    assert got[0, 1].item() == float((d * s.numpy()[0, 0]).astype(np.float16))
    c = cref.dequant_w4(wp.numpy(), _bits(s), _bits(z), 0.0, 2, 0)
    assert np.array_equal(c, _bits(got))


# ------------------------------------------------------------------------------------------------
# floating-point GEMM oracles
# ------------------------------------------------------------------------------------------------
def test_ref_program_fp16_literal_loop_and_identity_rows():
    M = N = K = 32
    gen = _rng(10)
    A = torch.randn(M, K, generator=gen).half()
    wp = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=gen)
    for out in ("float16", "bfloat16", "float32"):
        assert torch.equal(ref.ref_program_fp16(A, wp, out), ref.ref_program_fp16_loop(A, wp, out))
    # one-hot activations select weight columns: C[m, n] = W[n, m]
    eye = torch.eye(K, dtype=torch.float16)
    s = (torch.rand(N, 1, generator=gen) * 0.015 + 0.005).half()
    z = torch.randint(6, 10, (N, 1), generator=gen).half()
    W = ref.dequant_w4(wp, s, z, K, torch.float16)
    assert torch.equal(ref.ref_program_w4a16(eye, wp, s, z, K, "float16"), W.T)
    # no scales / zeros: the plain example
    assert torch.equal(ref.ref_program_w4a16(A, wp, None, None, K, "float16"), ref.ref_program_fp16(A, wp, "float16"))


@pytest.mark.parametrize("dtype,kind", [(torch.float16, 0), (torch.bfloat16, 1)])
def test_w4a16_oracle_against_c_restatement(dtype, kind):
    M, N, K, g = 5, 24, 96, 32
    gen = _rng(11)
    A = torch.randn(M, K, generator=gen).to(dtype)
    wp = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=gen)
    s = (torch.rand(N, K // g, generator=gen) * 0.015 + 0.005).to(dtype)
    z = torch.randint(6, 10, (N, K // g), generator=gen).to(dtype)
    W = ref.dequant_w4(wp, s, z, g, dtype)
    want32 = ref.ref_program_w4a16(A, wp, s, z, g, "float32").numpy()
    got32 = cref.gemm_w4a16(_bits(A), _bits(W), kind, 2)  # C accumulates in double
    np.testing.assert_allclose(got32, want32, rtol=2e-6, atol=1e-6)
    # exact rational check of one entry with Python fractions
    from fractions import Fraction

    acc = sum(Fraction(float(A[1, k])) * Fraction(float(W[3, k])) for k in range(K))
    assert abs(float(acc) - float(want32[1, 3])) <= 2e-6 * abs(float(acc)) + 1e-6


# ------------------------------------------------------------------------------------------------
# integer GEMM oracles
# ------------------------------------------------------------------------------------------------
def test_int_matmul_exact_brute_force_and_extremes():
    gen = _rng(12)
    A = torch.randint(-128, 128, (3, 17), dtype=torch.int8, generator=gen)
    B = torch.randint(-128, 128, (17, 5), dtype=torch.int8, generator=gen)
    want = [[sum(int(A[m, k]) * int(B[k, n]) for k in range(17)) for n in range(5)] for m in range(3)]
    assert ref.int_matmul_exact(A, B).tolist() == want
    assert cref.gemm_i8(A.numpy(), B.numpy(), 0).tolist() == want
    assert cref.gemm_i8(A.numpy(), B.T.contiguous().numpy(), 1).tolist() == want
    # closed form: all -128, K = 4096 -> 4096 * 16384 = 67 108 864
    K = 4096
    a = torch.full((2, K), -128, dtype=torch.int8)
    b = torch.full((K, 3), -128, dtype=torch.int8)
    assert ref.int_matmul_exact(a, b).tolist() == [[67108864] * 3] * 2
    assert cref.gemm_i8(a.numpy(), b.numpy(), 0).tolist() == [[67108864] * 3] * 2
    # torch's own int32 matmul (the reference's literal route) agrees
    big_a = torch.randint(-128, 128, (4, 512), dtype=torch.int8, generator=gen)
    big_b = torch.randint(-128, 128, (512, 6), dtype=torch.int8, generator=gen)
    assert torch.equal(ref.int_matmul_exact(big_a, big_b).int(), big_a.int() @ big_b.int())


def test_ref_program_int8_and_w4a8_shapes_and_values():
    gen = _rng(13)
    A = torch.randint(-128, 128, (4, 64), dtype=torch.int8, generator=gen)
    wp = torch.randint(0, 256, (6, 32), dtype=torch.uint8, generator=gen)
    u = ref.unpack_uint4(wp).astype(np.int64)
    want = A.numpy().astype(np.int64) @ u.T
    got = ref.ref_program_int8(A, wp, "int32")
    assert got.dtype == torch.int32 and np.array_equal(got.numpy(), want)
    assert ref.ref_program_int8(A, wp, "float16").dtype == torch.float16
    s4 = np.where(u >= 8, u - 16, u)
    t = ref.ref_program_w4a8(A, wp)
    assert t.shape == (6, 4) and t.dtype == torch.int32  # transposed [N, M]
    assert np.array_equal(t.numpy(), (A.numpy().astype(np.int64) @ s4.T).T)


def test_rescale_epilogues():
    gen = _rng(14)
    B_, M, N, K = 2, 5, 7, 64
    A = torch.randint(-127, 128, (B_, M, K), dtype=torch.int8, generator=gen)
    W = torch.randint(-127, 128, (B_, K, N), dtype=torch.int8, generator=gen)
    acc = ref.int_matmul_exact(A, W)
    for scale in (torch.tensor([0.0123]), torch.rand(N, generator=gen) * 0.009 + 0.001):
        for out in (torch.float16, torch.bfloat16, torch.float32):
            got = ref.ref_program_quant(A, W, scale, out)
            lit = ref.ref_program_quant(A, W, scale, out, literal=True)
            assert torch.equal(got, lit)
            f32 = (acc.numpy().astype(np.float32) * scale.numpy().astype(np.float32)).astype(np.float32)
            assert torch.equal(got, torch.from_numpy(f32).to(out))
            for b in range(B_):
                sb = scale.numpy()
                c = cref.rescale(acc[b].int().numpy(), None, sb, {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}[out])
                g = got[b]
                assert np.array_equal(c, g.numpy() if out == torch.float32 else _bits(g))
    # per-token x per-channel: kernel order (two fp32 multiplies) vs the outer-product golden
    sa = torch.rand(B_, M, generator=gen) * 0.04 + 0.01
    sb = torch.rand(N, generator=gen) * 0.009 + 0.001
    Wnk = W.transpose(1, 2).contiguous()
    seq = ref.ref_int8_gemm_sequential(A, Wnk[0], sa, sb, torch.float32)
    manual = (acc[0].numpy().astype(np.float32) * sa[0].numpy()[:, None]).astype(np.float32) * sb.numpy()[None, :]
    assert np.array_equal(seq[0].numpy(), manual.astype(np.float32))
    gold = ref.int8_gemm_torch_optimized(A[0], sa[0], Wnk[0], sb)
    torch.testing.assert_close(seq[0], gold, rtol=1e-5, atol=1e-5)
    c = cref.rescale(acc[0].int().numpy(), sa[0].numpy(), sb.numpy(), 2)
    assert np.array_equal(c, seq[0].numpy())


# ------------------------------------------------------------------------------------------------
# committed fixtures: inputs and outputs frozen from the two oracles (tests/golden/make_golden.py)
# ------------------------------------------------------------------------------------------------
def test_golden_fixtures_still_match_the_oracle():
    import importlib.util

    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(GOLDEN, "make_golden.py"))
    make_golden = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(make_golden)

    with np.load(os.path.join(GOLDEN, "w4a16_small.npz")) as f:
        fresh = make_golden.w4a16_cases()
        assert set(f.files) == set(fresh)
        for k in f.files:
            assert np.array_equal(f[k], fresh[k]), k
    with np.load(os.path.join(GOLDEN, "int8_small.npz")) as f:
        fresh = make_golden.int8_cases()
        assert set(f.files) == set(fresh)
        for k in f.files:
            assert np.array_equal(f[k], fresh[k]), k


# ---- the 2-bit / 1-bit lop3 decoders: every source value against closed forms that index the fields arithmetically ----
F16_ORDER = (0, 4, 1, 5, 2, 6, 3, 7)


def _fields(values, bits, count):
    """field j of every value, by division (not by the shifts the oracle uses)"""
    v = np.asarray(values, dtype=np.int64)
    return np.stack([(v // (2 ** (bits * j))) % (2 ** bits) for j in range(count)], axis=1)


def _rn16(x):
    return np.asarray(x, dtype=np.float64).astype(np.float16)


@pytest.mark.parametrize("bits", [2, 1])
def test_lowbit_lop3_decoders_to_fp16_on_every_source(bits):
    src = np.arange(2 ** (8 * bits), dtype=np.uint16 if bits == 2 else np.uint8)
    u = _fields(src, bits, 8)[:, F16_ORDER].astype(np.float64)
    assert np.array_equal(ref.lop3_decode_lowbit_to_f16(src, bits), _rn16(u))
    signed = u - 2 if bits == 2 else 2 * u - 1
    assert np.array_equal(ref.lop3_decode_lowbit_to_f16(src, bits, signed=True), _rn16(signed))
    s, z = np.float16(0.0371), np.float16(1.3125)
    assert np.array_equal(ref.lop3_decode_lowbit_to_f16(src, bits, scale=s), _rn16(u * float(s)))
    assert np.array_equal(ref.lop3_decode_lowbit_to_f16(src, bits, signed=True, scale=s), _rn16(signed * float(s)))
    orig = _rn16(_rn16(u - float(z)).astype(np.float64) * float(s))
    assert np.array_equal(ref.lop3_decode_lowbit_to_f16(src, bits, scale=s, zeros=z, zeros_mode="original"), orig)
    got = ref.lop3_decode_lowbit_to_f16(src, bits, scale=s, zeros=z, zeros_mode="rescale")
    if bits == 2:  # the product is rounded, then the zero point subtracted (lop3.py:626-627)
        assert np.array_equal(got, _rn16(_rn16(u * float(s)).astype(np.float64) - float(z)))
        s2, z2 = np.float16(0.74658203125), np.float16(1.287109375)  # constants that tell two roundings from one (at u = 3)
        got2 = ref.lop3_decode_lowbit_to_f16(src, bits, scale=s2, zeros=z2, zeros_mode="rescale")
        assert np.array_equal(got2, _rn16(_rn16(u * float(s2)).astype(np.float64) - float(z2)))
        assert not np.array_equal(got2, _rn16(u * float(s2) - float(z2)))
        qz = 3
        assert np.array_equal(ref.lop3_decode_lowbit_to_f16(src, bits, scale=s, zeros=qz, zeros_mode="quantized"), _rn16((u - qz) * float(s)))
    else:          # one multiply-add whose addend has its sign bit forced (lop3.py:870,880): -|z| for either sign of z
        assert np.array_equal(got, _rn16(u * float(s) - float(z)))
        assert np.array_equal(ref.lop3_decode_lowbit_to_f16(src, bits, scale=s, zeros=-z, zeros_mode="rescale"), got)
        s2, z2 = np.float16(0.74658203125), np.float16(1.287109375)
        assert np.array_equal(ref.lop3_decode_lowbit_to_f16(src, bits, scale=s2, zeros=z2, zeros_mode="rescale"), _rn16(u * float(s2) - float(z2)))


def test_lowbit_lop3_decoders_to_int8_and_int4():
    rng = np.random.default_rng(5)
    w32 = np.concatenate([rng.integers(0, 2 ** 32, 4096, dtype=np.uint64).astype(np.uint32), np.array([0, 0xFFFFFFFF, 0x1B1B1B1B], dtype=np.uint32)])
    f = _fields(w32, 2, 16)
    want = np.stack([f[:, 4 * b + i] for i in range(4) for b in range(4)], axis=1)  # word i, byte lane b holds field 4 b + i
    assert np.array_equal(ref.lop3_decode_lowbit_to_i8(w32, 2), want.astype(np.int8))
    assert np.array_equal(ref.lop3_decode_lowbit_to_i8(w32, 2, signed=True), (want - 2).astype(np.int8))
    w16 = np.arange(65536, dtype=np.uint16)
    b = _fields(w16, 1, 16)
    lanes = lambda i: (i, 8 + i, 4 + i, 12 + i)  # noqa: E731
    want1 = np.stack([b[:, j] for i in range(4) for j in lanes(i)], axis=1)
    assert np.array_equal(ref.lop3_decode_lowbit_to_i8(w16, 1), want1.astype(np.int8))
    assert np.array_equal(ref.lop3_decode_lowbit_to_i8(w16, 1, signed=True), (2 * want1 - 1).astype(np.int8))
    # 2-bit -> nibbles: nibble n of output word i holds field 2 n + i
    got = ref.lop3_decode_i2_to_i4(w32)
    nib = np.stack([_fields(got[:, i], 4, 8) for i in range(2)], axis=1)  # [n, word, nibble]
    assert np.array_equal(nib, np.stack([f[:, [2 * n + i for n in range(8)]] for i in range(2)], axis=1))


def test_lowbit_int8_decoder_undoes_the_reference_interleave():
    """interleave_weight(q, 2, "int8") (tilelang/quantize/utils.py:73-101, the one low-bit branch the reference can run) puts
    field 4 i + b of a word at byte lane b, slot i: decode_i2u_to_i8s of the result is the plain unpack in logical order."""
    q = torch.randint(-128, 128, (6, 16), dtype=torch.int8, generator=_rng(21))
    inter = ref.interleave_weight(q, 2, "int8")
    words = inter.contiguous().view(torch.int32).numpy().view(np.uint32).reshape(-1)
    plain = _fields(q.contiguous().view(torch.int32).numpy().view(np.uint32).reshape(-1), 2, 16)
    assert np.array_equal(ref.lop3_decode_lowbit_to_i8(words, 2), plain.astype(np.int8))
