"""tilelang_ascend_amd.quantize (product code, torch) against the oracle and closed forms.
The CPU cases run here; the GPU cases decode interleaved weights with the HIP fast decoders."""
import numpy as np
import pytest
import torch

from helpers import assert_bit_equal
from oracle import ref
from tilelang_ascend_amd import quantize as Q


def _rng(seed):
    return torch.Generator().manual_seed(seed)


def test_import_surface():
    for name in ("_tir_packed_int_to_int_convert", "_tir_packed_to_signed_convert", "_tir_packed_to_unsigned_convert",
                 "_tir_packed_to_fp4_to_f16", "_tir_u8_to_f8_e4m3_to_f16", "_tir_packed_to_unsigned_convert_with_zeros",
                 "gen_quant4", "general_compress", "interleave_weight", "get_lop3_intrin_group"):
        assert hasattr(Q, name), name


def test_element_converters_against_oracle_tables():
    val = torch.randint(0, 256, (5, 7), dtype=torch.uint8, generator=_rng(1))
    for pos in (0, 1):
        u = Q._tir_packed_to_unsigned_convert("uint", 8)(4, val, pos, "float16")
        assert u.dtype == torch.float16
        assert np.array_equal(u.numpy().astype(np.int64), ref.packed_to_unsigned(val.numpy(), pos))
        s = Q._tir_packed_to_signed_convert("uint", 8)(4, val, pos, "int8")
        assert np.array_equal(s.numpy().astype(np.int64), ref.packed_to_signed_offset(val.numpy(), pos))
        t = Q._tir_packed_int_to_int_convert("uint", 8)(4, val, pos, "int8")
        assert np.array_equal(t.numpy().astype(np.int64), ref.packed_int_to_int(val.numpy(), pos))
        f = Q._tir_packed_uint_to_uint_to_float(8)(4, val, pos, "float16")
        assert np.array_equal(f.numpy().astype(np.int64), ref.packed_uint_to_uint_to_float(val.numpy(), pos))
        z = Q._tir_packed_to_unsigned_convert_with_zeros("uint", 8)(4, val, pos, 9, "float16")
        assert np.array_equal(z.numpy().astype(np.int64), ref.packed_to_unsigned_with_zeros(val.numpy(), pos, 9))
        zf = Q._tir_packed_to_unsigned_convert_with_zeros("uint", 8)(4, val, pos, torch.tensor(7.5, dtype=torch.float16),
                                                                    "float16")
        assert torch.equal(zf, u - torch.tensor(7.5, dtype=torch.float16))
    # int8 storage: the same bytes viewed as signed
    sv = val.view(torch.int8)
    assert torch.equal(Q._tir_packed_to_unsigned_convert("int", 8)(4, sv, 1, "int8"),
                       Q._tir_packed_to_unsigned_convert("uint", 8)(4, val, 1, "int8"))
    # per-element positions: unpack a whole row at once
    packed = torch.tensor([[0x12, 0x34]], dtype=torch.uint8)
    k = torch.arange(4)
    got = Q._tir_packed_to_unsigned_convert("uint", 8)(4, packed[:, k // 2], k % 2, "int8")
    assert got.tolist() == [[2, 1, 4, 3]]
    with pytest.raises(AssertionError):
        Q._tir_packed_to_unsigned_convert("uint", 8)(4, val.to(torch.int32), 0, "int8")


def test_fp4_and_e4m3_closed_forms():
    codes = torch.arange(16, dtype=torch.uint8)
    got = Q._tir_packed_to_fp4_to_f16("uint", 8)(4, codes, 0, "float16")
    want = [0.0 if (c & 7) == 0 else (-1.0 if c >> 3 else 1.0) * 2.0 ** ((c & 7) - 7) for c in range(16)]
    assert got.tolist() == want
    # e4m3: every normal finite code must equal torch's own float8_e4m3fn conversion
    allc = torch.arange(256, dtype=torch.uint8)
    mine = Q._tir_u8_to_f8_e4m3_to_f16(8, allc, "float16")
    theirs = allc.view(torch.float8_e4m3fn).to(torch.float16)
    normal = ((allc & 0x78) != 0) & ((allc & 0x7F) != 0x7F)
    assert torch.equal(mine[normal], theirs[normal])


def test_general_compress_and_interleave_match_oracle():
    for bits in (4, 2, 1):
        w = torch.randint(0, 1 << bits, (6, 64), dtype=torch.int8, generator=_rng(2))
        assert torch.equal(Q.general_compress(w, bits, torch.int8), ref.general_compress(w, bits, torch.int8))
    w = torch.randint(-8, 8, (3, 16), dtype=torch.int8, generator=_rng(3))  # unmasked negatives: same smear
    assert torch.equal(Q.general_compress(w, 4, torch.int8), ref.general_compress(w, 4, torch.int8))
    assert Q.general_compress(w.half(), 4, torch.int32).dtype == torch.int32
    q = torch.randint(-128, 128, (5, 32), dtype=torch.int8, generator=_rng(4))
    for nbits, target in ((4, "float16"), (4, "int8"), (2, "int8")):
        assert torch.equal(Q.interleave_weight(q, nbits, target), ref.interleave_weight(q, nbits, target)), (nbits, target)
    # the reference's 1-bit and 2-bit/float16 branches call torch.int32(...) (utils.py:103-124): a TypeError there and here
    for nbits, target in ((1, "int8"), (1, "float16"), (2, "float16")):
        for fn in (Q.interleave_weight, ref.interleave_weight):
            with pytest.raises(TypeError, match="not callable"):
                fn(q, nbits, target)
    base = torch.tensor([[0x10, 0x32, 0x54, 0x76]], dtype=torch.uint8).view(torch.int8)
    assert ref.unpack_uint4(Q.interleave_weight(base, 4, "float16")).tolist() == [[0, 2, 4, 6, 1, 3, 5, 7]]
    assert ref.unpack_uint4(Q.interleave_weight(base, 4, "int8")).tolist() == [[0, 4, 1, 5, 2, 6, 3, 7]]


def test_gen_quant4_same_stream_and_values_as_oracle():
    for g in (64, -1):
        torch.manual_seed(5)
        a = Q.gen_quant4(256, 24, g)
        torch.manual_seed(5)
        b = ref.gen_quant4(256, 24, g)
        assert torch.equal(a[0], b[0]) and torch.equal(a[2], b[2]) and torch.equal(a[3], b[3])
        assert torch.equal(a[1].weight.data, b[1].weight.data)


def test_lop3_group_naming_grammar():
    g = Q.get_lop3_intrin_group("float16")
    assert g["func_name"] == "decode_i4u_to_f16" and "decode_i4u_to_f16(" in g["c_source"]
    assert Q.get_lop3_intrin_group("float16", source_format="int")["func_name"] == "decode_i4s_to_f16"
    assert Q.get_lop3_intrin_group("float16", with_scaling=True)["func_name"] == "decode_i4u_to_f16_scale"
    for mode in ("original", "rescale", "quantized"):
        name = Q.get_lop3_intrin_group("float16", with_scaling=True, with_zeros=True, zeros_mode=mode)["func_name"]
        assert name == f"decode_i4u_to_f16_scale_zeros_{mode}"
    assert Q.get_lop3_intrin_group("int8", source_format="int")["func_name"] == "decode_i4s_to_i8s"
    assert Q.get_lop3_intrin_group("int8")["func_name"] == "decode_i4u_to_i8s"
    with pytest.raises(ValueError):
        Q.get_lop3_intrin_group("float16", source_format="int", with_scaling=True, with_zeros=True)
    with pytest.raises(ValueError):
        Q.get_lop3_intrin_group("float16", source_format="float")
    with pytest.raises(AssertionError):
        Q.get_lop3_intrin_group("float32")
    # 2-bit and 1-bit sources: the names of the reference's table (lop3.py:1147-1170), KeyError for what it does not hold
    for kw, name in ((dict(source_bit=2), "decode_i2u_to_f16"), (dict(source_bit=2, source_format="int", with_scaling=True), "decode_i2s_to_f16_scale"),
                     (dict(source_bit=2, with_scaling=True, with_zeros=True, zeros_mode="quantized"), "decode_i2u_to_f16_scale_zeros_quantized"),
                     (dict(source_bit=2, with_scaling=True, with_zeros=True, zeros_mode="rescale"), "decode_i2u_to_f16_scale_zeros_rescale"),
                     (dict(source_bit=1, source_format="int"), "decode_i1s_to_f16"), (dict(source_bit=1, with_scaling=True), "decode_i1u_to_f16_scale"),
                     (dict(source_bit=1, with_scaling=True, with_zeros=True, zeros_mode="original"), "decode_i1u_to_f16_scale_zeros_original")):
        g = Q.get_lop3_intrin_group("float16", **kw)
        assert g["func_name"] == name and f" {name}(" in g["c_source"]
    assert Q.get_lop3_intrin_group("int8", source_bit=2, source_format="int")["func_name"] == "decode_i2s_to_i8s"
    assert Q.get_lop3_intrin_group("int8", source_bit=1)["func_name"] == "decode_i1u_to_i8s"
    for bad in (dict(out_dtype="float16", source_bit=1, with_scaling=True, with_zeros=True, zeros_mode="quantized"),
                dict(out_dtype="float16", source_bit=2, with_scaling=True, storage_scope="warp"),
                dict(out_dtype="int4", source_bit=1), dict(out_dtype="int8", source_bit=2, with_scaling=True),
                dict(out_dtype="float16", source_bit=3)):
        with pytest.raises(KeyError):
            Q.get_lop3_intrin_group(**bad)
    # storage_scope "warp" with scaling selects the two-group forms (lop3.py:1178-1180, 1196-1197)
    for kw, name in ((dict(), "decode_i4u_to_f16_scale_offset"),
                     (dict(source_format="int"), "decode_i4s_to_f16_scale_offset"),
                     (dict(with_zeros=True, zeros_mode="original"), "decode_i4u_to_f16_scale_zeros_original_offset"),
                     (dict(with_zeros=True, zeros_mode="rescale"), "decode_i4u_to_f16_scale_zeros_rescale_offset"),
                     (dict(with_zeros=True, zeros_mode="quantized"), "decode_i4u_to_f16_scale_zeros_quantized_offset")):
        g = Q.get_lop3_intrin_group("float16", with_scaling=True, storage_scope="warp", **kw)
        assert g["func_name"] == name and f" {name}(" in g["c_source"]
    assert Q.get_lop3_intrin_group("float16", storage_scope="warp")["func_name"] == "decode_i4u_to_f16"  # no scaling: no suffix
    assert Q.get_lop3_intrin_group("int4", source_bit=2, source_format="int")["func_name"] == "decode_i2s_to_i4s"
    with pytest.raises(KeyError):
        Q.get_lop3_intrin_group("int4")  # (4-bit sources have no 4-bit target)


# ------------------------------------------------------------------------------------------------
# GPU: the HIP fast decoders on interleaved weights
# ------------------------------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("signed", [False, True])
def test_gpu_decode_plain_and_signed(signed):
    from tilelang_ascend_amd.quantize import lop3

    q = torch.randint(0, 256, (64, 96), dtype=torch.uint8, generator=_rng(10))
    inter = Q.interleave_weight(q.view(torch.int8), 4, "float16").cuda()
    got = lop3.decode(inter, "float16", "int" if signed else "uint").cpu()
    want = ref.unpack_uint4(q).astype(np.float16) - (np.float16(8) if signed else np.float16(0))
    assert got.dtype == torch.float16 and np.array_equal(got.numpy(), want)
    inter8 = Q.interleave_weight(q.view(torch.int8), 4, "int8").cuda()
    got8 = lop3.decode(inter8, "int8", "int" if signed else "uint").cpu()
    want8 = ref.unpack_uint4(q).astype(np.int8) - (7 if signed else 0)
    assert got8.dtype == torch.int8 and np.array_equal(got8.numpy(), want8)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", [None, "original", "rescale", "quantized"])
def test_gpu_decode_scale_and_zeros(mode):
    from tilelang_ascend_amd.quantize import lop3

    N, K, g = 48, 256, 64
    gen = _rng(11)
    q = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=gen)
    s = (torch.rand(N, K // g, generator=gen) * 0.015 + 0.005).half()
    zf = (torch.rand(N, K // g, generator=gen) * 3 + 6).half()
    zi = torch.randint(0, 16, (N, K // g), generator=gen)
    inter = Q.interleave_weight(q.view(torch.int8), 4, "float16").cuda()
    zeros = None if mode is None else (zi if mode == "quantized" else zf)
    got = lop3.decode(inter, "float16", "uint", scale=s.cuda(), zeros=None if zeros is None else zeros.cuda(),
                      zeros_mode=mode, group_size=g).cpu()
    u = torch.from_numpy(ref.unpack_uint4(q).astype(np.float32)).half()
    sx = s.repeat_interleave(g, dim=1)
    if mode is None:
        want = u * sx
    elif mode == "original":
        want = (u - zf.repeat_interleave(g, dim=1)) * sx
    elif mode == "quantized":
        want = (u - zi.half().repeat_interleave(g, dim=1)) * sx
    else:  # one rounding
        want = (u.double() * sx.double() - zf.repeat_interleave(g, dim=1).double()).half()
    assert torch.equal(got, want)
    # the word-level closed form of the oracle gives the same numbers for a single group
    words = inter.cpu().contiguous().view(torch.int32).numpy().view(np.uint32).reshape(-1)[: g // 8]
    if mode in ("original", "rescale"):
        o = ref.lop3_decode_i4_to_f16(words, scale=float(s[0, 0]), zeros=float(zf[0, 0]), zeros_mode=mode)
        assert np.array_equal(o.reshape(-1), got[0, :g].numpy())


@pytest.mark.gpu
def test_gpu_quantize_utils_run_on_device_tensors():
    w = torch.randint(0, 16, (32, 128), dtype=torch.int8, generator=_rng(12))
    packed = Q.general_compress(w.cuda(), 4, torch.int8)
    assert packed.is_cuda and torch.equal(packed.cpu(), ref.general_compress(w, 4, torch.int8))
    inter = Q.interleave_weight(packed, 4, "float16")
    assert inter.is_cuda and torch.equal(inter.cpu(), ref.interleave_weight(packed.cpu(), 4, "float16"))


@pytest.mark.gpu
@pytest.mark.parametrize("mode", [None, "original", "rescale", "quantized"])
@pytest.mark.parametrize("offset", [0, 1, 5])
def test_gpu_decode_offset_forms(mode, offset):
    """The two-group decoders on the GPU against the oracle's word-level closed form, word by word: the first four
    weights of a word use group g, the last four group g + offset (zero points: field group_offset of the packed words
    g and g + zero_offset for the quantized mode)."""
    from tilelang_ascend_amd.quantize import lop3

    g_size, groups = 32, 12
    wpg = g_size // 8
    gen = _rng(21 + offset)
    q = torch.randint(0, 256, (groups * g_size // 2,), dtype=torch.uint8, generator=gen).reshape(1, -1)
    s = (torch.rand(groups + offset, generator=gen) * 0.015 + 0.005).half()
    zf = (torch.rand(groups + offset, generator=gen) * 3 + 6).half()
    zero_offset, group_offset = 2, 3
    qz_fields = torch.randint(0, 16, (groups + zero_offset, 8), generator=gen)
    qz_words = sum(qz_fields[:, j].to(torch.int64) << (4 * j) for j in range(8))
    qz_words = torch.where(qz_words >= (1 << 31), qz_words - (1 << 32), qz_words).to(torch.int32)
    inter = Q.interleave_weight(q.view(torch.int8), 4, "float16")
    zeros = None if mode is None else (qz_words if mode == "quantized" else zf)
    for signed in ((False, True) if mode is None else (False,)):
        got = lop3.decode_offset(inter.cuda(), s.cuda(), offset, "int" if signed else "uint",
                                 zeros=None if zeros is None else zeros.cuda(), zeros_mode=mode, group_size=g_size,
                                 zero_offset=zero_offset, group_offset=group_offset).cpu().numpy().reshape(-1, 8)
        words = inter.contiguous().view(torch.int32).numpy().view(np.uint32).reshape(-1)
        for i, word in enumerate(words):
            grp = i // wpg
            kw = {}
            if mode == "quantized":
                kw = dict(zeros=int(qz_fields[grp, group_offset]), zeros_r=int(qz_fields[grp + zero_offset, group_offset]), zeros_mode=mode)
            elif mode is not None:
                kw = dict(zeros=float(zf[grp]), zeros_r=float(zf[grp + offset]), zeros_mode=mode)
            want = ref.lop3_decode_i4_to_f16([word], signed=signed, scale=float(s[grp]), scale_r=float(s[grp + offset]), **kw)
            assert np.array_equal(got[i], want[0]), (mode, offset, signed, i)


@pytest.mark.gpu
def test_gpu_decode_offset_rejects_short_parameter_arrays():
    from tilelang_ascend_amd.quantize import lop3

    w = torch.zeros(1, 64, dtype=torch.uint8, device="cuda")  # 16 words = 4 groups of 32 weights
    s = torch.ones(4, dtype=torch.float16, device="cuda")
    assert lop3.decode_offset(w, s, 0, group_size=32).shape == (1, 128)
    with pytest.raises(RuntimeError, match="need 5 scales"):
        lop3.decode_offset(w, s, 1, group_size=32)
    with pytest.raises(RuntimeError, match="zeros"):
        lop3.decode_offset(w, torch.ones(5, dtype=torch.float16), 1, zeros=s, zeros_mode="original", group_size=32)
    with pytest.raises(RuntimeError, match="group_offset"):
        lop3.decode_offset(w, s, 0, zeros=torch.zeros(4, dtype=torch.int32), zeros_mode="quantized", group_size=32, group_offset=8)


# ------------------------------------------------------------------------------------------------
# 2-bit / 1-bit fast decoders on the GPU (csrc/decode_lowbit.h through tlq_decode_lowbit_interleaved) against the oracle's
# step-by-step restatement of lop3.py:423-996, 1048-1087, on every source value
# ------------------------------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("bits", [2, 1])
def test_gpu_lowbit_decoders_to_fp16_on_every_source(bits):
    from tilelang_ascend_amd.quantize import lop3

    n = 2 ** (8 * bits)
    src_np = np.arange(n, dtype=np.uint16 if bits == 2 else np.uint8)
    src = torch.from_numpy(src_np.view(np.uint8).copy()).cuda()
    s, z = 0.0371, 1.3125
    cases = [dict(), dict(signed=True), dict(scale=s), dict(signed=True, scale=s), dict(scale=s, zeros=z, zeros_mode="original"),
             dict(scale=s, zeros=z, zeros_mode="rescale"), dict(scale=s, zeros=-z, zeros_mode="rescale"),
             dict(scale=0.74658203125, zeros=1.287109375, zeros_mode="rescale")]  # (the last: one rounding and two differ at u = 3)
    if bits == 2:
        cases.append(dict(scale=s, zeros=3, zeros_mode="quantized"))
    for kw in cases:
        want = ref.lop3_decode_lowbit_to_f16(src_np, bits, **kw)
        sc = None if "scale" not in kw else torch.tensor([kw["scale"]], dtype=torch.float16)
        zs = None if "zeros" not in kw else torch.tensor([kw["zeros"]], dtype=torch.int16 if kw["zeros_mode"] == "quantized" else torch.float16)
        got = lop3.decode_lowbit(src, bits, "float16", "int" if kw.get("signed") else "uint", scale=sc, zeros=zs, zeros_mode=kw.get("zeros_mode"))
        assert got.shape == (n * 8,) and got.dtype == torch.float16
        assert_bit_equal(got.cpu().view(n, 8), torch.from_numpy(want), f"{bits}-bit {kw}")
    # one scale / zero per group of 16 weights (two units)
    sg = (torch.arange(n // 2, dtype=torch.float32) % 37 * 0.01 + 0.02).half()
    zg = (torch.arange(n // 2, dtype=torch.float32) % 5 * 0.25).half()
    got = lop3.decode_lowbit(src, bits, "float16", scale=sg, zeros=zg, zeros_mode="original", group_size=16).cpu().view(n, 8)
    for g in (0, 1, 77, n // 2 - 1):
        want = ref.lop3_decode_lowbit_to_f16(src_np[2 * g:2 * g + 2], bits, scale=sg[g].item(), zeros=zg[g].item(), zeros_mode="original")
        assert_bit_equal(got[2 * g:2 * g + 2], torch.from_numpy(want), f"group {g}")


@pytest.mark.gpu
def test_gpu_lowbit_decoders_to_int8_and_int4():
    from tilelang_ascend_amd import _abi
    from tilelang_ascend_amd.quantize import lop3

    rng = np.random.default_rng(9)
    w32 = np.concatenate([rng.integers(0, 2 ** 32, 5000, dtype=np.uint64).astype(np.uint32), np.array([0, 0xFFFFFFFF, 0x1B1B1B1B], dtype=np.uint32)])
    src32 = torch.from_numpy(w32.view(np.uint8).copy()).cuda()
    w16 = np.arange(65536, dtype=np.uint16)
    src16 = torch.from_numpy(w16.view(np.uint8).copy()).cuda()
    for signed in (False, True):
        fmt = "int" if signed else "uint"
        got = lop3.decode_lowbit(src32, 2, "int8", fmt).cpu().view(-1, 16)
        assert_bit_equal(got, torch.from_numpy(ref.lop3_decode_lowbit_to_i8(w32, 2, signed)), f"2-bit -> int8 {fmt}")
        got = lop3.decode_lowbit(src16, 1, "int8", fmt).cpu().view(-1, 16)
        assert_bit_equal(got, torch.from_numpy(ref.lop3_decode_lowbit_to_i8(w16, 1, signed)), f"1-bit -> int8 {fmt}")
        got = lop3.decode_lowbit(src32, 2, "int4", fmt).cpu().numpy().view(np.uint32).reshape(-1, 2)
        assert np.array_equal(got, ref.lop3_decode_i2_to_i4(w32)), f"2-bit -> int4 {fmt}"
    # empty input, and what the entry point refuses
    assert lop3.decode_lowbit(src32[:0], 2, "int8").numel() == 0
    lib, P = _abi.load(), _abi.ptr
    out = torch.empty(64, dtype=torch.uint8, device="cuda")
    one = torch.ones(1, dtype=torch.float16, device="cuda")
    for args, word in (((P(src32), None, None, P(out), 1, 1, 3, 16, 0, 0), "source_bit"), ((P(src32), None, None, P(out), 1, 1, 1, 4, 0, 0), "2-bit sources only"),
                       ((P(src32), P(one), P(one), P(out), 1, 1, 1, 16, 0, 3), "quantized"), ((P(src32), P(one), P(one), P(out), 1, 1, 2, 16, 1, 1), "signed"),
                       ((P(src32), P(one), None, P(out), 1, 1, 2, 8, 0, 0), "integer targets"), ((P(src32[1:]), None, None, P(out), 1, 1, 2, 16, 0, 0), "misaligned")):
        assert lib.tlq_decode_lowbit_interleaved(*args, None) != 0 and word in _abi.last_error(), (word, _abi.last_error())
