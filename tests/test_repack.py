"""GPU weight repacker: tlq_pack_int4 / tlq_quantize_sym4 against the restated
tilelang/quantize/utils.py (general_compress :53-69, interleave_weight :73-101, gen_quant4 :5-50)."""
import numpy as np
import pytest
import torch

from oracle import ref


def test_oracle_quantizer_matches_gen_quant4_transposed():
    """quantize_sym4 is gen_quant4's arithmetic on the transposed layout: feed it gen_quant4's own weights."""
    torch.manual_seed(5)
    w, _linear, s, q = ref.gen_quant4(256, 48, groupsize=64)       # w [k, n], s [k/64, n], q [k, n] (already - 8)
    q2, s2 = ref.quantize_sym4(w.t().contiguous(), 64)
    assert torch.equal(q2, q.t().to(torch.int8)) and torch.equal(s2, s.t().contiguous())
    assert int(q2.max()) == 8 and int(q2.min()) >= -8             # +max element reaches 16 - 8
    # dequantised value is within half a step of the weight
    deq = q2.float().view(48, 4, 64) * s2.float().view(48, 4, 1)
    assert float((deq - w.t().float().view(48, 4, 64)).abs().max() / s2.float().max()) <= 0.5 + 1e-3


def test_oracle_quantizer_zero_group():
    W = torch.zeros(2, 16, dtype=torch.float16)
    W[1, 3] = 2.0
    q, s = ref.quantize_sym4(W, 8)
    assert q[0].tolist() == [-8] * 16 and s[0].tolist() == [0.0, 0.0]
    assert q[1].tolist() == [0, 0, 0, 8] + [0] * 4 + [-8] * 8 and s[1, 0].item() == 0.25


@pytest.mark.gpu
@pytest.mark.parametrize("interleave", [None, "float16", "int8"])
@pytest.mark.parametrize("N,K", [(1, 8), (3, 24), (7, 40), (128, 4096), (11008, 4096), (5, 8)])
def test_pack_matches_general_compress_and_interleave(interleave, N, K):
    from tilelang_ascend_amd.quantize import gpu

    g = torch.Generator().manual_seed(N * 7 + K)
    vals = torch.randint(0, 16, (N, K), dtype=torch.int8, generator=g)
    want = ref.general_compress(vals, 4, torch.int8)
    if interleave:
        want = ref.interleave_weight(want, 4, interleave)
    got = gpu.pack_int4(vals.cuda(), interleave).cpu()
    assert got.dtype == torch.int8 and torch.equal(got, want)
    if interleave is None:  # the packed bytes are what the unpack kernel reads back
        assert np.array_equal(ref.unpack_uint4(got), vals.numpy().astype(np.uint8))


@pytest.mark.gpu
def test_pack_does_not_mask_like_the_reference():
    """Out-of-range values spill into their neighbours (the reference ORs unmasked int8 operands)."""
    from tilelang_ascend_amd.quantize import gpu

    vals = torch.tensor([[-1, 0, 16, 3, -8, 7, 127, -128]], dtype=torch.int8)
    want = ref.general_compress(vals, 4, torch.int8)
    got = gpu.pack_int4(vals.cuda()).cpu()
    assert torch.equal(got, want) and got.view(torch.uint8)[0, 0].item() == 0xFF
    g = torch.Generator().manual_seed(1)
    wild = torch.randint(-128, 128, (33, 64), dtype=torch.int8, generator=g)
    assert torch.equal(gpu.pack_int4(wild.cuda()).cpu(), ref.general_compress(wild, 4, torch.int8))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N,K,group", [(48, 256, 64), (11008, 4096, 128), (5, 4096, 4096), (3, 1536, 24), (64, 1024, 8),
                                       (7, 2048, 1024), (2, 128, -1)])
def test_quantizer_matches_gen_quant4_arithmetic(dtype, N, K, group):
    from tilelang_ascend_amd.quantize import gpu

    g = torch.Generator().manual_seed(N + K)
    W = torch.randn(N, K, generator=g).to(dtype)
    if N > 2:
        W[1, : (K if group == -1 else group)] = 0       # a group of zeros
        W[2] *= 1e-6                                     # tiny values: scales near the subnormal range
    q, s = gpu.quantize_sym4(W.cuda(), group)
    wq, ws = ref.quantize_sym4(W, K if group == -1 else group)
    assert torch.equal(s.cpu(), ws)
    assert torch.equal(q.cpu(), wq)


@pytest.mark.gpu
def test_quantize_pack_then_gemm_round_trip():
    """quantise -> pack on the GPU -> W4A16 GEMM with zero point 8 equals the GEMM on the dequantised weights."""
    from tilelang_ascend_amd.ops import w4a16_gemm
    from tilelang_ascend_amd.quantize import gpu

    M, N, K, group = 32, 256, 1024, 128
    g = torch.Generator().manual_seed(3)
    W = torch.randn(N, K, generator=g).half()
    A = torch.randn(M, K, generator=g).half()
    q, s = gpu.quantize_sym4(W.cuda(), group)
    q = q.clamp(max=7)                                   # the +max element (q = 16) does not fit a nibble
    packed = gpu.pack_int4((q + 8).to(torch.int8), None, torch.uint8)
    C = w4a16_gemm(M, N, K, group_size=group, zeros=8)(A.cuda(), packed, s)
    deq = (q.cpu().half().view(N, K // group, group) * s.cpu().view(N, K // group, 1)).view(N, K)
    want = (A.float() @ deq.float().T)
    rel = float((C.cpu().float() - want).norm() / want.norm())
    assert rel < 1e-3, rel


@pytest.mark.gpu
def test_repack_rejects_bad_arguments():
    from tilelang_ascend_amd import _abi
    from tilelang_ascend_amd.quantize import gpu

    lib, P = _abi.load(), _abi.ptr
    v = torch.zeros(4, 16, dtype=torch.int8, device="cuda")
    o = torch.zeros(4, 8, dtype=torch.int8, device="cuda")
    assert lib.tlq_pack_int4(P(v), P(o), 4, 12, 0, None) != 0 and "multiple of 8" in _abi.last_error()
    assert lib.tlq_pack_int4(P(v), P(o), 4, 16, 3, None) != 0
    assert lib.tlq_pack_int4(P(v), P(o), 0, 16, 0, None) == 0
    w = torch.zeros(4, 16, dtype=torch.float16, device="cuda")
    s = torch.zeros(4, 2, dtype=torch.float16, device="cuda")
    assert lib.tlq_quantize_sym4(P(w), P(v), P(s), 4, 16, 12, _abi.F16, None) != 0
    assert lib.tlq_quantize_sym4(P(w), P(v), P(s), 4, 16, 8, _abi.F32, None) != 0
    with pytest.raises(ValueError):
        gpu.pack_int4(v.cpu())
    with pytest.raises(ValueError):
        gpu.quantize_sym4(w.float())


@pytest.mark.gpu
@pytest.mark.parametrize("groupsize", [128, -1])
def test_gen_quant4_results_feed_the_w4a16_operands(groupsize):
    """gen_quant4 -> pack_gen_quant4 -> dequantize_w4(zero point 8) gives gen_quant4's own dequantised weight (the
    nn.Linear it returns), except where q = 16 was stored as 15; scales travel from [K/g, N] to [N, K/g]."""
    from tilelang_ascend_amd import quantize as Q
    from tilelang_ascend_amd.ops import dequantize_w4
    from tilelang_ascend_amd.quantize import gpu

    torch.manual_seed(11)
    k, n = 256, 72
    _, linear, s, q8 = Q.gen_quant4(k, n, groupsize)
    g = k if groupsize == -1 else groupsize
    assert s.shape == (k // g, n)
    assert torch.equal(gpu.scales_kn_to_nk(s), s.t())
    Bp, S = gpu.pack_gen_quant4(q8, s)
    assert Bp.shape == (n, k // 2) and Bp.dtype == torch.uint8 and S.shape == (n, k // g) and S.is_contiguous()
    W = dequantize_w4(Bp, S, 8, g, torch.float16).cpu()
    want = linear.weight.data  # [n, k] = ((q - 8).half() * s).T
    top = (q8.t() == 8)
    assert top.any()  # the positive maximum of a group always quantises to 16
    assert torch.equal(W[~top], want[~top])
    s_full = s.repeat_interleave(g, dim=0).t()
    assert torch.equal(W[top], (7 * s_full[top].float()).half())
    with pytest.raises(ValueError, match="four bits"):
        gpu.pack_gen_quant4(q8, s, saturate=False)
    with pytest.raises(ValueError):
        gpu.pack_gen_quant4(q8 + 5, s)


def test_packed_weights_round_trip_through_a_file(tmp_path):
    """save_packed / load_packed: plain tensors and numbers only, read back with a loader that executes nothing."""
    from tilelang_ascend_amd.quantize import load_packed, save_packed

    g = torch.Generator().manual_seed(5)
    N, K, group = 48, 256, 64
    Bp = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=g)
    s = (torch.rand(N, K // group, generator=g) * 0.015 + 0.005).half()
    z = torch.randint(6, 10, (N, K // group), generator=g).half()
    for layout, zeros in (("plain", z), ("interleaved", 8), ("plain", None)):
        path = tmp_path / f"w_{layout}_{type(zeros).__name__}.pt"
        save_packed(path, Bp, s, zeros, layout=layout, group=group)
        got = load_packed(path)
        assert got["layout"] == layout and got["group"] == group and (got["N"], got["K"]) == (N, K)
        assert torch.equal(got["B_packed"], Bp) and torch.equal(got["scales"], s)
        if torch.is_tensor(zeros):
            assert torch.equal(got["zeros"], zeros)
        else:
            assert got["zeros"] == zeros
    with pytest.raises(ValueError):
        save_packed(tmp_path / "bad.pt", Bp, s[:, :1], None, group=group)
    with pytest.raises(ValueError):
        save_packed(tmp_path / "bad.pt", Bp, s, None, layout="tiled", group=group)
    torch.save({"format": "something else"}, tmp_path / "other.pt")
    with pytest.raises(ValueError):
        load_packed(tmp_path / "other.pt")
