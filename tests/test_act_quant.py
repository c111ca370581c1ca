"""Per-token int8 activation quantiser: oracle pins (CPU) and kernel parity (GPU).

Reference: examples/deepseek_v4/act_quant.py (golden :112-142, test :151-168 with
Y atol=1 and S rtol=atol=1e-2).  The bar here is tighter: Y and S bit-exact with the golden's
float32 arithmetic.
"""
import numpy as np
import pytest
import torch

from oracle import ref


# ------------------------------------------------------------------ oracle pins (CPU)
def test_oracle_known_rows():
    x = torch.tensor([[127.0, 0.5, 1.5, 2.5, -0.5, -2.5, 3.49, -126.5],    # scale exactly 1: ties to even
                      [0.0] * 8,                                           # all-zero row: floor 1e-4
                      [-4.0] * 8,                                          # constant row -> -127
                      [254.0, -254.0, 127.0, 1.0, 0.99, -1.0, 3.0, 2.0]])  # scale exactly 2
    y, s = ref.act_quant_torch(x)
    assert y.dtype == torch.int8 and s.dtype == torch.float32 and s.shape == (4, 1)
    assert y[0].tolist() == [127, 0, 2, 2, 0, -2, 3, -126]
    assert s[0, 0].item() == 1.0
    assert y[1].tolist() == [0] * 8 and s[1, 0].item() == np.float32(1e-4) / np.float32(127)
    assert y[2].tolist() == [-127] * 8 and s[2, 0].item() == np.float32(4) / np.float32(127)
    assert y[3].tolist() == [127, -127, 64, 0, 0, 0, 2, 1] and s[3, 0].item() == 2.0


def test_oracle_invariants():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(37, 200, generator=g).bfloat16()
    y, s = ref.act_quant_torch(x)
    xf = x.float()
    # the row maximum maps to +-127 and nothing leaves the int8 range used
    idx = xf.abs().argmax(dim=1)
    assert torch.equal(y[torch.arange(37), idx].abs(), torch.full((37,), 127, dtype=torch.int8))
    assert int(y.min()) >= -127
    # rounding, not truncation: error at most half a step (plus float slack)
    assert float(((y.float() * s - xf).abs() / s).max()) <= 0.5 + 1e-4
    # odd symmetry and exact power-of-two scaling
    y2, s2 = ref.act_quant_torch(-x)
    assert torch.equal(y2, -y) and torch.equal(s2, s)
    y3, s3 = ref.act_quant_torch(x * 8)
    assert torch.equal(y3, y) and torch.equal(s3, s * 8)
    # 3-D input keeps its shape (act_quant.py:115-121, :137-139)
    y4, s4 = ref.act_quant_torch(x[:36].view(4, 9, 200))
    assert y4.shape == (4, 9, 200) and s4.shape == (4, 9, 1) and torch.equal(y4.view(36, 200), y[:36])


def test_oracle_matches_elementwise_loop():
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(9, 40, generator=g) * 3).bfloat16()
    x[4] = 0
    y, s = ref.act_quant_torch(x)
    yl, sl = ref.act_quant_loop(x)
    assert np.array_equal(y.numpy(), yl) and np.array_equal(s.view(-1).numpy(), sl)


def test_pow2_ceil_is_smallest_power_of_two_not_below():
    powers = np.float32(2.0) ** np.arange(-126, 127, dtype=np.float32)
    rng = np.random.default_rng(0)
    s = np.concatenate([np.exp(rng.uniform(-20, 20, 2000)).astype(np.float32), powers[20:200],
                        np.nextafter(powers[20:200], np.float32(np.inf)),
                        np.nextafter(powers[20:200], np.float32(0))])
    got = ref.pow2_ceil(s)
    want = powers[np.searchsorted(powers, s, side="left")]
    assert np.array_equal(got, want)


def test_round_scale_literal_and_exact_agree_away_from_powers_of_two():
    g = torch.Generator().manual_seed(7)
    x = torch.randn(64, 128, generator=g).bfloat16()
    y0, s0 = ref.act_quant_torch(x, round_scale=True)
    y1, s1 = ref.act_quant_torch(x, round_scale=True, exact_log2=True)
    assert torch.equal(s0, s1) and torch.equal(y0, y1)
    plain = ref.act_quant_torch(x)[1]
    assert bool(((s1 >= plain) & (s1 < 2 * plain)).all())
    # one ulp above a power of two: log2 rounds to the integer and the literal form stays below
    one_up = np.nextafter(np.float32(2.0 ** -7), np.float32(1))
    assert ref.pow2_ceil(one_up) == np.float32(2.0 ** -6)
    assert float(2 ** torch.ceil(torch.log2(torch.tensor(one_up)))) == 2.0 ** -7


def test_c_restatement_agrees():
    from oracle import cref

    g = torch.Generator().manual_seed(9)
    x = (torch.randn(50, 384, generator=g) * torch.logspace(-6, 6, 50).view(50, 1)).bfloat16()
    x[7] = 0
    for rs in (False, True):
        y, s = ref.act_quant_torch(x, round_scale=rs, exact_log2=True)
        yc, sc = cref.act_quant(x.float().numpy(), rs)
        assert np.array_equal(y.numpy(), yc) and np.array_equal(s.view(-1).numpy(), sc)


def test_reciprocal_fma_quotient_rounds_like_division():
    """The kernel replaces x / s by q0 = x * r, q = fma(fma(-q0, s, x), r, q0) with r = fl(1 / s); the
    integer it stores must be the one the division gives, ties included."""
    from oracle import cref

    bad_int, bad_q = cref.act_quant_quotient_check(30_000_000, seed=12345)
    assert bad_int == 0
    assert bad_q < 30_000_000 // 500      # raw quotients differ only where the remainder underflows


# ------------------------------------------------------------------ kernel parity (GPU)
def _kernel(N, **kw):
    from tilelang_ascend_amd.ops import act_quant_kernel_int8_optimized

    return act_quant_kernel_int8_optimized(N, **kw)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N", [(128, 1024), (1, 8), (3, 520), (33, 4096), (5, 7168), (4, 8192), (3, 8200),
                                 (2, 16384), (3, 32768), (2, 32776), (7, 33), (2, 1), (0, 64),
                                 (4100, 512), (4099, 4096), (4097, 2048), (4098, 1032)])
@pytest.mark.parametrize("dtype", ["bfloat16", "float16", "float32"])
def test_act_quant_matches_golden(M, N, dtype):
    tdt = ref.TORCH_DTYPE[dtype]
    g = torch.Generator().manual_seed(M * 131 + N)
    x = (torch.randn(M, N, generator=g) * 2.5).to(tdt)
    if M > 2:
        x[1] = 0                 # all-zero row
        x[2] = x[2, 0]           # constant row
    Y, S = _kernel(N, block_M=16, block_N=N, in_dtype=dtype)(x.cuda())
    assert Y.dtype == torch.int8 and S.dtype == torch.float32 and Y.shape == (M, N) and S.shape == (M,)
    y, s = ref.act_quant_torch(x)
    assert torch.equal(Y.cpu(), y)
    assert torch.equal(S.cpu(), s.view(M))


@pytest.mark.gpu
def test_act_quant_reference_example():
    """The reference's own test (act_quant.py:151-168): M=128, N=1024, block_M=16, block_N=N, with
    its tolerances, through the profiler-free call path it uses."""
    M, N = 128, 1024
    x = torch.randn(M, N, dtype=torch.bfloat16)
    Y, S = _kernel(N, block_M=16, block_N=N, round_scale=False)(x.cuda())
    y, s = ref.act_quant_torch(x)
    torch.testing.assert_close(Y.cpu(), y, rtol=1e-2, atol=1)
    torch.testing.assert_close(S.cpu().reshape(M), s.reshape(M), rtol=1e-2, atol=1e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_act_quant_round_scale(dtype):
    M, N = 96, 2048
    g = torch.Generator().manual_seed(11)
    x = (torch.randn(M, N, generator=g) * torch.logspace(-3, 3, M).view(M, 1)).to(ref.TORCH_DTYPE[dtype])
    x[5] = 0
    x[6, :] = 0
    x[6, 3] = 127 * 0.25      # amax / 127 exactly a power of two
    Y, S = _kernel(N, round_scale=True, in_dtype=dtype)(x.cuda())
    y, s = ref.act_quant_torch(x, round_scale=True, exact_log2=True)
    assert torch.equal(S.cpu(), s.view(M)) and torch.equal(Y.cpu(), y)
    assert S[6].item() == 0.25
    m = torch.frexp(S.cpu())[0]
    assert bool((m == 0.5).all())  # every scale is a power of two


@pytest.mark.gpu
def test_act_quant_ties_and_extremes():
    x = torch.tensor([[127.0, 0.5, 1.5, 2.5, -0.5, -2.5, 3.49, -126.5],
                      [0.0] * 8, [-4.0] * 8,
                      [254.0, -254.0, 127.0, 1.0, 0.99, -1.0, 3.0, 2.0]])
    for dtype in ("float32", "bfloat16", "float16"):
        xd = x.to(ref.TORCH_DTYPE[dtype])
        Y, S = _kernel(8, in_dtype=dtype)(xd.cuda())
        y, s = ref.act_quant_torch(xd)
        assert torch.equal(Y.cpu(), y) and torch.equal(S.cpu(), s.view(-1))
    big = torch.full((2, 64), 3.0e38)
    big[1, 1] = -3.0e38
    big[1, 2] = 1e-30
    Y, S = _kernel(64, in_dtype="float32")(big.cuda())
    y, s = ref.act_quant_torch(big)
    assert torch.equal(Y.cpu(), y) and torch.equal(S.cpu(), s.view(-1))


@pytest.mark.gpu
def test_act_quant_feeds_w8a8_gemm():
    """quantise -> int8 GEMM with the per-token scales reproduces the float product to
    quantisation accuracy (the end-to-end use in examples/deepseek_v4)."""
    from tilelang_ascend_amd.ops import int8_gemm_kernel_corrected

    M, N, K = 64, 256, 1024
    g = torch.Generator().manual_seed(2)
    a = torch.randn(M, K, generator=g).bfloat16()
    w = torch.randn(N, K, generator=g).bfloat16()
    Aq, Sa = _kernel(K)(a.cuda())
    Wq, Sw = _kernel(K)(w.cuda())
    C = int8_gemm_kernel_corrected(N, K, out_dtype="float32")(Aq, Wq, Sa, Sw)
    want = ref.ref_int8_gemm_sequential(Aq.cpu(), Wq.cpu(), Sa.cpu(), Sw.cpu(), torch.float32)
    assert torch.equal(C.cpu(), want)
    exact = a.float() @ w.float().T
    rel = float((C.cpu() - exact).norm() / exact.norm())
    assert rel < 2e-2, rel


@pytest.mark.gpu
def test_act_quant_rejects_bad_arguments():
    from tilelang_ascend_amd import _abi

    lib = _abi.load()
    x = torch.zeros(4, 64, device="cuda", dtype=torch.bfloat16)
    y = torch.empty(4, 64, device="cuda", dtype=torch.int8)
    s = torch.empty(4, device="cuda")
    P = _abi.ptr
    assert lib.tlq_act_quant_i8(P(x), P(y), P(s), 4, 64, _abi.I8, 0, None) != 0
    assert "in_dtype" in _abi.last_error()
    assert lib.tlq_act_quant_i8(P(x), P(y), P(s), -1, 64, _abi.BF16, 0, None) != 0
    assert lib.tlq_act_quant_i8(None, P(y), P(s), 4, 64, _abi.BF16, 0, None) != 0
    assert lib.tlq_act_quant_i8(P(x), P(y), P(s), 0, 64, _abi.BF16, 0, None) == 0
    with pytest.raises(ValueError):
        _kernel(64)(x.half())
