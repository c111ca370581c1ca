"""Tuned kernel choice: the library's table (M, N, K, group, in_dtype) -> kernel family that tlq_gemm_w4a16[_ws] consult
before their rules -- the place where a tuner's result lives for callers of the C ABI, as the reference keeps its tuner's
winner per call signature in memory and on disk (tilelang/autotuner/tuner.py:102-760, tilelang/cache/tuner_cache.py).
Host behaviour (table, files, workspace sizing) without a GPU; on the GPU: a choice is honoured (the bits of the chosen
kernel come back), a choice the kernel refuses falls back to the rules, the tuner measures, installs and persists."""
import os

import pytest
import torch

from helpers import assert_bit_equal, check_float_output, gen, make_w4, w4a16_reference
from tilelang_ascend_amd import _abi


@pytest.fixture()
def lib():
    lib = _abi.load()
    lib.tlq_w4a16_choice_clear()
    yield lib
    lib.tlq_w4a16_choice_clear()


def test_table_set_get_remove_clear(lib):
    assert lib.tlq_w4a16_choice_count() == 0
    assert lib.tlq_w4a16_choice_get(64, 4096, 4096, 128, _abi.F16) == _abi.ALGO_AUTO
    assert lib.tlq_w4a16_choice_set(64, 4096, 4096, 128, _abi.F16, _abi.ALGO_STREAM) == 0
    assert lib.tlq_w4a16_choice_set(64, 4096, 4096, 128, _abi.BF16, _abi.ALGO_MFMA) == 0
    assert lib.tlq_w4a16_choice_count() == 2
    # the whole signature is the key
    assert lib.tlq_w4a16_choice_get(64, 4096, 4096, 128, _abi.F16) == _abi.ALGO_STREAM
    assert lib.tlq_w4a16_choice_get(64, 4096, 4096, 128, _abi.BF16) == _abi.ALGO_MFMA
    for other in ((65, 4096, 4096, 128), (64, 4097, 4096, 128), (64, 4096, 4095, 128), (64, 4096, 4096, 64)):
        assert lib.tlq_w4a16_choice_get(*other, _abi.F16) == _abi.ALGO_AUTO
    # an entry is replaced, and removed by TLQ_ALGO_AUTO
    assert lib.tlq_w4a16_choice_set(64, 4096, 4096, 128, _abi.F16, _abi.ALGO_PANELM) == 0
    assert lib.tlq_w4a16_choice_get(64, 4096, 4096, 128, _abi.F16) == _abi.ALGO_PANELM and lib.tlq_w4a16_choice_count() == 2
    assert lib.tlq_w4a16_choice_set(64, 4096, 4096, 128, _abi.F16, _abi.ALGO_AUTO) == 0
    assert lib.tlq_w4a16_choice_get(64, 4096, 4096, 128, _abi.F16) == _abi.ALGO_AUTO and lib.tlq_w4a16_choice_count() == 1
    lib.tlq_w4a16_choice_clear()
    assert lib.tlq_w4a16_choice_count() == 0 and lib.tlq_w4a16_choice_get(64, 4096, 4096, 128, _abi.BF16) == _abi.ALGO_AUTO


def test_table_rejects_bad_entries(lib):
    assert lib.tlq_w4a16_choice_set(64, 4096, 4096, 128, _abi.F16, 10) != 0 and "bad algo" in _abi.last_error()
    assert lib.tlq_w4a16_choice_set(64, 4096, 4096, 128, _abi.F16, -1) != 0
    assert lib.tlq_w4a16_choice_set(0, 4096, 4096, 128, _abi.F16, _abi.ALGO_STREAM) != 0
    assert lib.tlq_w4a16_choice_set(64, 4096, 4096, 128, _abi.I8, _abi.ALGO_STREAM) != 0 and "in_dtype" in _abi.last_error()
    assert lib.tlq_w4a16_choice_count() == 0


def test_save_and_load_round_trip(lib, tmp_path):
    entries = [(64, 4096, 4096, 128, _abi.F16, _abi.ALGO_STREAM), (256, 14336, 4096, 64, _abi.BF16, _abi.ALGO_PANELM),
               (1024, 4096, 4096, 128, _abi.BF16, _abi.ALGO_TWO_PASS)]
    for e in entries:
        assert lib.tlq_w4a16_choice_set(*e) == 0
    path = str(tmp_path / "choices.txt")
    assert lib.tlq_w4a16_choice_save(path.encode()) == 0
    lines = [ln.split() for ln in open(path) if not ln.startswith("#")]
    assert sorted(tuple(int(x) for x in ln) for ln in lines) == sorted(entries)
    lib.tlq_w4a16_choice_clear()
    # load adds to what the table holds and overrides an entry for the same signature
    assert lib.tlq_w4a16_choice_set(64, 4096, 4096, 128, _abi.F16, _abi.ALGO_MFMA) == 0
    assert lib.tlq_w4a16_choice_set(48, 1024, 1024, 128, _abi.F16, _abi.ALGO_SKINNY) == 0
    assert lib.tlq_w4a16_choice_load(path.encode()) == 0
    assert lib.tlq_w4a16_choice_count() == 4
    for e in entries:
        assert lib.tlq_w4a16_choice_get(*e[:5]) == e[5]
    assert lib.tlq_w4a16_choice_get(48, 1024, 1024, 128, _abi.F16) == _abi.ALGO_SKINNY


@pytest.mark.parametrize("bad", ["64 4096 4096 128 0\n", "64 4096 4096 128 0 5 7\n", "64 4096 4096 128 0 42\n", "64 4096 4096 128 3 5\n",
                                 "64 4096 4096 128 0 0\n", "x y z\n", "-1 4096 4096 128 0 5\n"])
def test_a_malformed_file_changes_nothing(lib, tmp_path, bad):
    assert lib.tlq_w4a16_choice_set(64, 4096, 4096, 128, _abi.F16, _abi.ALGO_MFMA) == 0
    path = tmp_path / "choices.txt"
    path.write_text("# comment\n\n32 1024 1024 128 0 6\n" + bad)
    assert lib.tlq_w4a16_choice_load(str(path).encode()) != 0
    assert "line 4" in _abi.last_error()
    assert lib.tlq_w4a16_choice_count() == 1 and lib.tlq_w4a16_choice_get(32, 1024, 1024, 128, _abi.F16) == _abi.ALGO_AUTO
    assert lib.tlq_w4a16_choice_load(str(tmp_path / "absent.txt").encode()) != 0 and "cannot read" in _abi.last_error()


def test_workspace_size_covers_the_chosen_family(lib):
    M, N, K = 64, 14336, 4096
    base = lib.tlq_w4a16_workspace_bytes(M, N, K)
    two = lib.tlq_w4a16_workspace_bytes_for(M, N, K, _abi.ALGO_TWO_PASS)
    assert two >= N * K * 2 > base
    assert lib.tlq_w4a16_workspace_bytes_for(M, N, K, _abi.ALGO_AUTO) == base
    assert lib.tlq_w4a16_workspace_bytes_for(M, N, K, _abi.ALGO_GEMV) == 0 == lib.tlq_w4a16_workspace_bytes_for(M, N, K, _abi.ALGO_SKINNY)
    # a choice for the shape (any group, any type) raises what the automatic size asks for; removing it restores it
    assert lib.tlq_w4a16_choice_set(M, N, K, 64, _abi.BF16, _abi.ALGO_TWO_PASS) == 0
    assert lib.tlq_w4a16_workspace_bytes(M, N, K) == two
    assert lib.tlq_w4a16_workspace_bytes(M, N, K + 128) < two  # another shape is not affected
    assert lib.tlq_w4a16_choice_set(M, N, K, 64, _abi.BF16, _abi.ALGO_AUTO) == 0
    assert lib.tlq_w4a16_workspace_bytes(M, N, K) == base
    # the panel families' sizes are what their plans ask for
    plan = (__import__("ctypes").c_int64 * 5)()
    assert lib.tlq_debug_panelm_plan(256, N, K, 128, lib.tlq_device_cu_count() or 256, plan) == 1
    assert lib.tlq_w4a16_workspace_bytes_for(256, N, K, _abi.ALGO_PANELM) >= (plan[2] * 256 * N * 4 if plan[2] > 1 else 0)


def test_choice_file_path_and_python_wrappers(lib, tmp_path, monkeypatch):
    from tilelang_ascend_amd import autotuner

    monkeypatch.setenv("TLQ_CACHE_DIR", str(tmp_path))
    p = autotuner.w4a16_choice_path(cus=256)
    assert p == os.path.join(str(tmp_path), "autotuner", "w4a16_choices_256cu.txt")
    assert autotuner.load_w4a16_choices(p) == 0  # no file: nothing installed
    assert lib.tlq_w4a16_choice_set(24, 4096, 4096, 128, _abi.F16, _abi.ALGO_SKINNY) == 0
    assert autotuner.save_w4a16_choices(p) == p and os.path.exists(p)
    autotuner.clear_w4a16_choices()
    assert lib.tlq_w4a16_choice_count() == 0
    assert autotuner.load_w4a16_choices(p) == 1
    assert lib.tlq_w4a16_choice_get(24, 4096, 4096, 128, _abi.F16) == _abi.ALGO_SKINNY
    # the cache's clear removes the file with the rest of the tuner records
    from tilelang_ascend_amd import cache

    cache.clear_cache()
    assert not os.path.exists(p)


# ---- on the GPU ----------------------------------------------------------------------------------------------------

def run_ws(lib, A, Wp, s, z, group, algo, need=None, dtype=torch.float16):
    P = _abi.ptr
    M, K = A.shape
    N = Wp.shape[0]
    code = _abi.F16 if dtype == torch.float16 else _abi.BF16
    if need is None:
        need = max(lib.tlq_w4a16_workspace_bytes_for(M, N, K, algo), lib.tlq_w4a16_workspace_bytes(M, N, K), 16)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    C = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
    print(f"tuned choice M={M} N={N} K={K} g={group} algo={algo} workspace={need}", flush=True)
    lib.tlq_debug_launch_log(1)
    rc = lib.tlq_gemm_w4a16_ws(P(A), P(Wp), P(s), P(z), P(C), M, N, K, group, 0.0, code, code, algo, P(ws), need,
                               torch.cuda.current_stream().cuda_stream)
    log = lib.tlq_debug_launch_log_text().decode()
    lib.tlq_debug_launch_log(0)
    _abi.check(rc)
    torch.cuda.synchronize()
    return C.cpu(), log


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K,group,chosen", [(64, 4096, 4096, 128, "ALGO_MFMA"), (64, 4096, 4096, 128, "ALGO_SKINNY"),
                                                (24, 4096, 4096, 128, "ALGO_STREAM"), (256, 2048, 2048, 128, "ALGO_PANELM"),
                                                (256, 1024, 1024, 64, "ALGO_TWO_PASS"), (16, 4096, 4096, 128, "ALGO_GEMV")])
def test_a_choice_is_honoured_and_removed(lib, M, N, K, group, chosen):
    algo = getattr(_abi, chosen)
    Wp, s, z = make_w4(N, K, group, torch.float16, "int", seed=M + N)
    A = torch.randn(M, K, generator=gen(M)).half()
    dev = [t.cuda() for t in (A, Wp, s, z)]
    auto, auto_log = run_ws(lib, *dev, group, _abi.ALGO_AUTO)
    explicit, explicit_log = run_ws(lib, *dev, group, algo)
    assert explicit_log != auto_log, "pick a family the rules do not take for this shape"
    assert lib.tlq_w4a16_choice_set(M, N, K, group, _abi.F16, algo) == 0
    tuned, tuned_log = run_ws(lib, *dev, group, _abi.ALGO_AUTO)
    assert tuned_log == explicit_log, (tuned_log, explicit_log)
    assert_bit_equal(tuned, explicit, chosen)
    check_float_output(tuned, w4a16_reference(A, Wp, s, z, group), chosen)
    # another type or group is another signature
    assert lib.tlq_w4a16_choice_set(M, N, K, group, _abi.F16, _abi.ALGO_AUTO) == 0
    assert lib.tlq_w4a16_choice_set(M, N, K, group, _abi.BF16, algo) == 0
    again, again_log = run_ws(lib, *dev, group, _abi.ALGO_AUTO)
    assert again_log == auto_log
    assert_bit_equal(again, auto, "rules")


@pytest.mark.gpu
def test_a_choice_the_kernel_refuses_falls_back_to_the_rules(lib):
    M, N, K, group = 24, 2048, 2048, 128
    Wp, s, z = make_w4(N, K, group, torch.float16, "int", seed=5)
    A = torch.randn(M, K, generator=gen(3)).half()
    dev = [t.cuda() for t in (A, Wp, s, z)]
    auto, auto_log = run_ws(lib, *dev, group, _abi.ALGO_AUTO)
    # the GEMV kernel takes 16 rows at most; the two passes need the dequantised matrix in the workspace
    for algo, need in ((_abi.ALGO_GEMV, None), (_abi.ALGO_TWO_PASS, 4096)):
        assert lib.tlq_w4a16_choice_set(M, N, K, group, _abi.F16, algo) == 0
        got, log = run_ws(lib, *dev, group, _abi.ALGO_AUTO, need=need)
        assert log == auto_log and _abi.last_error() == ""
        assert_bit_equal(got, auto, f"fallback from algo {algo}")
    # the entry point without a workspace consults the table as well, for the families it can run
    P = _abi.ptr
    C = torch.empty(M, N, dtype=torch.float16, device="cuda")
    lib.tlq_w4a16_choice_set(M, N, K, group, _abi.F16, _abi.ALGO_SKINNY)
    lib.tlq_debug_launch_log(1)
    _abi.check(lib.tlq_gemm_w4a16(P(dev[0]), P(dev[1]), P(dev[2]), P(dev[3]), P(C), M, N, K, group, 0.0, _abi.F16, _abi.F16,
                                  _abi.ALGO_AUTO, torch.cuda.current_stream().cuda_stream))
    log = lib.tlq_debug_launch_log_text().decode()
    lib.tlq_debug_launch_log(0)
    torch.cuda.synchronize()
    assert "skinny" in log, log
    check_float_output(C.cpu(), w4a16_reference(A, Wp, s, z, group), "skinny by choice")


@pytest.mark.gpu
def test_the_tuner_measures_installs_and_persists(lib, tmp_path, monkeypatch):
    from tilelang_ascend_amd import autotuner

    monkeypatch.setenv("TLQ_CACHE_DIR", str(tmp_path))
    M, N, K, group = 48, 2048, 2048, 128
    res = autotuner.tune_w4a16_choice(M, N, K, group, "float16", zeros="tensor", rep=5, rounds=2)
    print("tuner:", res, flush=True)
    assert "auto" in res["latency_us"] and len(res["latency_us"]) >= 3
    assert "gemv" in res["skipped"] and "decode" in res["skipped"]  # 48 rows: more than those kernels take
    assert not res["rejected"], res["rejected"]
    assert res["path"] == autotuner.w4a16_choice_path() and os.path.exists(res["path"])
    want = _abi.ALGO_AUTO if res["choice"] == "auto" else autotuner.W4A16_FAMILIES[res["choice"]]
    assert lib.tlq_w4a16_choice_get(M, N, K, group, _abi.F16) == want
    if res["choice"] != "auto":
        assert res["latency_us"][res["choice"]] <= res["latency_us"]["auto"] * 0.97
    # a forced win: with only one candidate and any gain accepted the entry must appear, persist and load again
    res = autotuner.tune_w4a16_choice(M, N, K, group, "float16", zeros="tensor", candidates=["mfma"], rep=5, rounds=2, min_gain=-10.0)
    assert res["choice"] == "mfma" and lib.tlq_w4a16_choice_get(M, N, K, group, _abi.F16) == _abi.ALGO_MFMA
    autotuner.clear_w4a16_choices()
    assert autotuner.load_w4a16_choices() == 1 and lib.tlq_w4a16_choice_get(M, N, K, group, _abi.F16) == _abi.ALGO_MFMA
    # and the operator surface runs the tuned family
    from tilelang_ascend_amd import ops

    Wp, s, z = make_w4(N, K, group, torch.float16, "int", seed=9)
    A = torch.randn(M, K, generator=gen(4)).half()
    kernel = ops.w4a16_gemm(M, N, K, group_size=group, zeros="tensor")
    C = kernel(A.cuda(), Wp.cuda(), s.cuda(), z.cuda())
    explicit = ops.w4a16_gemm(M, N, K, group_size=group, zeros="tensor", algo="mfma")(A.cuda(), Wp.cuda(), s.cuda(), z.cuda())
    assert_bit_equal(C.cpu(), explicit.cpu(), "operator with a tuned choice")
    check_float_output(C.cpu(), w4a16_reference(A, Wp, s, z, group), "operator with a tuned choice")
