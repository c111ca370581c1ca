"""Autotuner: interface and caching logic (CPU) and a real search over kernel variants (GPU).

Reference: tilelang/autotuner/tuner.py (AutoTuner :102-595, autotune :675-760), examples/autotune.
"""
import json
import os

import pytest
import torch

import tilelang_ascend_amd as tl
from tilelang_ascend_amd import autotuner as at
from tilelang_ascend_amd.ops import w4a16_gemm


def test_surface_and_lazy_exports():
    assert tl.autotune is at.autotune and tl.AutoTuner is at.AutoTuner
    tuner = at.AutoTuner.from_kernel(kernel=w4a16_gemm, configs=[{"tile": 64}])
    assert tuner.set_compile_args(out_idx=[-1], target="auto") is tuner
    assert tuner.set_profile_args(warmup=3, rep=5, ref_prog=None, skip_check=True) is tuner
    assert tuner.profile_args.warmup == 3 and tuner.profile_args.skip_check
    with pytest.raises(ValueError, match="not supported yet"):
        at.autotune(lambda: None, configs=[])


def test_all_tunables_given_skips_the_search():
    calls = []

    def configs(*a, **k):
        calls.append((a, k))
        return [{"tile": 64, "algo": "mfma"}, {"tile": 128, "algo": "mfma"}]

    tuned = at.autotune(configs=configs)(w4a16_gemm)
    kernel = tuned(64, 128, 256, tile=128, algo="mfma")        # nothing left to tune: no GPU needed
    assert kernel.spec.attrs["tile"] == 128 and kernel.get_tuner_result() is None
    assert kernel is w4a16_gemm(64, 128, 256, tile=128, algo="mfma")
    assert calls and calls[0][0] == (64, 128, 256)


def test_cache_key_depends_on_arguments_and_configs():
    def key(args, configs):
        t = at.AutoTuner(w4a16_gemm, configs)
        t.set_kernel_parameters(at._normalize(args), None)
        return t.generate_cache_key(configs)

    a = key([[64, 128, 256], {}], [{"tile": 64}])
    assert a == key([[64, 128, 256], {}], [{"tile": 64}])
    assert a != key([[64, 128, 512], {}], [{"tile": 64}])
    assert a != key([[64, 128, 256], {}], [{"tile": 128}])


def test_result_round_trips_through_the_disk_cache(tmp_path, monkeypatch):
    monkeypatch.setenv("TLQ_CACHE_DIR", str(tmp_path))
    t = at.AutoTuner(w4a16_gemm, [{"tile": 64}])
    res = at.AutotuneResult(latency=0.5, config={"tile": 64}, ref_latency=2.0, trials=[({"tile": 64}, 0.5, None),
                                                                                     ({"tile": 16}, None, "boom")])
    t._save_result_to_disk("k1", res)
    assert os.path.isdir(os.path.join(str(tmp_path), "autotuner"))
    back = t._load_result_from_disk("k1")
    assert back.config == {"tile": 64} and back.latency == 0.5 and back.ref_latency == 2.0 and len(back.trials) == 2
    assert t._load_result_from_disk("missing") is None
    tl.cache.clear_cache()
    assert t._load_result_from_disk("k1") is None              # clear_cache empties the tuning records too


def test_set_autotune_inputs_nests():
    assert at.get_autotune_inputs() is None
    with at.set_autotune_inputs(1, 2):
        assert at.get_autotune_inputs() == [1, 2]
        with at.set_autotune_inputs([3]):
            assert at.get_autotune_inputs() == [3]
        assert at.get_autotune_inputs() == [1, 2]
    assert at.get_autotune_inputs() is None


# ------------------------------------------------------------------------------------------ GPU
def _ref(A, Bp, S):
    from tilelang_ascend_amd.examples._checks import unpack_nibbles

    W = (unpack_nibbles(Bp).to(torch.float16) - 8.0) * S.cpu().repeat_interleave(128, dim=1)
    return (A.cpu().float() @ W.float().T).to(A.dtype)


def _supply(M, N, K):
    def prog(_params):
        g = torch.Generator().manual_seed(0)
        return [torch.randn(M, K, generator=g).half().cuda(),
                torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, generator=g).cuda(),
                (torch.rand(N, K // 128, generator=g) * 0.015 + 0.005).half().cuda()]
    return prog


@pytest.mark.gpu
def test_search_picks_a_valid_kernel_and_caches_it(tmp_path, monkeypatch):
    monkeypatch.setenv("TLQ_CACHE_DIR", str(tmp_path))
    at.AutoTuner._memory_cache.clear()
    M, N, K = 48, 512, 1024
    configs = [{"algo": "mfma", "tile": 16}, {"algo": "mfma", "tile": 64}, {"algo": "skinny", "tile": 0},
               {"algo": "gemv", "tile": 0}]                      # gemv is rejected for M = 48: recorded, not fatal
    tuned = tl.autotune(configs=configs, ref_prog=_ref, supply_prog=_supply(M, N, K), warmup=2, rep=5)(w4a16_gemm)
    kernel = tuned(M, N, K, group_size=128, zeros=8)
    res = kernel.get_tuner_result()
    assert res.config in configs[:3] and res.latency > 0 and res.ref_latency is not None
    errors = [e for _, _, e in res.trials if e]
    assert len(res.trials) == 4 and len(errors) == 1 and "RuntimeError" in errors[0]
    A, Bp, S = _supply(M, N, K)(None)
    torch.testing.assert_close(kernel(A, Bp, S).cpu(), _ref(A, Bp, S), rtol=1e-2, atol=1e-2)
    assert tuned(M, N, K, group_size=128, zeros=8) is kernel    # memory cache per call signature
    files = os.listdir(os.path.join(str(tmp_path), "autotuner"))
    assert len(files) == 1 and json.load(open(os.path.join(str(tmp_path), "autotuner", files[0])))["config"] == res.config

    # a fresh decorator (new process in real use) takes the stored result without timing anything
    at.AutoTuner._memory_cache.clear()
    monkeypatch.setattr(at, "do_bench", lambda *a, **k: (_ for _ in ()).throw(AssertionError("timed again")))
    again = tl.autotune(configs=configs, ref_prog=_ref, supply_prog=_supply(M, N, K), warmup=2, rep=5)(w4a16_gemm)
    k2 = again(M, N, K, group_size=128, zeros=8)
    assert k2.get_tuner_result().config == res.config


@pytest.mark.gpu
def test_every_configuration_failing_raises(tmp_path, monkeypatch):
    monkeypatch.setenv("TLQ_CACHE_DIR", str(tmp_path))
    at.AutoTuner._memory_cache.clear()
    tuned = tl.autotune(configs=[{"algo": "gemv"}], supply_prog=_supply(48, 512, 1024), warmup=1, rep=2)(w4a16_gemm)
    with pytest.raises(RuntimeError, match="no configuration produced a valid kernel"):
        tuned(48, 512, 1024, group_size=128, zeros=8)


@pytest.mark.gpu
def test_autotune_example(capsys):
    from tilelang_ascend_amd.examples.autotune import example_gemm_autotune as ex

    ex.main(["--m", "32", "--n", "512", "--k", "1024"])
    out = capsys.readouterr().out
    assert "Best Config: {" in out and out.rstrip().endswith("Test passed!")
