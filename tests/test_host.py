"""Host-side logic that needs no GPU: the jit front door, the kernel cache and the launch
contract's validation (reference: tilelang/jit/__init__.py:197-247, tilelang/jit/adapter/base.py:22-46,
tilelang/jit/adapter/cython/cython_wrapper.pyx:102-203, tilelang/cache/kernel_cache.py)."""
import os
import threading

import pytest
import torch

import tilelang_ascend_amd as tl
from tilelang_ascend_amd import cache, ops
from tilelang_ascend_amd.jit import JITKernel, KernelSpec, Param, _legalize_idx


@pytest.fixture(autouse=True)
def _cache_in_tmp(tmp_path, monkeypatch):
    monkeypatch.setenv("TLQ_CACHE_DIR", str(tmp_path / "cache"))
    tl.enable_cache()
    cache.clear_cache()
    yield
    tl.enable_cache()


def _spec(name="k", launch=None):
    return KernelSpec(name, [Param("A", (4, 8), "int8"), Param("B", (8, 16), "int8"), Param("C", (4, 16), "int32"),
                             Param("ws", (4, 16), "int32")], launch or (lambda t, s, st: None))


def test_idx_legalisation():
    assert _legalize_idx(None, 4, "result_idx") == []
    assert _legalize_idx(2, 4, "result_idx") == [2]
    assert _legalize_idx([-1, -2], 4, "result_idx") == [3, 2]
    for bad in (4, -5, [0, 7]):
        with pytest.raises(ValueError, match="should be an integer between -4 and 3"):
            _legalize_idx(bad, 4, "result_idx")
    with pytest.raises(ValueError, match="list of integers"):
        _legalize_idx("1", 4, "result_idx")


def test_factory_memoises_per_arguments():
    k1 = ops.simple_quant_batch_matmul(2, 64, 64, 64, "N", 128, 256, 64)
    k2 = ops.simple_quant_batch_matmul(2, 64, 64, 64, "N", 128, 256, 64)
    k3 = ops.simple_quant_batch_matmul(2, 64, 64, 64, "1", 128, 256, 64)
    k4 = ops.simple_quant_batch_matmul(2, 64, 64, 64, "N", 128, 256, 64, out_dtype="bfloat16")
    assert k1 is k2 and k1 is not k3 and k1 is not k4
    assert isinstance(k1, JITKernel)
    assert k1.result_idx == [3] and k1.workspace_idx == [4] and k1.input_idx == [0, 1, 2]
    assert [p.name for p in k1.params] == ["A", "B", "scale", "C", "workspace_1"]
    assert k3.params[2].shape == (1,) and k1.params[2].shape == (64,)
    assert k4.params[3].dtype == "bfloat16"
    assert "simple_quant_batch_matmul" in k1.get_kernel_source()
    with pytest.raises(ValueError, match='scale_size must be "1" or "N"'):
        ops.simple_quant_batch_matmul(2, 64, 64, 64, "M", 128, 256, 64)


def test_disable_cache_builds_fresh_kernels_and_clear_cache_is_harmless():
    a = ops.w4a8_gemm_cv(64, 64, 128)
    assert ops.w4a8_gemm_cv(64, 64, 128) is a
    tl.disable_cache()
    assert not tl.is_cache_enabled()
    b = ops.w4a8_gemm_cv(64, 64, 128)
    assert b is not a
    tl.enable_cache()
    from tilelang_ascend_amd import build

    before = os.path.getmtime(build.LIB_PATH)
    tl.cache.clear_cache()  # the reference's examples do this at import time
    assert os.path.exists(build.LIB_PATH) and os.path.getmtime(build.LIB_PATH) == before
    assert os.path.isdir(cache.cache_dir()) and os.listdir(cache.cache_dir()) == []


def test_cache_key_covers_spec_indices_and_pass_configs():
    s = _spec()
    base = cache.make_key(s, [2], [3], "auto", "ctypes", None)
    assert base == cache.make_key(_spec(), [2], [3], "auto", "ctypes", None)
    assert base != cache.make_key(_spec("other"), [2], [3], "auto", "ctypes", None)
    assert base != cache.make_key(s, [-2], [3], "auto", "ctypes", None)
    assert base != cache.make_key(s, [2], None, "auto", "ctypes", None)
    assert base != cache.make_key(s, [2], [3], "auto", "ctypes", {tl.PassConfigKey.TL_ASCEND_AUTO_SYNC: True})
    assert base != cache.make_key(s, [2], [3], "auto", "ctypes", {"some.unknown.key": 1})  # unknown keys still count
    k = tl.compile(s, out_idx=[2], workspace_idx=[3])
    assert tl.compile(_spec(), out_idx=[2], workspace_idx=[3]) is k
    assert len(os.listdir(cache.cache_dir())) == 1
    with pytest.raises(TypeError):
        tl.compile(lambda: None)


def test_cache_is_thread_safe():
    made = []

    def builder():
        made.append(1)
        return JITKernel(_spec("threaded"), [2], [3])

    got = []
    ts = [threading.Thread(target=lambda: got.append(cache.cached("same-key", builder))) for _ in range(8)]
    [t.start() for t in ts]
    [t.join() for t in ts]
    assert len({id(g) for g in got}) == 1  # every thread sees the one published kernel


def test_forward_validation_errors():
    seen = {}

    def launch(tensors, symbols, stream):
        seen["called"] = True

    k = tl.compile(_spec("validate", launch), out_idx=[2], workspace_idx=[3])
    A = torch.zeros(4, 8, dtype=torch.int8)
    B = torch.zeros(8, 16, dtype=torch.int8)
    with pytest.raises(ValueError, match="Expected 2 inputs, got 1 with 4 params"):
        k(A)
    with pytest.raises(ValueError, match="Unsupported tensor type"):
        k(A, [1, 2])
    with pytest.raises(ValueError, match="Input tensor at index 1 must be contiguous"):
        k(A, torch.zeros(16, 8, dtype=torch.int8).t())
    with pytest.raises(ValueError, match="Buffer dtype mismatch for parameter A"):
        k(A.to(torch.int32), B)
    with pytest.raises(ValueError, match="Static shape mismatch for parameter B"):
        k(A, torch.zeros(8, 32, dtype=torch.int8))
    with pytest.raises(ValueError, match="Static shape mismatch for parameter A"):
        k(torch.zeros(4, 8, 1, dtype=torch.int8), B)
    # every check passed, but the tensors are on the host: there is no CPU implementation
    with pytest.raises(ValueError, match="Buffer device mismatch"):
        k(A, B)
    with pytest.raises(ValueError, match="Buffer device mismatch"):
        k(A, B, torch.zeros(3))  # surplus positionals are ignored, as in the reference
    assert "called" not in seen


def test_symbolic_dimension_is_resolved_from_the_inputs():
    k = ops.int8_gemm_kernel_corrected(64, 128)
    assert k.params[0].shape[0] == "M" and k.result_idx == [4] and k.workspace_idx == [5]
    sym = k._resolve([torch.zeros(24, 128, dtype=torch.int8), torch.zeros(64, 128, dtype=torch.int8)])
    assert sym == {"M": 24}


def test_cpu_wrappers_fail_loudly_without_a_gpu():
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    f = ops.dequant_gemm_fp16_wrapper(16, 64, 64, 128, 256, 64)
    with pytest.raises((RuntimeError, ValueError, AssertionError)):
        f(torch.zeros(16, 64, dtype=torch.float16), torch.zeros(64, 32, dtype=torch.uint8))
    with pytest.raises((RuntimeError, ValueError, AssertionError)):
        ops.torch_unpack_uint4_to_fp16(torch.zeros(4, 4, dtype=torch.uint8))


def test_profiler_module_surface():
    from tilelang_ascend_amd import profiler

    k = tl.compile(_spec("prof"), out_idx=[2], workspace_idx=[3])
    p = k.get_profiler()
    assert isinstance(p, profiler.Profiler)
    assert [q.name for q in p._get_params()] == ["A", "B"]
    assert [q.name for q in p._get_params(with_output=True)] == ["A", "B", "C"]
    assert profiler.TensorSupplyType.Auto.value == 7 and callable(profiler.do_bench)


def test_profiler_assert_consistent_compares_repeated_runs(monkeypatch):
    """The reference's race check (tilelang/profiler/__init__.py:188-205) on a stand-in kernel: equal runs pass, a run
    that differs in one bit fails, and the inputs of every run are the same tensors."""
    from tilelang_ascend_amd import profiler

    monkeypatch.setattr(torch.cuda, "synchronize", lambda *a, **k: None)

    class Fake:
        params, result_idx, workspace_idx = [], [], []

        def __init__(self, flaky_at=None):
            self.calls, self.flaky_at = 0, flaky_at

        def __call__(self, x):
            self.calls += 1
            out = x * 2
            if self.calls == self.flaky_at:
                out = out.clone()
                out.view(torch.int16)[3] ^= 1  # one mantissa bit: allclose would let it pass
            return out

    x = torch.arange(16, dtype=torch.float16)
    good = Fake()
    profiler.Profiler(good).assert_consistent(repeat=4, input_tensors=[x])
    assert good.calls == 5
    with pytest.raises(AssertionError, match="not consistent: run 3"):
        profiler.Profiler(Fake(flaky_at=3)).assert_consistent(repeat=4, input_tensors=[x])


def test_build_lock_is_exclusive_and_stale_libraries_are_detected(tmp_path, monkeypatch):
    """Two builders never run at once (advisory file lock), and a library whose build record names other sources
    than those on disk counts as stale; one without a record is taken as it is."""
    import fcntl
    import subprocess
    import sys

    from tilelang_ascend_amd import build

    monkeypatch.setattr(build, "LIB_DIR", str(tmp_path))
    monkeypatch.setattr(build, "LIB_PATH", str(tmp_path / "libtlq.so"))
    monkeypatch.setattr(build, "STAMP_PATH", str(tmp_path / "libtlq.fingerprint"))
    with build.build_lock():
        probe = ("import fcntl,sys\nf=open(sys.argv[1],'w')\n"
                 "try:\n fcntl.flock(f, fcntl.LOCK_EX|fcntl.LOCK_NB); print('free')\nexcept BlockingIOError:\n print('held')\n")
        out = subprocess.run([sys.executable, "-c", probe, str(tmp_path / ".build.lock")], capture_output=True, text=True)
        assert out.stdout.strip() == "held"
    with open(tmp_path / ".build.lock", "w") as f:
        fcntl.flock(f, fcntl.LOCK_EX | fcntl.LOCK_NB)  # released on leaving the context
    assert build.is_stale() and not build.is_current()  # no library
    (tmp_path / "libtlq.so").write_bytes(b"")
    assert not build.is_stale() and not build.is_current()  # no record: cannot be judged
    (tmp_path / "libtlq.fingerprint").write_text("0" * 64 + "\n")
    assert build.is_stale()
    (tmp_path / "libtlq.fingerprint").write_text(build.source_fingerprint() + "\n")
    assert not build.is_stale() and build.is_current()


def test_tile_choice_by_machine_fill():
    """128 x 128 or 256 x 256 output tiles: the choice follows how full each makes the machine (256 CUs without a GPU),
    the small tiles' fill weighted by their pace.  The table is what was measured faster on an MI355X."""
    from tilelang_ascend_amd import _abi

    tile = _abi.load().tlq_debug_gemm_tile
    if _abi.load().tlq_device_cu_count() not in (0, -1, 256):
        import pytest

        pytest.skip("table holds for 256 CUs")
    plain = {(1, 2048, 4096): 128, (1, 1536, 4096): 128, (1, 3072, 4096): 256, (1, 4096, 4096): 256, (1, 2048, 11008): 256,
             (1, 1024, 14336): 256, (1, 1024, 4096): 128, (1, 2560, 5120): 256, (1, 512, 14336): 128, (1, 768, 8192): 128,
             (8, 2048, 4096): 256, (3, 2048, 4096): 256, (2, 1024, 4096): 128, (1, 8192, 14336): 256, (1, 100, 4096): 128}
    for (b, m, n), want in plain.items():
        assert tile(b, m, n, 0) == want, (b, m, n)
    fused = {(1, 2048, 4096): 128, (1, 1536, 4096): 128, (1, 3072, 4096): 256, (1, 2048, 11008): 256, (1, 512, 14336): 128,
             (1, 1024, 14336): 256, (1, 4096, 4096): 256}
    for (b, m, n), want in fused.items():
        assert tile(b, m, n, 1) == want, (b, m, n)
