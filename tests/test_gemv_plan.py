"""Launch geometry of the register-resident decode GEMV, computed on the host (tlq_debug_gemv_rows_plan): the
activations, scales and zero points a work-group keeps in LDS never exceed the 64 KB a kernel gets without asking for more,
every row is covered, and shapes whose staging data cannot fit are handed to the streaming kernel instead."""
import ctypes

import pytest

from tilelang_ascend_amd import _abi


def plan(batch, N, K, group, cus=256):
    out = (ctypes.c_int64 * 4)()
    rc = _abi.load().tlq_debug_gemv_rows_plan(batch, N, K, group, cus, ctypes.cast(out, ctypes.c_void_p))
    return rc, list(out)


@pytest.mark.parametrize("K", [64, 1024, 2048, 4096, 5120, 8192, 11008 - 11008 % 128, 14336, 16384])
@pytest.mark.parametrize("group", [32, 64, 128, 256])
@pytest.mark.parametrize("N", [1, 77, 4096, 11008, 14336, 49152, 128256, 1 << 20])
def test_lds_budget_and_coverage(N, K, group):
    if K % group:
        pytest.skip("group does not divide K")
    for batch in (1, 3, 24):
        rc, (rpb, blocks, lds, wpb) = plan(batch, N, K, group)
        assert rc in (0, 1)
        if rc == 0:
            continue
        groups = K // group
        assert lds == (K // 32) * 72 + rpb * groups * 4
        assert lds <= 64 * 1024, (N, K, group, lds)
        assert rpb % 4 == 0 and rpb >= 4 and rpb * blocks >= N and rpb * (blocks - 1) < N
        assert wpb * 64 >= K // 32  # one staging thread per activation chunk


def test_the_case_that_overflowed():
    # M = 1, N = 128256, K = 8192, group 128 once asked for 67584 bytes; K = 16384 for 86 KB
    for K in (8192, 16384):
        rc, (rpb, blocks, lds, _) = plan(1, 128256, K, 128)
        assert rc == 1 and lds <= 65536 and rpb * blocks >= 128256
    # K = 16384 with groups of 32: 512 groups per row, 36 KB of activations -- 12 rows per work-group still fit
    rc, (rpb, _, lds, wpb) = plan(1, 4096, 16384, 32)
    assert rc == 1 and lds <= 65536 and rpb >= wpb


def test_bad_arguments():
    assert plan(1, 16, 96, 48)[0] == -1   # group not a power of two
    assert plan(1, 16, 32768, 128)[0] == -1
    assert plan(0, 16, 4096, 128)[0] == -1
