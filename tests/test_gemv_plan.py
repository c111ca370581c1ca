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


def ring_plan(N, K, group, cus=256, M=1):
    out = (ctypes.c_int64 * 6)()
    rc = _abi.load().tlq_debug_gemv_ring_plan(M, N, K, group, cus, ctypes.cast(out, ctypes.c_void_p))
    return rc, list(out)


@pytest.mark.parametrize("K", [256, 1024, 2048, 2080, 4096])
@pytest.mark.parametrize("group", [32, 64, 128, 256])
@pytest.mark.parametrize("N", [1, 16, 77, 1000, 4096, 11008, 14336, 32000, 128256])
def test_ring_kernel_geometry_and_addressing(N, K, group):
    """The ring kernel's launch, walked on the host before it ever runs: every direct load inside its tensor and its LDS
    area, every staging piece and every row covered once, no slot overwritten before it was read and no row read under
    the kernel's wait counts while one of its loads may still be in flight."""
    if K % group:
        pytest.skip("group does not divide K")
    lib = _abi.load()
    for cus, M in ((256, 1), (64, 1), (8, 1), (256, 2), (64, 2)):
        rc, (iters, depth, waves, rpb, blocks, lds) = ring_plan(N, K, group, cus, M)
        groups = K // group
        if groups % 8 or rc == 0:
            assert rc == 0  # 16-byte staging pieces need a multiple of 8 groups per row; or LDS does not hold the rows' scales
            continue
        assert rc == 1
        assert iters == (2 if K > 2048 else 1) and waves == 16 and 1 <= depth <= (3 if M == 1 else 2)
        assert rpb >= waves and rpb * blocks >= N and rpb * (blocks - 1) < N and (blocks <= cus or rpb == waves)
        assert lds <= 160 * 1024
        assert lib.tlq_debug_check_gemv_ring_addressing(M, N, K, group, rpb, waves, depth) == 0, _abi.last_error()


def test_ring_walker_catches_a_wrong_launch():
    lib = _abi.load()
    # rows per work-group whose scales overflow the 160 KB of LDS
    assert lib.tlq_debug_check_gemv_ring_addressing(1, 11008, 4096, 32, 4096, 16, 3) != 0
    assert "LDS" in _abi.last_error()
    # a group count that is not a multiple of 8
    assert lib.tlq_debug_check_gemv_ring_addressing(1, 1024, 1024, 256, 16, 16, 1) != 0
    assert lib.tlq_debug_check_gemv_ring_addressing(3, 1024, 1024, 32, 16, 16, 1) != 0  # at most two activation rows
    assert ring_plan(1024, 1024, 32, M=3)[0] == 0
    assert ring_plan(1024, 1024, 256)[0] == 0
    assert ring_plan(1024, 8192, 128)[0] == 0  # rows longer than 4096 values stay with the register-resident kernel
    assert ring_plan(1024, 1024, 96)[0] == -1
