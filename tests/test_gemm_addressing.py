"""Host-side walk of the MFMA GEMM kernels' address arithmetic (csrc/gemm_addr.h through
tlq_debug_check_gemm_addressing / tlq_debug_check_slots_schedule): the functions the kernels use for their
global offsets, LDS offsets and for the five-slot issue / wait order are evaluated on the
CPU for every tile, thread and stage of a launch and compared with the buffer extents.  The shapes are those of
the GPU comparison test of the two GEMM main loops plus ragged and very short cases.
"""
import pytest

from tilelang_ascend_amd import _abi


def _ok(rc):
    assert rc == 0, _abi.last_error()


# (rows, K in 16-bit values): the activation (rows = M) and [N, K] weight (rows = N) operands of the 16-bit GEMMs
SHAPES_16 = [(256, 256, 64), (300, 520, 192), (1000, 1288, 4160), (4096, 4096, 4096), (260, 264, 96), (2048, 2304, 72),
             (2900, 2900, 64), (2900, 2824, 128), (3000, 2820, 192), (2816, 3072, 320), (2820, 2900, 72),
             (1, 8, 8), (7, 16, 24), (255, 257 * 8, 64), (513, 1000, 136)]
W8A8 = [(1, 256, 256, 128), (2, 300, 528, 384), (1, 2048, 4096, 4096), (3, 512, 272, 640), (1, 260, 512, 144),
        (1, 1, 16, 16), (1, 33, 48, 272)]


@pytest.mark.parametrize("tile,threads", [(256, 512), (128, 256)])
def test_row_operands_of_the_16_bit_gemms(tile, threads):
    lib = _abi.load()
    for M, N, K in SHAPES_16:
        for rows in (M, N):
            _ok(lib.tlq_debug_check_gemm_addressing(0, rows, K * 2, tile, threads))


def test_int8_operands():
    lib = _abi.load()
    for _, M, N, K in W8A8:
        for tile, threads in ((256, 512), (128, 256), (32, 256)):
            _ok(lib.tlq_debug_check_gemm_addressing(0, M, K, tile, threads))        # activations [M, K]
        for tile, threads in ((256, 512), (128, 256)):
            _ok(lib.tlq_debug_check_gemm_addressing(0, N, K, tile, threads))        # weights [N, K]
            _ok(lib.tlq_debug_check_gemm_addressing(1, K, N, tile, threads))        # weights [K, N]
        _ok(lib.tlq_debug_check_gemm_addressing(1, K, N, 128, 256))                 # the 32-row kernel's weights


def test_the_walker_rejects_what_it_should():
    lib = _abi.load()
    assert lib.tlq_debug_check_gemm_addressing(0, 256, 256, 250, 512) != 0      # tile rows not a multiple of 8
    assert lib.tlq_debug_check_gemm_addressing(0, 256, 256, 64, 1024) != 0      # fewer load instructions than wavefronts
    assert lib.tlq_debug_check_gemm_addressing(0, 1 << 20, 1 << 13, 256, 512) != 0  # 8 GiB operand: 32-bit offsets
    assert lib.tlq_debug_check_gemm_addressing(1, 128, 24, 256, 512) != 0       # N not a multiple of 16
    assert lib.tlq_debug_check_gemm_addressing(3, 128, 128, 256, 512) != 0
    assert "bad source kind" in _abi.last_error()
    assert lib.tlq_debug_check_gemm_addressing(2, 128, 100, 256, 512) != 0      # 16-bit [K, N]: N not a multiple of 8
    assert lib.tlq_debug_check_gemm_addressing(2, 128, 128, 64, 256) != 0       # ... tiles of 128 or 256 columns only
    assert lib.tlq_debug_check_gemm_addressing(2, 128, 128, 256, 768) != 0      # ... 32 load instructions do not split over 12 wavefronts


def test_16_bit_kn_operand_of_the_five_slot_kernel():
    """[K, N] weights of the plain 16-bit GEMM (the reference's fp16_gemm layout, example_dequant_gemm_fine_grained.py:60-115):
    direct loads inside the matrix for full, ragged and narrow column tiles, every LDS cell written once, the transposing
    operand reads on the right rows and columns, and no bank met twice by a half-wavefront."""
    lib = _abi.load()
    for K, N in ((64, 8), (64, 256), (128, 264), (256, 1000), (4096, 4096), (1024, 11008), (192, 40), (72, 264), (328, 4104), (1, 8), (40, 72)):
        _ok(lib.tlq_debug_check_gemm_addressing(2, K, N, 256, 512))   # five-slot and two-stage kernels, 256 x 256 tiles
        _ok(lib.tlq_debug_check_gemm_addressing(2, K, N, 128, 256))   # two-stage kernel, 128 x 128 tiles


def test_five_slot_schedule():
    """Every tile is waited for and published by a barrier before it is multiplied, and no load overwrites a tile
    that some wavefront may still read: for 1..64 stages, with the four load instructions per wavefront and tile that
    the kernel's waits count.  With fewer loads per tile the same waits would leave two tiles in flight, and the check
    says so; with more they wait for more than they need to."""
    lib = _abi.load()
    for stages in range(1, 65):
        _ok(lib.tlq_debug_check_slots_schedule(stages, 4))
    assert lib.tlq_debug_check_slots_schedule(8, 2) != 0
    assert "before its loads were waited for" in _abi.last_error()
    _ok(lib.tlq_debug_check_slots_schedule(8, 8))



@pytest.mark.parametrize("tm,depth", [(2, 5), (4, 4), (6, 3), (8, 3)])
def test_streaming_kernel_addressing(tm, depth):
    """Streaming W4A16 kernel: every direct load stays inside the packed weights / the activations (rows past the
    matrices are clamped), lands on the LDS cell its operand read expects, and the ring never multiplies a step before
    its loads were waited for nor reloads a slot that may still be read."""
    lib = _abi.load()
    for M, N, K in [(17, 256, 128), (64, 14336, 4096), (100, 4096, 14336), (33, 1000, 256), (512, 260, 1152), (128, 8, 128)]:
        _ok(lib.tlq_debug_check_stream_addressing(M, N, K, tm, depth))
    assert lib.tlq_debug_check_stream_addressing(64, 256, 100, tm, depth) != 0   # K not a multiple of 128
    assert lib.tlq_debug_check_stream_addressing(64, 1 << 22, 4096, tm, depth) != 0  # packed weights of 8 GiB
