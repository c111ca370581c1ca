"""The C-ABI shared library: it loads without a GPU, exports every symbol include/tlq.h (the operator boundary) and
include/tlq_debug.h (self-checks and tuning hooks) declare, with the declared argument lists, and rejects bad arguments
before touching a device."""
import ctypes
import os
import re

import pytest

from tilelang_ascend_amd import _abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tlq.h")
DEBUG_HEADER = os.path.join(ROOT, "include", "tlq_debug.h")

CTYPE = {"const void*": ctypes.c_void_p, "void*": ctypes.c_void_p, "int64_t": ctypes.c_int64, "int": ctypes.c_int,
         "float": ctypes.c_float, "const char*": ctypes.c_char_p}
RESTYPE = {"int": ctypes.c_int, "int64_t": ctypes.c_int64, "void": None, "const char*": ctypes.c_char_p}


def declared(headers=(HEADER, DEBUG_HEADER)):
    """name -> (return type, [argument types]) parsed from the header texts."""
    text = "\n".join(open(h).read() for h in headers)
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    out = {}
    for m in re.finditer(r"(const char\*|int64_t|int|void)\s+(tlq_\w+)\s*\(([^)]*)\)\s*;", text):
        ret, name, args = m.group(1), m.group(2), " ".join(m.group(3).split())
        types = []
        if args != "void":
            for a in args.split(","):
                a = a.strip()
                t = re.match(r"(const void\*|void\*|const char\*|int64_t|int|float)\s*\w+$", a)
                assert t, f"{name}: argument '{a}' is not a plain pointer / size / code"
                types.append(t.group(1))
        out[name] = (ret, types)
    return out


def test_header_declares_only_plain_c_types():
    d = declared()
    assert len(d) >= 15
    assert "torch" not in open(HEADER).read().lower().replace("torch_unpack", "").replace("torch_convert", "")


def test_the_operator_header_carries_no_test_or_tuning_hooks():
    ops = declared((HEADER,))
    assert ops and not [n for n in ops if n.startswith(("tlq_debug_", "tlq_tune_"))]
    dev = declared((DEBUG_HEADER,))
    assert dev and all(n.startswith(("tlq_debug_", "tlq_tune_")) for n in dev)


def test_library_exports_every_declared_symbol():
    lib = _abi.load()
    for name in declared():
        assert hasattr(lib, name), f"libtlq.so does not export {name}"
    assert lib.tlq_abi_version() == _abi.ABI_VERSION
    m = re.search(r"#define TLQ_ABI_VERSION (\d+)", open(HEADER).read())
    assert int(m.group(1)) == _abi.ABI_VERSION


def test_ctypes_signatures_match_the_header():
    d = declared()
    assert set(d) == set(_abi.SIGNATURES)
    for name, (ret, types) in d.items():
        res, args = _abi.SIGNATURES[name]
        assert res is RESTYPE[ret], name
        assert args == [CTYPE[t] for t in types], name


def test_enum_codes_match_the_header():
    text = open(HEADER).read()
    for name, val in (("TLQ_F16", _abi.F16), ("TLQ_BF16", _abi.BF16), ("TLQ_F32", _abi.F32), ("TLQ_I8", _abi.I8),
                      ("TLQ_I32", _abi.I32), ("TLQ_U4", _abi.U4), ("TLQ_S4_TWOS", _abi.S4_TWOS),
                      ("TLQ_S4_OFFSET8", _abi.S4_OFFSET8), ("TLQ_S4_OFFSET7", _abi.S4_OFFSET7), ("TLQ_B_KN", _abi.B_KN),
                      ("TLQ_B_NK", _abi.B_NK), ("TLQ_ALGO_AUTO", _abi.ALGO_AUTO), ("TLQ_ALGO_GEMV", _abi.ALGO_GEMV),
                      ("TLQ_ALGO_MFMA", _abi.ALGO_MFMA), ("TLQ_ALGO_SKINNY", _abi.ALGO_SKINNY),
                      ("TLQ_ALGO_TWO_PASS", _abi.ALGO_TWO_PASS)):
        m = re.search(rf"\b{name}\s*=\s*(\d+)", text)
        assert m and int(m.group(1)) == val, name


# Argument validation runs on the host before any launch, so it can be exercised without a GPU.
# The pointer values below are never dereferenced: every call is rejected.
FAKE = ctypes.c_void_p(0x1000)
ODD = ctypes.c_void_p(0x1004)
ODD2 = ctypes.c_void_p(0x1002)
NULL = ctypes.c_void_p(0)


def _rejected(rc, *needles):
    assert rc != 0
    msg = _abi.last_error()
    for n in needles:
        assert n in msg, msg
    with pytest.raises(RuntimeError):
        _abi.check(rc)


def test_rejects_bad_w4a16_arguments():
    lib = _abi.load()
    f = lib.tlq_gemm_w4a16
    _rejected(f(FAKE, FAKE, NULL, NULL, FAKE, 4, 64, 100, 32, 0.0, _abi.F16, _abi.F16, 0, NULL), "K=100", "multiple of 64")
    _rejected(f(FAKE, FAKE, NULL, NULL, FAKE, 4, 64, 128, 48, 0.0, _abi.F16, _abi.F16, 0, NULL), "group=48")
    _rejected(f(FAKE, FAKE, NULL, NULL, FAKE, 4, 64, 128, 32, 0.0, _abi.I8, _abi.F16, 0, NULL), "in_dtype")
    _rejected(f(FAKE, FAKE, NULL, NULL, FAKE, 4, 64, 128, 32, 0.0, _abi.F16, _abi.I32, 0, NULL), "out_dtype")
    _rejected(f(FAKE, FAKE, NULL, NULL, FAKE, 4, 64, 128, 32, 0.0, _abi.F16, _abi.F16, 7, NULL), "algo")
    _rejected(f(NULL, FAKE, NULL, NULL, FAKE, 4, 64, 128, 32, 0.0, _abi.F16, _abi.F16, 0, NULL), "null pointer")
    _rejected(f(ODD, FAKE, NULL, NULL, FAKE, 4, 64, 128, 32, 0.0, _abi.F16, _abi.F16, 0, NULL), "16-byte aligned")
    _rejected(f(FAKE, FAKE, NULL, NULL, FAKE, -1, 64, 128, 32, 0.0, _abi.F16, _abi.F16, 0, NULL), "bad shape")
    _rejected(f(FAKE, FAKE, NULL, NULL, FAKE, 32, 64, 128, 32, 0.0, _abi.F16, _abi.F16, _abi.ALGO_GEMV, NULL), "M <= 16")
    _rejected(f(FAKE, FAKE, NULL, NULL, FAKE, 32, 66, 128, 32, 0.0, _abi.F16, _abi.F16, _abi.ALGO_MFMA, NULL), "N % 4")
    _rejected(f(FAKE, FAKE, NULL, NULL, FAKE, 32, 64, 192, 96, 0.0, _abi.F16, _abi.F16, _abi.ALGO_MFMA, NULL), "power of two")
    _rejected(f(FAKE, FAKE, NULL, NULL, FAKE, 1 << 20, 64, 4096, 128, 0.0, _abi.F16, _abi.F16, _abi.ALGO_MFMA, NULL),
              "4 GiB")
    # empty problems are accepted and launch nothing
    assert f(NULL, NULL, NULL, NULL, NULL, 0, 64, 128, 32, 0.0, _abi.F16, _abi.F16, 0, NULL) == 0
    assert f(NULL, NULL, NULL, NULL, NULL, 4, 0, 128, 32, 0.0, _abi.F16, _abi.F16, 0, NULL) == 0


def test_rejects_bad_integer_gemm_arguments():
    lib = _abi.load()
    _rejected(lib.tlq_gemm_i8(FAKE, FAKE, FAKE, 1, 8, 16, 24, _abi.B_KN, NULL), "K=24")
    _rejected(lib.tlq_gemm_i8(FAKE, FAKE, FAKE, 1, 8, 20, 32, _abi.B_KN, NULL), "N=20")
    _rejected(lib.tlq_gemm_i8(FAKE, FAKE, FAKE, 1, 8, 16, 32, 5, NULL), "b_layout")
    _rejected(lib.tlq_gemm_i8(FAKE, FAKE, FAKE, -2, 8, 16, 32, _abi.B_KN, NULL), "batch")
    _rejected(lib.tlq_gemm_w4a8(FAKE, FAKE, FAKE, 8, 16, 48, _abi.S4_TWOS, NULL), "K=48")
    _rejected(lib.tlq_gemm_w4a8(FAKE, FAKE, FAKE, 8, 16, 64, 9, NULL), "sign_mode")
    _rejected(lib.tlq_gemm_w8a8(FAKE, FAKE, FAKE, FAKE, FAKE, 1, 8, 16, 32, 3, _abi.B_KN, _abi.F16, NULL), "n_scale_b=3")
    _rejected(lib.tlq_gemm_w8a8(FAKE, FAKE, FAKE, FAKE, FAKE, 1, 8, 16, 32, 16, _abi.B_KN, _abi.I32, NULL), "out_dtype")
    _rejected(lib.tlq_gemm_w8a8(FAKE, FAKE, ODD2, FAKE, FAKE, 1, 8, 16, 32, 16, _abi.B_KN, _abi.F16, NULL), "misaligned")
    _rejected(lib.tlq_gemm_f16(FAKE, FAKE, FAKE, 8, 16, 12, _abi.F16, _abi.F16, _abi.B_KN, NULL), "K=12")
    _rejected(lib.tlq_gemv_w4a16_batched(FAKE, FAKE, NULL, NULL, FAKE, 70000, 1, 64, 128, 32, 0.0, 0, 0, NULL), "batch=70000")
    assert lib.tlq_gemm_i8(NULL, NULL, NULL, 0, 8, 16, 32, _abi.B_KN, NULL) == 0


def test_rejects_bad_unpack_arguments():
    lib = _abi.load()
    _rejected(lib.tlq_unpack_int4(FAKE, FAKE, 4, 7, _abi.I8, _abi.U4, NULL), "K")
    _rejected(lib.tlq_unpack_int4(FAKE, FAKE, 4, 8, _abi.I32, _abi.U4, NULL), "out_dtype")
    _rejected(lib.tlq_unpack_int4(NULL, FAKE, 4, 8, _abi.I8, _abi.U4, NULL), "null")
    _rejected(lib.tlq_dequant_w4(FAKE, NULL, NULL, FAKE, 4, 64, 24, 0.0, _abi.F16, NULL), "group")
    _rejected(lib.tlq_dequant_w4(FAKE, NULL, NULL, FAKE, 4, 64, 32, 0.0, _abi.I8, NULL), "dtype")


def test_error_string_is_thread_local():
    import threading

    lib = _abi.load()
    lib.tlq_gemm_i8(FAKE, FAKE, FAKE, 1, 8, 16, 24, _abi.B_KN, NULL)
    seen = {}

    def other():
        seen["before"] = _abi.last_error()
        lib.tlq_gemm_w4a8(FAKE, FAKE, FAKE, 8, 16, 48, _abi.S4_TWOS, NULL)
        seen["after"] = _abi.last_error()

    t = threading.Thread(target=other)
    t.start()
    t.join()
    assert seen["before"] == "" and "tlq_gemm_w4a8" in seen["after"]
    assert "tlq_gemm_i8" in _abi.last_error()


def test_rejects_bad_arguments_of_the_widened_entry_points():
    """Activation quantiser, repacker, plain GEMV / split-K and the workspace entry point validate before any GPU call."""
    lib = _abi.load()
    _rejected(lib.tlq_act_quant_i8(FAKE, FAKE, FAKE, 4, 0, _abi.BF16, 0, NULL), "rows are empty")
    _rejected(lib.tlq_act_quant_i8(FAKE, FAKE, FAKE, 4, 64, _abi.I8, 0, NULL), "in_dtype")
    _rejected(lib.tlq_act_quant_i8(NULL, FAKE, FAKE, 4, 64, _abi.BF16, 0, NULL), "null pointer")
    _rejected(lib.tlq_act_quant_i8(FAKE, FAKE, ODD2, 4, 64, _abi.BF16, 0, NULL), "misaligned")
    _rejected(lib.tlq_pack_int4(FAKE, FAKE, 4, 12, 0, NULL), "K=12")
    _rejected(lib.tlq_pack_int4(FAKE, FAKE, 4, 16, 3, NULL), "interleave")
    _rejected(lib.tlq_pack_int4(ODD, FAKE, 4, 16, 0, NULL), "aligned")
    _rejected(lib.tlq_quantize_sym4(FAKE, FAKE, FAKE, 4, 64, 12, _abi.F16, NULL), "group=12")
    _rejected(lib.tlq_quantize_sym4(FAKE, FAKE, FAKE, 4, 64, 32, _abi.F32, NULL), "dtype")
    _rejected(lib.tlq_gemv(FAKE, FAKE, FAKE, 8, 12, _abi.F16, _abi.F16, NULL), "K=12")
    _rejected(lib.tlq_gemv(FAKE, FAKE, FAKE, 8, 64, _abi.I8, _abi.F16, NULL), "dtype")
    _rejected(lib.tlq_gemv(ODD, FAKE, FAKE, 8, 64, _abi.F16, _abi.F16, NULL), "16-byte aligned")
    _rejected(lib.tlq_gemm_w4a16_ws(FAKE, FAKE, NULL, NULL, FAKE, 512, 64, 128, 32, 0.0, _abi.F16, _abi.F16, _abi.ALGO_TWO_PASS,
                                    NULL, 0, NULL), "two-pass path needs", "workspace")
    _rejected(lib.tlq_gemm_w4a16_ws(FAKE, FAKE, NULL, NULL, FAKE, 512, 64, 128, 32, 0.0, _abi.F16, _abi.F16, 10, NULL, 0, NULL),
              "bad algo")
    # empty problems launch nothing
    assert lib.tlq_act_quant_i8(NULL, NULL, NULL, 0, 64, _abi.BF16, 0, NULL) == 0
    assert lib.tlq_gemv(NULL, NULL, NULL, 0, 64, _abi.F16, _abi.F16, NULL) == 0


def test_workspace_size_rules():
    """tlq_w4a16_workspace_bytes: nothing for decode shapes, fp32 partial sums of the K slices for small and middle M,
    a dequantised copy of the weights (N * K 16-bit values) for large M -- and, from M = 256 on, where the plain GEMM of
    the two passes has few output tiles, room for its K slices behind that copy (which of the kernels runs depends on the
    group size, so the size covers both)."""
    lib = _abi.load()
    ws = lib.tlq_w4a16_workspace_bytes
    assert ws(1, 11008, 4096) == 0 and ws(16, 14336, 4096) == 0
    assert ws(4096, 4096, 4096) == 4096 * 4096 * 2
    assert ws(8192, 14336, 4096) == 14336 * 4096 * 2
    def row_values(N, K):  # rows whose length is no power of two: room for one scale / zero point per row written out per group
        if K & (K - 1) == 0:
            return 0
        g = min(K & -K, 1024)
        return 2 * ((N * (K // g) * 2 + 15) // 16 * 16) + 16

    for M, N, K in ((64, 14336, 4096), (200, 4096, 4096), (255, 4096, 14336)):
        b = ws(M, N, K) - row_values(N, K)
        assert b > 0 and b % (M * N * 4) == 0, (M, N, K, b)
        split = b // (M * N * 4)
        assert 2 <= split <= 16, (M, N, K, split)  # room for the most K slices any kernel and group size may cut
    for M, N, K in ((256, 4096, 14336), (512, 4096, 4096), (1024, 4096, 14336)):
        b = ws(M, N, K)
        assert b >= N * K * 2 + lib.tlq_f16_workspace_bytes(1, M, N, K) and b >= 2 * M * N * 4, (M, N, K, b)
        assert lib.tlq_f16_workspace_bytes(1, M, N, K) > 0
    assert ws(1024, 14336, 4096) == 14336 * 4096 * 2  # many output tiles already: no K slices, two passes
    assert ws(64, 0, 4096) == 0 and ws(64, 128, 0) == 0
    # a weight-row count that is no multiple of four, more than 32 activation rows: what the multiple of 16 below asks for, then
    # its packed result (sized for fp32 outputs)
    a16 = lambda b: (b + 15) // 16 * 16  # noqa: E731
    assert ws(100, 1001, 512) == a16(ws(100, 992, 512)) + a16(100 * 992 * 4)
    assert ws(300, 50257, 4096) == a16(ws(300, 50256, 4096)) + a16(300 * 50256 * 4)
    assert ws(32, 1001, 512) == ws(32, 1000, 512) and ws(100, 1004, 512) == 0
    assert ws(100, 7, 512) == 0 and ws(1000, 15, 4096) == 0  # fewer than 16 weight rows: the last-rows kernel alone, no packed result
    assert ws(600, 1036, 1024) == a16(ws(600, 1024, 1024)) + a16(600 * 1024 * 4)  # (above 512 rows: multiples of four that are no multiples of eight, too)


def test_tuning_hooks_are_per_thread():
    """A value set through a tlq_tune_* hook belongs to the calling thread: launches prepared on another thread keep the
    automatic choice.  Observed through the workspace rule, which follows the number of K slices that
    tlq_tune_w4a16_split forces."""
    import threading

    from tilelang_ascend_amd import _abi

    lib = _abi.load()
    M, N, K = 200, 4096, 4096
    auto = lib.tlq_w4a16_workspace_bytes(M, N, K)
    assert auto == 8 * M * N * 4
    lib.tlq_tune_w4a16_split(16)
    try:
        here = lib.tlq_w4a16_workspace_bytes(M, N, K)
        seen = []
        t = threading.Thread(target=lambda: seen.append(lib.tlq_w4a16_workspace_bytes(M, N, K)))
        t.start()
        t.join()
    finally:
        lib.tlq_tune_w4a16_split(0)
    assert here == 16 * M * N * 4, "the override is not seen on the thread that set it"
    assert seen == [auto], "another thread saw this thread's override"
    assert lib.tlq_w4a16_workspace_bytes(M, N, K) == auto
