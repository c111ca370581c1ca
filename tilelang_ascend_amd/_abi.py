"""ctypes binding of libtlq.so (the C ABI declared in include/tlq.h).

Plays the part of the reference's ``lib.call(*void_ptrs, [dyn ints], stream)`` step
(tilelang/jit/adapter/cython/cython_wrapper.pyx:189-197): raw device pointers first, sizes
after, the stream last.  There is no CPU fallback: if the library cannot be loaded the
operators raise.
"""
from __future__ import annotations

import contextlib
import ctypes
import os
import threading

from . import build as _build

# type codes of include/tlq.h
F16, BF16, F32, I8, I32 = 0, 1, 2, 3, 4
U4, S4_TWOS, S4_OFFSET8, S4_OFFSET7 = 0, 1, 2, 3
B_KN, B_NK = 0, 1
W_PLAIN, W_INTERLEAVED_F16 = 0, 1
ALGO_AUTO, ALGO_GEMV, ALGO_MFMA, ALGO_SKINNY, ALGO_TWO_PASS, ALGO_STREAM, ALGO_DECODE, ALGO_PANEL, ALGO_PANEL256, ALGO_PANELM = 0, 1, 2, 3, 4, 5, 6, 7, 8, 9
ABI_VERSION = 1

_vp, _i64, _int, _f32, _cstr = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_char_p

# name -> (restype, argtypes); kept in step with include/tlq.h (a test compares the two)
SIGNATURES = {
    "tlq_abi_version": (_int, []),
    "tlq_last_error": (ctypes.c_char_p, []),
    "tlq_device_cu_count": (_int, []),
    "tlq_unpack_int4": (_int, [_vp, _vp, _i64, _i64, _int, _int, _vp]),
    "tlq_dequant_w4": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _f32, _int, _vp]),
    "tlq_decode_i4_interleaved": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _int, _int, _int, _vp]),
    "tlq_decode_i4_interleaved_offset": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _int, _int, _vp]),
    "tlq_decode_lowbit_interleaved": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _int, _int, _int, _int, _vp]),
    "tlq_gemm_w4a16": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _f32, _int, _int, _int, _vp]),
    "tlq_gemv_w4a16_batched": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _f32, _int, _int, _vp]),
    "tlq_gemm_f16": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _int, _int, _int, _vp]),
    "tlq_gemm_f16_batched": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _vp]),
    "tlq_gemm_i8": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "tlq_gemm_w4a8": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "tlq_gemm_w4a8_ws": (_int, [_vp, _vp, _vp, _i64, _vp, _i64, _i64, _i64, _int, _vp]),
    "tlq_gemm_w8a8": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int, _int, _vp]),
    "tlq_gemm_w8a8_ws": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, _vp]),
    "tlq_w4a16_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "tlq_w4a16_workspace_bytes_min": (_i64, [_i64, _i64, _i64]),
    "tlq_w4a16_workspace_bytes_for": (_i64, [_i64, _i64, _i64, _int]),
    "tlq_w4a16_choice_set": (_int, [_i64, _i64, _i64, _i64, _int, _int]),
    "tlq_w4a16_choice_get": (_int, [_i64, _i64, _i64, _i64, _int]),
    "tlq_w4a16_choice_clear": (None, []),
    "tlq_w4a16_choice_count": (_i64, []),
    "tlq_w4a16_choice_save": (_int, [_cstr]),
    "tlq_w4a16_choice_load": (_int, [_cstr]),
    "tlq_gemm_w4a16_ws": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _f32, _int, _int, _int, _vp, _i64, _vp]),
    "tlq_gemm_w4a16_layout_ws": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _f32, _int, _int, _int, _int, _vp, _i64, _vp]),
    "tlq_dequant_w4_layout": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _f32, _int, _int, _vp]),
    "tlq_gemm_w4a16_noalloc_init": (_int, []),
    "tlq_gemm_w4a16_noalloc": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _f32, _int, _int, _int, _vp]),
    "tlq_gemm_f16_splitk": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _vp]),
    "tlq_gemv": (_int, [_vp, _vp, _vp, _i64, _i64, _int, _int, _vp]),
    "tlq_pack_int4": (_int, [_vp, _vp, _i64, _i64, _int, _vp]),
    "tlq_quantize_sym4": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "tlq_act_quant_i8": (_int, [_vp, _vp, _vp, _i64, _i64, _int, _int, _vp]),
    "tlq_debug_check_gemm_addressing": (_int, [_int, _i64, _i64, _int, _int]),
    "tlq_debug_check_slots_schedule": (_int, [_int, _int]),
    "tlq_debug_check_stream_addressing": (_int, [_i64, _i64, _i64, _int, _int]),
    "tlq_debug_check_decode_addressing": (_int, [_i64, _i64, _i64, _i64, _int, _int, _int, _int]),
    "tlq_debug_decode_plan": (_int, [_i64, _i64, _i64, _i64, _int, _vp]),
    "tlq_debug_launch_log": (None, [_int]),
    "tlq_debug_launch_log_text": (ctypes.c_char_p, []),
    "tlq_debug_check_panel_addressing": (_int, [_i64, _i64, _i64, _i64, _int]),
    "tlq_debug_panel_plan": (_int, [_i64, _i64, _i64, _i64, _int, _vp]),
    "tlq_debug_check_panel256_addressing": (_int, [_i64, _i64, _i64, _i64, _int]),
    "tlq_debug_panel256_plan": (_int, [_i64, _i64, _i64, _i64, _int, _vp]),
    "tlq_debug_check_panel256_schedule": (_int, [_int, _int, _int]),
    "tlq_debug_panelm_plan": (_int, [_i64, _i64, _i64, _i64, _int, _vp]),
    "tlq_debug_check_panelm_addressing": (_int, [_i64, _i64, _i64, _i64, _int, _int]),
    "tlq_debug_check_panelm_schedule": (_int, [_int, _int, _int, _int, _int]),
    "tlq_tune_w4a16_decode": (None, [_int]),
    "tlq_debug_gemv_rows_plan": (_int, [_i64, _i64, _i64, _i64, _int, _vp]),
    "tlq_tune_gemv": (None, [_int, _int]),
    "tlq_tune_gemv_unroll": (None, [_int]),
    "tlq_tune_gemv_depth": (None, [_int]),
    "tlq_tune_gemv_ring": (None, [_int]),
    "tlq_debug_gemv_ring_plan": (_int, [_i64, _i64, _i64, _i64, _int, _vp]),
    "tlq_debug_check_gemv_ring_addressing": (_int, [_i64, _i64, _i64, _i64, _int, _int, _int]),
    "tlq_tune_gemm_band": (None, [_int]),
    "tlq_tune_gemm_slots": (None, [_int]),
    "tlq_tune_gemm_tile": (None, [_int]),
    "tlq_debug_gemm_tile": (_int, [_i64, _i64, _i64, _int]),
    "tlq_tune_w4a16_stream": (None, [_int]),
    "tlq_tune_w4a16_stream_slice": (None, [_int]),
    "tlq_tune_w4a16_panel": (None, [_int]),
    "tlq_tune_w4a16_panel_slice": (None, [_int]),
    "tlq_tune_w4a16_panelm_rows": (None, [_int]),
    "tlq_tune_w4a16_tile": (None, [_int]),
    "tlq_tune_w4a16_split": (None, [_int]),
    "tlq_tune_w4a16_skinny": (None, [_int, _int]),
    "tlq_tune_i8_tile": (None, [_int]),
    "tlq_tune_i8_split": (None, [_int]),
    "tlq_tune_w4a8_ws": (None, [_int]),
    "tlq_tune_f16_split": (None, [_int]),
    "tlq_debug_f16_split": (_int, [_i64, _i64, _i64]),
    "tlq_f16_workspace_bytes": (_i64, [_i64, _i64, _i64, _i64]),
    "tlq_gemm_f16_ws": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int, _int, _int, _vp]),
    "tlq_debug_i8_split": (_int, [_i64, _i64, _i64, _int]),
    "tlq_w8a8_workspace_bytes": (_i64, [_i64, _i64, _i64, _i64]),
}

_lock = threading.Lock()
_lib = None
_build_failure = None


def library_path() -> str:
    return os.environ.get("TLQ_LIBRARY", _build.LIB_PATH)


def load():
    """Load libtlq.so once per process (mutex; the reference guards its library cache the same
    way, tilelang/jit/adapter/cython/adapter.py:79-98).  Builds it when it is absent or was built from other
    sources than those on disk (fingerprint record next to the library) and hipcc is available; otherwise raises --
    there is no other implementation to fall back to."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = library_path()
        # a library built from other sources than the ones on disk is never loaded: rebuild it (under the build
        # lock, so concurrent processes compile once), or say so when that is impossible
        if path == _build.LIB_PATH and _build.is_stale():
            state = "not found" if not os.path.exists(path) else "older than the kernel sources"
            global _build_failure
            if _build_failure is not None:  # one attempt per process: sources that do not compile fail every caller at once
                raise RuntimeError(f"libtlq.so at {path} is {state} and could not be built ({_build_failure})")
            try:
                path = _build.build_library(force=False)
            except Exception as e:  # noqa: BLE001
                _build_failure = e
                raise RuntimeError(
                    f"libtlq.so at {path} is {state} and could not be built ({e}); "
                    "run `python -m tilelang_ascend_amd.build`"
                ) from e
        elif not os.path.exists(path):
            raise RuntimeError(f"libtlq.so not found at {path}")
        lib = ctypes.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        if lib.tlq_abi_version() != ABI_VERSION:
            raise RuntimeError(f"libtlq.so ABI version {lib.tlq_abi_version()} != expected {ABI_VERSION}")
        _lib = lib
    return _lib


def last_error() -> str:
    msg = load().tlq_last_error()
    return msg.decode() if msg else ""


def check(rc: int) -> None:
    """Non-zero return -> RuntimeError carrying the library's message."""
    if rc != 0:
        raise RuntimeError(last_error() or f"libtlq call failed with code {rc}")


def ptr(t) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


_tuning_lock = threading.RLock()


@contextlib.contextmanager
def tuning(w4a16_tile: int = 0, i8_tile: int = 0, gemv: tuple = None, skinny: tuple = None):
    """Applies tiling choices to the launches made inside the block, then restores the automatic
    choice.  The hooks set thread-local values that are only read on the host while a launch is being set up
    (asynchronous execution is not affected): another thread that launches at the same time keeps the automatic
    choice.  The lock only keeps nested uses on one thread orderly."""
    lib = load()
    active = bool(w4a16_tile or i8_tile or gemv or skinny)
    if not active:
        yield
        return
    with _tuning_lock:
        try:
            if w4a16_tile:
                lib.tlq_tune_w4a16_tile(int(w4a16_tile))
            if i8_tile:
                lib.tlq_tune_i8_tile(int(i8_tile))
            if gemv:
                rows, waves, blocks_per_cu, depth = (tuple(gemv) + (0, 0, 0, 0))[:4]
                lib.tlq_tune_gemv(int(rows), int(waves))
                lib.tlq_tune_gemv_unroll(int(blocks_per_cu))
                lib.tlq_tune_gemv_depth(int(depth))
            if skinny:
                lib.tlq_tune_w4a16_skinny(int(skinny[0]), int(skinny[1]))
            yield
        finally:
            if w4a16_tile:
                lib.tlq_tune_w4a16_tile(0)
            if i8_tile:
                lib.tlq_tune_i8_tile(0)
            if gemv:
                lib.tlq_tune_gemv(0, 0)
                lib.tlq_tune_gemv_unroll(0)
                lib.tlq_tune_gemv_depth(0)
            if skinny:
                lib.tlq_tune_w4a16_skinny(0, 0)


def scratch(nbytes: int, device, stream: int):
    """A per-call workspace of `nbytes` bytes from torch's caching allocator, safe to hand to a kernel launched on the raw
    stream `stream`: the allocator orders reuse of a block by the stream that was current when it was allocated, so when
    the launch stream is another one the block is recorded on it (otherwise the block could be handed out again, on the
    current stream, while the kernel still writes it).  None for nbytes == 0."""
    import torch

    if not nbytes:
        return None
    ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
    if stream and stream != torch.cuda.current_stream(ws.device).cuda_stream:
        ws.record_stream(torch.cuda.ExternalStream(stream, device=ws.device))
    return ws
