"""Builds libtlq.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python -m tilelang_ascend_amd.build [--force]

Mirrors the role of the reference's LibraryGenerator.compile_lib
(tilelang/jit/adapter/libgen.py:106-232: write source, shell out to the device compiler,
produce a .so that ctypes loads), except that the kernels are fixed sources rather than
generated ones, so there is one library for all operators.
"""
from __future__ import annotations

import contextlib
import fcntl
import hashlib
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
CSRC_DIR = os.path.join(PKG_DIR, "csrc")
INCLUDE_DIR = os.path.join(REPO_DIR, "include")
LIB_DIR = os.path.join(PKG_DIR, "lib")
OBJ_DIR = os.path.join(LIB_DIR, "obj")
LIB_PATH = os.path.join(LIB_DIR, "libtlq.so")

ARCH = "gfx950"
SOURCES = [
    "abi.hip",
    "unpack_dequant.hip",
    "decode_i4.hip",
    "decode_lowbit.hip",
    "act_quant.hip",
    "repack.hip",
    "gemv_plain.hip",
    "gemv_w4a16.hip",
    "gemm_w4a16.hip",
    "gemm_w4a16_stream.hip",
    "gemm_w4a16_panel.hip",
    "gemm_w4a16_panel256.hip",
    "gemm_w4a16_panelm.hip",
    "w4a16_choice.hip",
    "gemm_w4a16_decode.hip",
    "gemm_int8.hip",
    "gemm_f16.hip",
    "gemm_api.hip",
    "gemm_addr_check.hip",
    "gemm_w4a16_noalloc.hip",
]
# packed-fp32 VALU forms are disabled on purpose (some have produced silent wrong results on
# this hardware pool); hipcc's host pass warns that it does not know the feature.
HIPCC_FLAGS = [
    "-O3",
    "-std=c++17",
    "-fPIC",
    f"--offload-arch={ARCH}",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-ffp-contract=off",
    "-Wno-unused-command-line-argument",
    "-Wno-unknown-warning-option",
    f"-I{INCLUDE_DIR}",
    f"-I{CSRC_DIR}",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: cannot build libtlq.so")


def source_fingerprint() -> str:
    """sha256 over kernel sources, headers and flags -- the analogue of the reference's kernel
    cache key (tilelang/cache/kernel_cache.py:71-117: hash of source + target + options)."""
    h = hashlib.sha256()
    h.update(" ".join(HIPCC_FLAGS).encode())
    names = sorted(os.listdir(CSRC_DIR)) + ["../../include/tlq.h", "../../include/tlq_debug.h"]
    for name in names:
        path = os.path.join(CSRC_DIR, name)
        if os.path.isfile(path):
            h.update(name.encode())
            with open(path, "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def _compile_one(src: str, verbose: bool) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc_path(), *HIPCC_FLAGS, "-c", os.path.join(CSRC_DIR, src), "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"Compilation Failed! {' '.join(cmd)}\n{res.stdout}")
    noise = ("packed-fp32-ops", "is not a recognized feature")
    out = "\n".join(l for l in res.stdout.splitlines() if not any(n in l for n in noise))
    if verbose and out.strip():
        print(out)
    return obj


STAMP_PATH = os.path.join(LIB_DIR, "libtlq.fingerprint")


def built_fingerprint():
    """Fingerprint the library on disk was built from (None when there is no record)."""
    try:
        with open(STAMP_PATH) as f:
            return f.read().strip() or None
    except OSError:
        return None


def is_current() -> bool:
    return os.path.exists(LIB_PATH) and built_fingerprint() == source_fingerprint()


def is_stale() -> bool:
    """True when the library is absent, or carries a build record that names other sources than those on disk.
    A library without a record (copied on its own) cannot be judged and is taken as it is."""
    if not os.path.exists(LIB_PATH):
        return True
    fp = built_fingerprint()
    return fp is not None and fp != source_fingerprint()


@contextlib.contextmanager
def build_lock():
    """Exclusive advisory lock on lib/.build.lock: two processes (pytest workers, a test run next to a benchmark)
    never compile into the same object directory or replace the library under each other.  The reference
    serialises its kernel cache the same way (tilelang/cache/kernel_cache.py:119-160, a lock around save / load)."""
    os.makedirs(LIB_DIR, exist_ok=True)
    with open(os.path.join(LIB_DIR, ".build.lock"), "w") as f:
        fcntl.flock(f, fcntl.LOCK_EX)
        try:
            yield
        finally:
            fcntl.flock(f, fcntl.LOCK_UN)


def build_library(force: bool = True, verbose: bool = False, jobs: int = 6) -> str:
    """Compile every kernel source for gfx950 and link libtlq.so.  With force=False an
    up-to-date library (matching fingerprint) is reused.  Holds the build lock throughout; a process that waited
    for another one's build finds the library current and (force=False) returns at once."""
    with build_lock():
        return _build_locked(force, verbose, jobs)


def _build_locked(force: bool, verbose: bool, jobs: int) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    stamp = STAMP_PATH
    fp = source_fingerprint()
    if not force and is_current():
        return LIB_PATH
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC_DIR, s))]
    missing = sorted(set(SOURCES) - set(srcs))
    if missing:
        raise RuntimeError(f"kernel sources missing: {missing}")
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile_one(s, verbose), srcs))
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc_path(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", tmp, *objs]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"Compilation Failed! {' '.join(cmd)}\n{res.stdout}")
    os.replace(tmp, LIB_PATH)
    with open(stamp, "w") as f:
        f.write(fp + "\n")
    return LIB_PATH


if __name__ == "__main__":
    path = build_library(force="--force" in sys.argv or True, verbose=True)
    print("built", path)
