"""Builds libelutq_hip.so in-tree with hipcc for gfx950.

    python -m elutq_amd.build            # compile every source (in parallel), link
    python -m elutq_amd.build --changed  # recompile only sources older than their object file
"""
from __future__ import annotations

import ctypes
import glob
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

_PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_PKG, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_PATH = os.path.join(_PKG, "libelutq_hip.so")
SOURCES = ["hlq_gemv.hip", "hlq_gemm.hip", "hlq_misc.hip", "hlq_sparse.hip", "decode_ops.hip", "hlq_repack.cpp",
           "hlq_static.hip", "hlq_gemv_mfma.hip", "hlq_gemv_narrow.hip", "fp16_gemv.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]
NOISE = "is not a recognized feature for this target"


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found (need ROCm with gfx950 support)")
    return exe


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if NOISE not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build(verbose: bool = False, force: bool = True, jobs: int = 6) -> str:
    """Compiles each source to an object file (up to `jobs` at a time) and links the shared library.
    force=False skips sources whose object file is newer than the source and every header."""
    srcs = [os.path.join(CSRC, s) for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    os.makedirs(OBJ_DIR, exist_ok=True)
    include = os.path.join(_PKG, "..", "include")
    headers = glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(include, "*.h"))
    newest_header = max(os.path.getmtime(h) for h in headers)
    todo, objs = [], []
    for src in srcs:
        obj = os.path.join(OBJ_DIR, os.path.basename(src) + ".o")
        objs.append(obj)
        if force or not os.path.exists(obj) or os.path.getmtime(obj) < max(os.path.getmtime(src), newest_header):
            todo.append((src, obj))
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        list(pool.map(lambda so: _run([hipcc(), *HIPCC_FLAGS, "-I", include, "-c", "-o", so[1], so[0]], verbose), todo))
    tmp = LIB_PATH + ".tmp"
    _run([hipcc(), "--offload-arch=gfx950", "-fPIC", "-shared", "-o", tmp, *objs], verbose)
    # A kernel whose host stub the compiler dropped links as an undefined symbol: load the library now
    # (all symbols resolved at once) rather than find out at the first call.
    try:
        ctypes.CDLL(tmp, mode=os.RTLD_NOW)
    except OSError as e:
        os.unlink(tmp)
        raise RuntimeError(f"the linked library does not load: {e}") from e
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True, force="--changed" not in sys.argv[1:]))
