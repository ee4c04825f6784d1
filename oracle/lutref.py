"""ctypes binding of oracle/liblutref.so (the C restatement).  TEST INFRASTRUCTURE ONLY.

build() compiles it with the Makefile beside this file; load() returns the
library or raises.  The wrappers take/return NumPy arrays in the export layout
and do the reference's loader permutation (elutq_ref_rearrange) themselves, so a
caller sees the same interface as oracle.hlq_oracle.gemv_fp16_chain.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liblutref.so")
_lib = None


def build(force: bool = False) -> str:
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-s", "-C", _HERE, "liblutref.so"], check=True)
    return _SO


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_SO):
        raise RuntimeError(f"{_SO} is not built; run `make -C oracle` (or __graft_entry__.build())")
    lib = ctypes.CDLL(_SO)
    vp, ci = ctypes.c_void_p, ctypes.c_int
    lib.elutq_ref_rearrange.argtypes = [ci, ci, ci, ci, ci, vp, vp, vp, vp, vp, vp]
    lib.elutq_ref_rearrange.restype = ci
    lib.elutq_ref_lut.argtypes = [ci, vp, vp]
    lib.elutq_ref_lut.restype = None
    lib.elutq_ref_gemv.argtypes = [ci, ci, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci]
    lib.elutq_ref_gemv.restype = ci
    lib.elutq_ref_gemm.argtypes = [ci, ci, ci, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci]
    lib.elutq_ref_gemm.restype = ci
    lib.elutq_ref_rearrange_sparse.argtypes = [ci, ci, ci, ci, vp, ctypes.c_uint32, vp, vp, vp, vp, vp, vp]
    lib.elutq_ref_rearrange_sparse.restype = ci
    lib.elutq_ref_gemv_sparse.argtypes = [ci, ci, vp, vp, vp, vp, vp, vp, vp, ctypes.c_uint32, ci, ci, ci, ci]
    lib.elutq_ref_gemv_sparse.restype = ci
    lib.elutq_ref_gemv_fast.argtypes = [ci, ci, vp, vp, vp, vp, vp, vp, ci, ci, ci]
    lib.elutq_ref_gemv_fast.restype = ci
    _lib = lib
    return lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


class RefWeight:
    """Export arrays permuted once by the reference's loader for `threads` threads
    (the layout is only valid for that thread count, as in the reference)."""

    def __init__(self, w_quant, w_scale, w_zero, group: int, threads: int, bias=None):
        lib = load()
        w_quant = np.ascontiguousarray(w_quant, dtype=np.uint8)
        w_scale = np.ascontiguousarray(w_scale, dtype=np.float16)
        w_zero = np.ascontiguousarray(w_zero, dtype=np.float16)
        self.bits, self.n, k8 = w_quant.shape
        self.k, self.group, self.threads = k8 * 8, int(group), int(threads)
        chunk = (self.n + threads - 1) // threads
        if chunk % 32 or self.n % 32:
            raise ValueError("reference layout needs 32-channel tiles in every thread chunk")
        self.weight = np.empty(w_quant.size, dtype=np.uint8)
        self.scale = np.empty(w_scale.size, dtype=np.float16)
        self.zero = np.empty(w_zero.size, dtype=np.float16)
        ok = lib.elutq_ref_rearrange(self.n, self.k, self.bits, self.group, self.threads,
                                     _p(w_quant), _p(w_scale), _p(w_zero),
                                     _p(self.weight), _p(self.scale), _p(self.zero))
        if ok != 1:
            raise RuntimeError("elutq_ref_rearrange: element count mismatch")
        self.bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.float16)

    def gemv(self, x, fused: bool = True) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float16).reshape(-1)
        assert x.size == self.k
        y = np.empty(self.n, dtype=np.float16)
        rc = load().elutq_ref_gemv(self.k, self.n, _p(x), _p(y), _p(self.weight), _p(self.scale),
                                   _p(self.zero), _p(self.bias), self.group, self.bits,
                                   self.threads, int(fused))
        if rc:
            raise MemoryError("elutq_ref_gemv")
        return y

    def gemm(self, x, fused: bool = True) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float16)
        m = x.shape[0]
        assert x.shape[1] == self.k
        y = np.empty((m, self.n), dtype=np.float16)
        rc = load().elutq_ref_gemm(m, self.k, self.n, _p(x), _p(y), _p(self.weight), _p(self.scale),
                                   _p(self.zero), _p(self.bias), self.group, self.bits,
                                   self.threads, int(fused))
        if rc:
            raise MemoryError("elutq_ref_gemm")
        return y

    def gemv_fast(self, x) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float16).reshape(-1)
        y = np.empty(self.n, dtype=np.float16)
        rc = load().elutq_ref_gemv_fast(self.k, self.n, _p(x), _p(y), _p(self.weight), _p(self.scale),
                                        _p(self.zero), _p(self.bias), self.group, self.bits, self.threads)
        if rc:
            raise MemoryError("elutq_ref_gemv_fast")
        return y


class RefSparseWeight:
    """A use_sparse layer after the reference's loader: `w_quant_bytes` / `w_scale_bytes` /
    `mask_bytes` are the contents of w_quant.bin / w_scale.bin / weight_mask.bin (dense part
    followed by the block data), `base_bits` the number of dense planes."""

    def __init__(self, w_quant_bytes: bytes, w_scale_bytes: bytes, w_zero, mask_bytes: bytes,
                 k: int, n: int, base_bits: int, group: int, bias=None):
        lib = load()
        if n % 32:
            raise ValueError("reference layout needs 32-channel tiles")
        self.k, self.n, self.bits, self.group = int(k), int(n), int(base_bits) + 1, int(group)
        wq = np.frombuffer(w_quant_bytes, dtype=np.uint8).copy()
        ws = np.frombuffer(w_scale_bytes, dtype=np.float16).copy()
        wz = np.ascontiguousarray(w_zero, dtype=np.float16)
        self.mask = np.frombuffer(mask_bytes, dtype=np.uint32).copy()
        self.weight, self.scale, self.zero = np.empty_like(wq), np.empty_like(ws), np.empty(wz.size, np.float16)
        ok = lib.elutq_ref_rearrange_sparse(self.n, self.k, self.bits, self.group, _p(self.mask), self.mask.size,
                                            _p(wq), _p(ws), _p(wz), _p(self.weight), _p(self.scale), _p(self.zero))
        if ok != 1:
            raise RuntimeError("elutq_ref_rearrange_sparse: element count mismatch")
        self.bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.float16)

    def gemv(self, x, threads: int = 1, fused: bool = True) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float16).reshape(-1)
        assert x.size == self.k
        chunk = (self.n + threads - 1) // threads
        if chunk % 32:
            raise ValueError("reference layout needs 32-channel tiles in every thread chunk")
        y = np.empty(self.n, dtype=np.float16)
        rc = load().elutq_ref_gemv_sparse(self.k, self.n, _p(x), _p(y), _p(self.weight), _p(self.scale),
                                          _p(self.zero), _p(self.bias), _p(self.mask), self.mask.size,
                                          self.group, self.bits, threads, int(fused))
        if rc:
            raise MemoryError("elutq_ref_gemv_sparse")
        return y


def lut(x) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float16).reshape(-1)
    out = np.empty((x.size // 4, 16), dtype=np.float16)
    load().elutq_ref_lut(x.size, _p(x), _p(out))
    return out
