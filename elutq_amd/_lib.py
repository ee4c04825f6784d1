"""ctypes binding of libelutq_hip.so (the C ABI declared in include/elutq_hip.h).

The library is the only compute path: if it is missing or a symbol is absent this
module raises; there is no PyTorch or CPU fallback.
"""
from __future__ import annotations

import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libelutq_hip.so")

_vp, _ci, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/elutq_hip.h
SIGNATURES = {
    "elutq_version": (_ci, []),
    "elutq_status_string": (ctypes.c_char_p, [_ci]),
    "elutq_hlq_planes_bytes": (_sz, [_ci, _ci, _ci]),
    "elutq_hlq_scales_bytes": (_sz, [_ci, _ci, _ci, _ci]),
    "elutq_hlq_zeros_bytes": (_sz, [_ci, _ci, _ci]),
    "elutq_hlq_repack_host": (_ci, [_vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp, _vp, _vp]),
    "elutq_hlq_unpack_host": (_ci, [_vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp, _vp, _vp]),
    "elutq_hlq_workspace_bytes": (_sz, [_ci, _ci, _ci, _ci, _ci]),
    "elutq_hlq_workspace_init": (_ci, [_vp, _sz, _vp]),
    "elutq_hlq_gemv_f16": (_ci, [_vp] * 6 + [_ci] * 4 + [_vp, _sz, _vp]),
    "elutq_hlq_gemv_f16_tuned": (_ci, [_vp] * 6 + [_ci] * 4 + [_vp, _sz, _vp, _ci, _ci]),
    "elutq_hlq_gemv_int8lut_f16": (_ci, [_vp] * 6 + [_ci] * 4 + [_vp, _sz, _vp]),
    "elutq_hlq_gemv_fused_f16": (_ci, [_vp] * 6 + [_ci] * 4 + [_vp, _sz, _vp, _vp, _ci, _ci]),
    "elutq_hlq_gemv_slices": (_ci, [_ci] * 6),
    "elutq_hlq_gemv_fault_count": (_ci, [_ci]),
    "elutq_hlq_set_gemv_engine": (_ci, [_ci]),
    "elutq_hlq_get_gemv_engine": (_ci, []),
    "elutq_hlq_static_scratch_bytes": (_sz, []),
    "elutq_hlq_static_init": (_ci, []),
    "elutq_hlq_gemv_f16_static": (_ci, [_vp] * 6 + [_ci] * 4 + [_vp]),
    "elutq_hlq_gemv_accepts_slices": (_ci, [_ci] * 7),
    "elutq_decode_rope_attn_f16": (_ci, [_vp] * 5 + [_ci] * 4 + [ctypes.c_float, _vp]),
    "elutq_decode_rope_attn_split_f16": (_ci, [_vp] * 5 + [_ci] * 4 + [ctypes.c_float, _ci, _vp, _sz, _vp]),
    "elutq_decode_attn_workspace_bytes": (_sz, [_ci] * 3),
    "elutq_decode_rope_attn_sliced_f16": (_ci, [_vp, _ci, _ci, _vp, _vp, _vp, _vp] + [_ci] * 4 + [ctypes.c_float, _ci, _vp, _sz, _vp]),
    "elutq_decode_embed_f16": (_ci, [_vp] * 3 + [_ci, _ci, _vp]),
    "elutq_decode_rmsnorm_f16": (_ci, [_vp] * 3 + [_ci, ctypes.c_float, _vp]),
    "elutq_fp16_gemv_f16": (_ci, [_vp] * 4 + [_ci, _ci, _vp, ctypes.c_float, _vp]),
    "elutq_decode_argmax_f16": (_ci, [_vp, _ci, _vp, _vp, _vp]),
    "elutq_decode_argmax_ws_f16": (_ci, [_vp, _ci, _vp, _vp, _vp, _sz, _vp]),
    "elutq_hlq_gemv_group_workspace_bytes": (_sz, [_vp, _ci, _ci, _ci]),
    "elutq_hlq_gemv_group_create": (_ci, [_vp, _ci, _ci, _ci, _vp, _sz, _vp]),
    "elutq_hlq_gemv_group_run": (_ci, [_vp, _vp]),
    "elutq_hlq_gemv_group_destroy": (_ci, [_vp]),
    "elutq_hlq_gemm_f16": (_ci, [_vp] * 6 + [_ci] * 5 + [_vp, _sz, _vp]),
    "elutq_hlq_gemm_f16_tuned": (_ci, [_vp] * 6 + [_ci] * 5 + [_vp, _sz, _vp, _ci, _ci]),
    "elutq_hlq_dequant_f16": (_ci, [_vp] * 4 + [_ci] * 4 + [_vp]),
    "elutq_hlq_sparse_index_bytes": (_sz, [_ci, _ci]),
    "elutq_hlq_sparse_index_host": (_ci, [_vp, _ci, _ci, _ci, _ci, _vp]),
    "elutq_hlq_sparse_workspace_bytes": (_sz, [_ci] * 5),
    "elutq_hlq_sparse_gemv_f16": (_ci, [_vp] * 7 + [_ci] + [_vp] * 2 + [_ci] * 4 + [_vp, _sz, _vp]),
    "elutq_hlq_sparse_gemm_f16": (_ci, [_vp] * 7 + [_ci] + [_vp] * 2 + [_ci] * 5 + [_vp, _sz, _vp]),
    "elutq_hlq_sparse_gemv_fused_f16": (_ci, [_vp] * 7 + [_ci] + [_vp] * 2 + [_ci] * 4 + [_vp, _sz, _vp, _vp, _ci, _ci]),
    "elutq_hlq_sparse_dequant_add_f16": (_ci, [_vp] * 3 + [_ci, _vp] + [_ci] * 3 + [_vp]),
    "elutq_hlq_sparse_inline_bytes": (_sz, [_ci] * 4),
    "elutq_hlq_sparse_inline_host": (_ci, [_vp, _ci, _vp, _vp, _ci, _ci, _ci, _vp, _vp]),
    "elutq_hlq_sparse_gemv_inline_f16": (_ci, [_vp] * 5 + [_sz] + [_vp] * 2 + [_ci] * 4 + [_vp, _sz, _vp, _vp, _ci, _ci]),
}



class GemvFusion(ctypes.Structure):
    """struct elutq_gemv_fusion of include/elutq_hip.h."""
    _fields_ = [("prologue", ctypes.c_int), ("eps", ctypes.c_float),
                ("d_norm_weight", ctypes.c_void_p), ("d_residual", ctypes.c_void_p),
                ("d_slices_out", ctypes.c_void_p), ("d_slices_in", ctypes.c_void_p),
                ("n_slices_in", ctypes.c_int), ("d_x_out", ctypes.c_void_p),
                ("slices_out_bytes", ctypes.c_size_t), ("slices_in_bytes", ctypes.c_size_t)]


class GemvProblem(ctypes.Structure):
    """struct elutq_gemv_problem of include/elutq_hip.h."""
    _fields_ = [("d_planes", ctypes.c_void_p), ("d_scales", ctypes.c_void_p), ("d_zeros", ctypes.c_void_p),
                ("d_bias", ctypes.c_void_p), ("d_x", ctypes.c_void_p), ("d_y", ctypes.c_void_p),
                ("K", ctypes.c_int), ("N", ctypes.c_int)]


_lib = None


class ElutqError(RuntimeError):
    def __init__(self, status: int, where: str):
        self.status = status
        msg = lib().elutq_status_string(status).decode()
        super().__init__(f"{where}: {msg} (status {status})")


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m elutq_amd.build` "
                "(there is no fallback path)")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)          # AttributeError if the symbol is not exported
            fn.restype, fn.argtypes = res, args
        # ELUTQ_GEMV_ENGINE=lut|mfma|auto pins the batch-1 GEMV kernel for the process (tests, benchmarks)
        engine = os.environ.get("ELUTQ_GEMV_ENGINE", "").lower()
        if engine:
            if engine not in GEMV_ENGINES:
                raise RuntimeError(f"ELUTQ_GEMV_ENGINE must be one of {sorted(GEMV_ENGINES)}, not {engine!r}")
            handle.elutq_hlq_set_gemv_engine(GEMV_ENGINES[engine])
        _lib = handle
    return _lib


GEMV_ENGINES = {"auto": 0, "lut": 1, "mfma": 2}
# values of the `ksplit` tuning argument that name a kernel instead of a slice count (include/elutq_hip.h)
GEMV_NARROW16, GEMV_NARROW32, GEMV_WIDE = -16, -32, -64
ERR_SPARSE = -8        # ELUTQ_ERR_SPARSE: a block list that a form of the sparse extra plane cannot hold


def set_gemv_engine(name: str) -> None:
    """Which kernel the batch-1 GEMV entry points launch: "lut", "mfma" or "auto" (the default)."""
    check(lib().elutq_hlq_set_gemv_engine(GEMV_ENGINES[name]), "elutq_hlq_set_gemv_engine")


def check(status: int, where: str) -> None:
    if status != 0:
        raise ElutqError(status, where)
