"""HLQLinear: the quantized-linear module of the HLQ path on MI355X.

On the Python side the reference has no quantized module: GPTQ/HLQ.py:173 writes the
dequantized weight back into ``nn.Linear`` and the forward is ``x @ W_deq.T + bias``.
HLQLinear keeps that ``nn.Linear`` surface (``in_features``, ``out_features``, optional
``bias``, ``forward(x[..., K]) -> [..., N]``) but holds the packed planes / scales / zeros
of the export files and runs the HIP LUT kernels through the C ABI, as the C++ runtime's
``arm_gemm(m, k, n, input, output, temp, weight_tensor*, ...)`` does on the CPU
(C++/ops/include/arm/arm_gemm.h:4-14).
"""
from __future__ import annotations

import ctypes
import os

import numpy as np
import torch
from torch import nn

from . import _lib
from .export_io import (ExportedLinear, SparseBlocks, densify_sparse, is_repacked_dir, read_export_dir,
                        read_repacked_dir, read_repacked_sparse)

_workspaces: dict = {}


def _workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    """One zero-initialised scratch buffer per (device, stream); calls on a stream are
    ordered, which is what the kernels' arrival counters need."""
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.zeros(max(nbytes, 1 << 21), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


def repack_export_arrays(w_quant, w_scale, w_zero, group: int):
    """Export-layout NumPy arrays -> (planes, scales, zeros) uint8 NumPy arrays in the
    kernel layout (host-side permutation done by the library)."""
    L = _lib.lib()
    w_quant = np.ascontiguousarray(w_quant, dtype=np.uint8)
    w_scale = np.ascontiguousarray(w_scale, dtype=np.float16)
    w_zero = np.ascontiguousarray(w_zero, dtype=np.float16)
    bits, n, k8 = w_quant.shape
    k = k8 * 8
    if w_scale.shape != (bits, n, k // group) or w_zero.shape != (n, k // group):
        raise ValueError("w_scale / w_zero shapes do not match w_quant and the group size")
    planes = np.empty(L.elutq_hlq_planes_bytes(k, n, bits), dtype=np.uint8)
    scales = np.empty(L.elutq_hlq_scales_bytes(k, n, bits, group), dtype=np.uint8)
    zeros = np.empty(L.elutq_hlq_zeros_bytes(k, n, group), dtype=np.uint8)
    if planes.size == 0 or scales.size == 0:
        raise ValueError(f"unsupported HLQ shape K={k} N={n} bits={bits} group={group} "
                         "(need K a multiple of 128 -- or of 64 at group 64 --, bits 1..4, group 64 or 128)")
    vp = ctypes.c_void_p
    _lib.check(L.elutq_hlq_repack_host(w_quant.ctypes.data_as(vp), w_scale.ctypes.data_as(vp),
                                       w_zero.ctypes.data_as(vp), k, n, bits, group,
                                       planes.ctypes.data_as(vp), scales.ctypes.data_as(vp),
                                       zeros.ctypes.data_as(vp)), "elutq_hlq_repack_host")
    return planes, scales, zeros


def unpack_to_export_arrays(planes, scales, zeros, k: int, n: int, bits: int, group: int):
    """Inverse of repack_export_arrays."""
    L = _lib.lib()
    vp = ctypes.c_void_p
    planes = np.ascontiguousarray(planes, dtype=np.uint8)
    scales = np.ascontiguousarray(scales, dtype=np.uint8)
    zeros = np.ascontiguousarray(zeros, dtype=np.uint8)
    w_quant = np.empty((bits, n, k // 8), dtype=np.uint8)
    w_scale = np.empty((bits, n, k // group), dtype=np.float16)
    w_zero = np.empty((n, k // group), dtype=np.float16)
    _lib.check(L.elutq_hlq_unpack_host(planes.ctypes.data_as(vp), scales.ctypes.data_as(vp),
                                       zeros.ctypes.data_as(vp), k, n, bits, group,
                                       w_quant.ctypes.data_as(vp), w_scale.ctypes.data_as(vp),
                                       w_zero.ctypes.data_as(vp)), "elutq_hlq_unpack_host")
    return w_quant, w_scale, w_zero


def sparse_inline(mask, blocks, scales, k: int, n: int, group: int) -> np.ndarray | None:
    """The inline form of a sparse extra plane (elutq_hlq_sparse_inline_host): what the batch-1 GEMV needs to look
    the blocks up inside its own launch.  None where the block list does not fit that form (blocks off the grid of
    the quantization groups, or two on one cell): such a plane runs as a launch of its own."""
    L = _lib.lib()
    mask = np.ascontiguousarray(mask, dtype=np.uint32).reshape(-1)
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    scales = np.ascontiguousarray(scales, dtype=np.float16)
    out = np.zeros(L.elutq_hlq_sparse_inline_bytes(k, n, group, mask.size // 2), dtype=np.uint8)
    used = ctypes.c_size_t(0)
    vp = ctypes.c_void_p
    rc = L.elutq_hlq_sparse_inline_host(mask.ctypes.data_as(vp), mask.size, blocks.ctypes.data_as(vp), scales.ctypes.data_as(vp),
                                        k, n, group, out.ctypes.data_as(vp), ctypes.byref(used))
    if rc == _lib.ERR_SPARSE:
        return None
    _lib.check(rc, "elutq_hlq_sparse_inline_host")
    return out[:used.value].copy()


def sparse_index(mask, k: int, n: int, group: int) -> np.ndarray:
    """(channel start, k start) pairs of a sparse extra plane -> the int32 index the kernels read
    (elutq_hlq_sparse_index_host; raises on a malformed list)."""
    L = _lib.lib()
    mask = np.ascontiguousarray(mask, dtype=np.uint32).reshape(-1)
    index = np.zeros(L.elutq_hlq_sparse_index_bytes(n, mask.size // 2) // 4, dtype=np.int32)
    vp = ctypes.c_void_p
    _lib.check(L.elutq_hlq_sparse_index_host(mask.ctypes.data_as(vp), mask.size, k, n, group,
                                             index.ctypes.data_as(vp)), "elutq_hlq_sparse_index_host")
    return index


class HLQLinear(nn.Module):
    """``nn.Linear``-shaped module over HLQ-packed weights (fp16 activations).

    `sparse`: optional block-sparse extra plane of a ``use_sparse`` export as device tensors
    (blocks uint8 [nblk, 32, G/8], scales fp16 [nblk, 32], index int32 from `sparse_index`);
    `bits` counts the dense planes only, as ``base_bit`` does in the export's json."""

    use_sparse_inline = True    # batch-1 calls look a sparse extra plane up inside the dense launch where its blocks allow it

    def __init__(self, in_features: int, out_features: int, bits: int, group_size: int,
                 planes: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor,
                 bias: torch.Tensor | None = None, sparse: tuple | None = None):
        super().__init__()
        self.in_features, self.out_features = int(in_features), int(out_features)
        self.bits, self.group_size = int(bits), int(group_size)
        self.register_buffer("planes", planes)
        self.register_buffer("scales", scales)
        self.register_buffer("zeros", zeros)
        self.register_buffer("bias", bias)
        sp_blocks, sp_scales, sp_index = sparse if sparse is not None else (None, None, None)
        self.register_buffer("sparse_blocks", sp_blocks)
        self.register_buffer("sparse_scales", sp_scales)
        self.register_buffer("sparse_index", sp_index)
        self.sparse_count = 0 if sp_scales is None else int(sp_scales.shape[0])
        if sparse is not None:
            want = _lib.lib().elutq_hlq_sparse_index_bytes(self.out_features, self.sparse_count)
            if (sp_index.dtype != torch.int32 or sp_index.numel() * 4 != want or sp_scales.dtype != torch.float16
                    or tuple(sp_scales.shape) != (self.sparse_count, 32) or sp_blocks.dtype != torch.uint8
                    or sp_blocks.numel() != self.sparse_count * 32 * self.group_size // 8):
                raise ValueError("sparse buffers do not match the layer: need blocks uint8 [nblk, 32, G/8], "
                                 "scales fp16 [nblk, 32] and the int32 index of sparse_index()")
        # the inline form of the plane, where its blocks fit it: batch-1 calls then take one launch (the blocks are
        # looked up in the dense GEMV's own tables) instead of two; `use_sparse_inline = False` keeps the two launches
        self.register_buffer("sparse_inline", None)
        if self.sparse_count and self.bits <= 3:
            form = sparse_inline(self.sparse_pairs(), sp_blocks.cpu().numpy(), sp_scales.cpu().numpy(), self.in_features,
                                 self.out_features, self.group_size)
            if form is not None:
                self.sparse_inline = torch.from_numpy(form).to(sp_blocks.device)
        self._ws_bytes = _lib.lib().elutq_hlq_workspace_bytes(self.in_features, self.out_features,
                                                              self.bits, self.group_size, 1)
        if self._ws_bytes == 0:
            raise ValueError(f"unsupported HLQ shape K={in_features} N={out_features} bits={bits} "
                             f"group={group_size} (need K a multiple of 128 -- or of 64 at group 64 --, bits 1..4, group 64 or 128)")
        self._ws_cache: dict = {}
        self.ksplit, self.waves = 0, 0      # 0 = library default; set for tuning

    def sparse_pairs(self) -> np.ndarray:
        """uint32 [nblk, 2]: the (channel start, k start) pairs of the sparse extra plane's blocks, in list order
        (the contents of weight_mask.bin), read back from the index the kernels use."""
        tiles = (self.out_features + 31) // 32
        idx = self.sparse_index.cpu().numpy()
        counts = np.diff(idx[:tiles + 1])
        return np.stack([np.repeat(np.arange(tiles, dtype=np.int64) * 32, counts),
                         idx[tiles + 1:tiles + 1 + self.sparse_count]], 1).astype(np.uint32)

    def _ws_bytes_for(self, m: int) -> int:
        key = 64 if m > 32 else 32
        if key not in self._ws_cache:
            self._ws_cache[key] = _lib.lib().elutq_hlq_workspace_bytes(
                self.in_features, self.out_features, self.bits, self.group_size, key)
        return self._ws_cache[key]

    # -- construction ------------------------------------------------------------------
    @classmethod
    def from_export_arrays(cls, w_quant, w_scale, w_zero, group_size: int, bias=None,
                           device="cuda", sparse: SparseBlocks | None = None, sparse_mode: str = "auto") -> "HLQLinear":
        """`sparse_mode` says how a block-sparse extra plane is held: "dense" writes it out as one more
        dense plane (scale 0 where no block exists: the same W, every kernel and every fusion applies, at
        the price of a whole plane of memory); "blocks" keeps the file form (two launches per call, no fused
        or grouped launch); "auto" = "dense" where the plane fits that form (export_io.densify_sparse),
        else "blocks".  On this GPU a launch costs more than the plane's bytes, hence the default."""
        if sparse_mode not in ("auto", "dense", "blocks"):
            raise ValueError('sparse_mode must be "auto", "dense" or "blocks"')
        if sparse is not None and sparse_mode != "blocks":
            dense = densify_sparse(w_quant, w_scale, sparse, group_size)
            if dense is not None:
                (w_quant, w_scale), sparse = dense, None
            elif sparse_mode == "dense":
                raise ValueError("the sparse extra plane cannot be written as a dense plane (more than four planes, "
                                 "a block off the group grid, or two blocks on one tile and group)")
        planes, scales, zeros = repack_export_arrays(w_quant, w_scale, w_zero, group_size)
        bits, n, k8 = np.asarray(w_quant).shape
        dev = torch.device(device)
        b = None if bias is None else torch.from_numpy(np.ascontiguousarray(bias, dtype=np.float16)).to(dev)
        return cls(k8 * 8, n, bits, group_size, torch.from_numpy(planes).to(dev),
                   torch.from_numpy(scales).to(dev), torch.from_numpy(zeros).to(dev), b,
                   cls._sparse_to_device(sparse, k8 * 8, n, group_size, dev))

    @staticmethod
    def _sparse_to_device(sparse: SparseBlocks | None, k: int, n: int, group: int, dev):
        if sparse is None:
            return None
        index = sparse_index(sparse.mask, k, n, group)
        blocks = np.ascontiguousarray(sparse.blocks, dtype=np.uint8)
        scale = np.ascontiguousarray(sparse.scale, dtype=np.float16).reshape(-1, 32)
        if blocks.size != scale.shape[0] * 32 * group // 8 or 2 * scale.shape[0] != np.asarray(sparse.mask).size:
            raise ValueError("sparse blocks / scales / mask disagree about the number of blocks")
        return (torch.from_numpy(blocks.reshape(-1, 32, group // 8).copy()).to(dev), torch.from_numpy(scale.copy()).to(dev),
                torch.from_numpy(index).to(dev))

    @classmethod
    def from_export(cls, e: ExportedLinear, device="cuda", sparse_mode: str = "auto") -> "HLQLinear":
        return cls.from_export_arrays(e.w_quant, e.w_scale, e.w_zero, e.group, e.bias, device, e.sparse, sparse_mode)

    @classmethod
    def from_export_dir(cls, path: str, device="cuda", group_size: int | None = None,
                        sparse_mode: str = "auto") -> "HLQLinear":
        """A linear directory of the reference's export, or the same after `python -m elutq_amd.repack`
        (which has settled how a sparse extra plane is held: `sparse_mode` applies to export directories)."""
        if is_repacked_dir(path):
            return cls.from_repacked_dir(path, device)
        return cls.from_export(read_export_dir(path, group_size), device, sparse_mode)

    @classmethod
    def from_repacked_dir(cls, path: str, device="cuda") -> "HLQLinear":
        k, n, bits, group, planes, scales, zeros, bias = read_repacked_dir(path)
        L = _lib.lib()
        want = (L.elutq_hlq_planes_bytes(k, n, bits), L.elutq_hlq_scales_bytes(k, n, bits, group),
                L.elutq_hlq_zeros_bytes(k, n, group))
        if 0 in want or (planes.size, scales.size, zeros.size) != want:
            raise ValueError(f"{path}: buffer sizes {(planes.size, scales.size, zeros.size)} do not match "
                             f"K={k} N={n} bits={bits} group={group} (expected {want})")
        dev = torch.device(device)
        b = None if bias is None else torch.from_numpy(bias).to(dev)
        return cls(k, n, bits, group, torch.from_numpy(planes).to(dev), torch.from_numpy(scales).to(dev),
                   torch.from_numpy(zeros).to(dev), b,
                   cls._sparse_to_device(read_repacked_sparse(path), k, n, group, dev))

    def with_bits(self, bits: int) -> "HLQLinear":
        """The same layer with `bits` planes: the added planes are all zero with scale 0, so W is unchanged.
        Lets layers of different depth share a launch (q|k|v where only one of them carries an extra plane)."""
        if bits == self.bits:
            return self
        if bits < self.bits or bits > 4:
            raise ValueError(f"cannot turn a {self.bits}-plane layer into a {bits}-plane one")
        ncb = (self.out_features + 63) // 64
        add = bits - self.bits

        def widen(buf: torch.Tensor, unit_bytes: int) -> torch.Tensor:      # [ncb][units][planes][64 * unit_bytes]
            v = buf.view(ncb, -1, self.bits, 64 * unit_bytes)
            z = torch.zeros(ncb, v.shape[1], add, 64 * unit_bytes, dtype=buf.dtype, device=buf.device)
            return torch.cat([v, z], 2).reshape(-1)

        sparse = (self.sparse_blocks, self.sparse_scales, self.sparse_index) if self.sparse_count else None
        return HLQLinear(self.in_features, self.out_features, bits, self.group_size, widen(self.planes, 16),
                         widen(self.scales, 4), self.zeros, self.bias, sparse)

    # -- compute -----------------------------------------------------------------------
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if x.shape[-1] != self.in_features:
            raise ValueError(f"expected last dim {self.in_features}, got {tuple(x.shape)}")
        if not x.is_cuda:
            raise RuntimeError("HLQLinear runs on the GPU only (there is no CPU path)")
        in_dtype = x.dtype
        x2 = x.reshape(-1, self.in_features)
        if x2.dtype != torch.float16:
            x2 = x2.to(torch.float16)
        x2 = x2.contiguous()
        m = x2.shape[0]
        y = torch.empty((m, self.out_features), dtype=torch.float16, device=x.device)
        if m:
            L = _lib.lib()
            if self.sparse_count:
                need = L.elutq_hlq_sparse_workspace_bytes(self.in_features, self.out_features, self.bits,
                                                          self.group_size, m)
            else:
                need = self._ws_bytes if m == 1 else self._ws_bytes_for(m)
            ws = _workspace(x.device, need)
            stream = torch.cuda.current_stream(x.device).cuda_stream
            bias = self.bias.data_ptr() if self.bias is not None else None
            if m == 1 and self._inline():
                rc = L.elutq_hlq_sparse_gemv_inline_f16(self.planes.data_ptr(), self.scales.data_ptr(), self.zeros.data_ptr(),
                                                        bias, self.sparse_inline.data_ptr(), self.sparse_inline.numel(), x2.data_ptr(), y.data_ptr(),
                                                        self.in_features, self.out_features, self.bits, self.group_size,
                                                        ws.data_ptr(), ws.numel(), stream, None, self.ksplit, self.waves)
                _lib.check(rc, "elutq_hlq_sparse_gemv_inline_f16")
            elif self.sparse_count:
                rc = L.elutq_hlq_sparse_gemm_f16(self.planes.data_ptr(), self.scales.data_ptr(), self.zeros.data_ptr(),
                                                 bias, self.sparse_blocks.data_ptr(), self.sparse_scales.data_ptr(),
                                                 self.sparse_index.data_ptr(), self.sparse_count, x2.data_ptr(),
                                                 y.data_ptr(), m, self.in_features, self.out_features, self.bits,
                                                 self.group_size, ws.data_ptr(), ws.numel(), stream)
                _lib.check(rc, "elutq_hlq_sparse_gemm_f16")
            elif m == 1:
                rc = L.elutq_hlq_gemv_f16_tuned(self.planes.data_ptr(), self.scales.data_ptr(), self.zeros.data_ptr(),
                                                bias, x2.data_ptr(), y.data_ptr(), self.in_features,
                                                self.out_features, self.bits, self.group_size,
                                                ws.data_ptr(), ws.numel(), stream, self.ksplit, self.waves)
                _lib.check(rc, "elutq_hlq_gemv_f16")
            else:
                rc = L.elutq_hlq_gemm_f16(self.planes.data_ptr(), self.scales.data_ptr(), self.zeros.data_ptr(),
                                          bias, x2.data_ptr(), y.data_ptr(), m, self.in_features,
                                          self.out_features, self.bits, self.group_size,
                                          ws.data_ptr(), ws.numel(), stream)
                _lib.check(rc, "elutq_hlq_gemm_f16")
        y = y.reshape(*x.shape[:-1], self.out_features)
        return y if in_dtype == torch.float16 else y.to(in_dtype)

    def _inline(self) -> bool:
        """Whether batch-1 calls look the sparse extra plane up inside the dense launch."""
        return bool(self.sparse_count) and self.sparse_inline is not None and self.use_sparse_inline

    @property
    def sparse_own_launch(self) -> bool:
        """A sparse extra plane that runs as a launch of its own in front of the dense one (such a layer neither
        takes nor leaves K slices)."""
        return bool(self.sparse_count) and not self._inline()

    def gemv_int8lut(self, x: torch.Tensor) -> torch.Tensor:
        """Batch-1 GEMV with the lookup tables quantized to int8 per group, as the reference's int8-LUT variant
        quantizes them (elutq_hlq_gemv_int8lut_f16; arm_gemv.cpp:4-34, arm_t_mac_kernal.cpp:15-93): lossy."""
        if self.sparse_count:
            raise NotImplementedError("the int8-LUT GEMV takes dense layers only")
        if x.dtype != torch.float16 or x.numel() != self.in_features or not x.is_cuda:
            raise ValueError("x must be fp16 [in_features] on the GPU")
        x = x.contiguous()
        y = torch.empty((1, self.out_features), dtype=torch.float16, device=x.device)
        ws = _workspace(x.device, self._ws_bytes)
        rc = _lib.lib().elutq_hlq_gemv_int8lut_f16(
            self.planes.data_ptr(), self.scales.data_ptr(), self.zeros.data_ptr(),
            self.bias.data_ptr() if self.bias is not None else None, x.data_ptr(), y.data_ptr(), self.in_features,
            self.out_features, self.bits, self.group_size, ws.data_ptr(), ws.numel(),
            torch.cuda.current_stream(x.device).cuda_stream)
        _lib.check(rc, "elutq_hlq_gemv_int8lut_f16")
        return y

    def gemv_fused(self, x: torch.Tensor, out: torch.Tensor, ws: torch.Tensor, prologue: int = 0,
                   norm_weight: torch.Tensor | None = None, eps: float = 0.0,
                   residual: torch.Tensor | None = None, slices_out: torch.Tensor | None = None,
                   slices_in: torch.Tensor | None = None, x_out: torch.Tensor | None = None) -> torch.Tensor:
        """Batch-1 GEMV into a caller-owned `out`, optionally fused with the RMSNorm in front of
        the projection (prologue 1), the SiLU(gate)*up in front of it (prologue 2; x holds 2K
        values) and a residual added to the result.  No allocation: `ws` is the caller's
        zero-initialised workspace.  See elutq_hlq_gemv_fused_f16 in include/elutq_hip.h.
        `slices_out` (fp32 [self.slices, N]): the K slices are left unsummed there and `out` is
        not written; `slices_in` (fp32 [S, K], prologue 1): x is the sum of those slices plus `x`,
        rounded to fp16 (what the producer would have written with residual = x), and `x_out`
        receives it.
        A layer with a sparse extra plane held as blocks takes two launches (the plane's fp32 term with
        the same prologue, then the dense kernel, elutq_hlq_sparse_gemv_fused_f16), `ws` of
        self.workspace_bytes, and no slices in either direction."""
        if self.sparse_count and not self._inline() and (slices_out is not None or slices_in is not None):
            raise ValueError("a layer whose sparse extra plane runs as a launch of its own neither takes nor leaves K slices")
        f = _lib.GemvFusion(prologue, eps, norm_weight.data_ptr() if norm_weight is not None else None,
                            residual.data_ptr() if residual is not None else None,
                            slices_out.data_ptr() if slices_out is not None else None,
                            slices_in.data_ptr() if slices_in is not None else None,
                            slices_in.shape[0] if slices_in is not None else 0,
                            x_out.data_ptr() if x_out is not None else None,
                            slices_out.numel() * slices_out.element_size() if slices_out is not None else 0,
                            slices_in.numel() * slices_in.element_size() if slices_in is not None else 0)
        if slices_out is not None and (slices_out.dtype != torch.float32 or slices_out.numel() < self.slices * self.out_features):
            raise ValueError("slices_out must be fp32 [slices, out_features]")
        if slices_in is not None and (slices_in.dtype != torch.float32 or slices_in.dim() != 2
                                      or slices_in.shape[1] != self.in_features or not slices_in.is_contiguous()):
            raise ValueError("slices_in must be contiguous fp32 [S, in_features]")
        if self._inline():
            rc = _lib.lib().elutq_hlq_sparse_gemv_inline_f16(
                self.planes.data_ptr(), self.scales.data_ptr(), self.zeros.data_ptr(),
                self.bias.data_ptr() if self.bias is not None else None, self.sparse_inline.data_ptr(), self.sparse_inline.numel(), x.data_ptr(),
                out.data_ptr(), self.in_features, self.out_features, self.bits, self.group_size, ws.data_ptr(), ws.numel(),
                torch.cuda.current_stream(x.device).cuda_stream, ctypes.byref(f), self.ksplit, self.waves)
            _lib.check(rc, "elutq_hlq_sparse_gemv_inline_f16")
            return out
        if self.sparse_count:
            rc = _lib.lib().elutq_hlq_sparse_gemv_fused_f16(
                self.planes.data_ptr(), self.scales.data_ptr(), self.zeros.data_ptr(),
                self.bias.data_ptr() if self.bias is not None else None, self.sparse_blocks.data_ptr(),
                self.sparse_scales.data_ptr(), self.sparse_index.data_ptr(), self.sparse_count, x.data_ptr(), out.data_ptr(),
                self.in_features, self.out_features, self.bits, self.group_size, ws.data_ptr(), ws.numel(),
                torch.cuda.current_stream(x.device).cuda_stream, ctypes.byref(f), self.ksplit, self.waves)
            _lib.check(rc, "elutq_hlq_sparse_gemv_fused_f16")
            return out
        rc = _lib.lib().elutq_hlq_gemv_fused_f16(
            self.planes.data_ptr(), self.scales.data_ptr(), self.zeros.data_ptr(),
            self.bias.data_ptr() if self.bias is not None else None, x.data_ptr(), out.data_ptr(),
            self.in_features, self.out_features, self.bits, self.group_size, ws.data_ptr(), ws.numel(),
            torch.cuda.current_stream(x.device).cuda_stream, ctypes.byref(f), self.ksplit, self.waves)
        _lib.check(rc, "elutq_hlq_gemv_fused_f16")
        return out

    @property
    def workspace_bytes(self) -> int:
        """Workspace of a batch-1 call (with a sparse extra plane held as blocks: its fp32 term behind the dense part)."""
        if self.sparse_count:
            return _lib.lib().elutq_hlq_sparse_workspace_bytes(self.in_features, self.out_features, self.bits,
                                                               self.group_size, 1)
        return self._ws_bytes

    @property
    def slices(self) -> int:
        """K slices across workgroups of this layer's batch-1 launch (1 = none)."""
        return _lib.lib().elutq_hlq_gemv_slices(self.in_features, self.out_features, self.bits, self.group_size,
                                                self.ksplit, self.waves)

    def accepts_slices(self, n_slices: int) -> bool:
        """Whether this layer's batch-1 launch takes `n_slices` handed-over K slices in its RMSNorm prologue
        (gemv_fused(..., slices_in=...)); a producer may leave its slices unsummed only then."""
        return bool(_lib.lib().elutq_hlq_gemv_accepts_slices(self.in_features, self.out_features, self.bits,
                                                             self.group_size, self.ksplit, self.waves, n_slices))

    def dequantize(self) -> torch.Tensor:
        """Dense fp16 W [N, K] (``dequantize_with_scales``, GPTQ/quant.py:176-183)."""
        w = torch.empty((self.out_features, self.in_features), dtype=torch.float16, device=self.planes.device)
        stream = torch.cuda.current_stream(self.planes.device).cuda_stream
        rc = _lib.lib().elutq_hlq_dequant_f16(self.planes.data_ptr(), self.scales.data_ptr(), self.zeros.data_ptr(),
                                              w.data_ptr(), self.in_features, self.out_features, self.bits,
                                              self.group_size, stream)
        _lib.check(rc, "elutq_hlq_dequant_f16")
        if self.sparse_count:
            rc = _lib.lib().elutq_hlq_sparse_dequant_add_f16(
                self.sparse_blocks.data_ptr(), self.sparse_scales.data_ptr(), self.sparse_index.data_ptr(),
                self.sparse_count, w.data_ptr(), self.in_features, self.out_features, self.group_size, stream)
            _lib.check(rc, "elutq_hlq_sparse_dequant_add_f16")
        return w

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, bits={self.bits}, "
                f"group_size={self.group_size}, bias={self.bias is not None}"
                + (f", sparse_blocks={self.sparse_count}" if self.sparse_count else ""))


class GemvGroup:
    """Independent batch-1 GEMVs that share one launch (elutq_hlq_gemv_group_* of the C ABI).

    `mods`, `xs`, `ys`: equally long lists of HLQLinear layers (same bits and group size), their
    fp16 inputs [1, K] and caller-owned fp16 outputs [1, N].  Creation allocates the device-side
    problem list and a workspace; `run()` is one kernel launch on the current stream and can be
    captured in a HIP graph.  Inputs and outputs are referenced, not copied: refill them in place."""

    def __init__(self, mods, xs, ys):
        if not mods or not (len(mods) == len(xs) == len(ys)):
            raise ValueError("need equally long, non-empty lists of layers, inputs and outputs")
        bits, group = mods[0].bits, mods[0].group_size
        arr = (_lib.GemvProblem * len(mods))()
        for p, m, x, y in zip(arr, mods, xs, ys):
            if (m.bits, m.group_size) != (bits, group):
                raise ValueError("all layers of a group must share bits and group size")
            if m.sparse_count:
                raise NotImplementedError("layers with a sparse extra plane cannot join a grouped launch")
            if x.dtype != torch.float16 or y.dtype != torch.float16 or x.numel() != m.in_features or y.numel() != m.out_features:
                raise ValueError("inputs must be fp16 [K], outputs fp16 [N]")
            p.d_planes, p.d_scales, p.d_zeros = m.planes.data_ptr(), m.scales.data_ptr(), m.zeros.data_ptr()
            p.d_bias = m.bias.data_ptr() if m.bias is not None else None
            p.d_x, p.d_y, p.K, p.N = x.data_ptr(), y.data_ptr(), m.in_features, m.out_features
        L = _lib.lib()
        self._keep = (list(mods), list(xs), list(ys))
        self._device = mods[0].planes.device
        nbytes = L.elutq_hlq_gemv_group_workspace_bytes(ctypes.byref(arr), len(mods), bits, group)
        if nbytes == 0:
            raise ValueError("unsupported shape in the group")
        self.ws = torch.zeros(nbytes, dtype=torch.uint8, device=self._device)
        plan = ctypes.c_void_p()
        _lib.check(L.elutq_hlq_gemv_group_create(ctypes.byref(arr), len(mods), bits, group, self.ws.data_ptr(),
                                                 self.ws.numel(), ctypes.byref(plan)), "elutq_hlq_gemv_group_create")
        self._plan = plan

    def run(self) -> None:
        _lib.check(_lib.lib().elutq_hlq_gemv_group_run(self._plan, torch.cuda.current_stream(self._device).cuda_stream),
                   "elutq_hlq_gemv_group_run")

    def close(self) -> None:
        if self._plan is not None:
            torch.cuda.synchronize(self._device)
            _lib.lib().elutq_hlq_gemv_group_destroy(self._plan)
            self._plan = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def replace_linear(model: nn.Module, export_root: str, device="cuda", group_size: int | None = None) -> int:
    """Swaps every ``nn.Linear`` that has an export directory for an HLQLinear.

    Directories follow the reference: ``<export_root>/<layer id>/<name>`` with ``name`` the
    module path inside the decoder layer (``self_attn.q_proj`` ... ``mlp.down_proj``,
    GPTQ/llama.py:90-95, GPTQ/HLQ.py:73).  Returns the number of modules replaced."""
    replaced = 0
    for full_name, mod in list(model.named_modules()):
        if not isinstance(mod, nn.Linear):
            continue
        parts = full_name.split(".")
        idx = next((i for i, p in enumerate(parts) if p.isdigit()), None)
        if idx is None:
            continue
        path = os.path.join(export_root, parts[idx], ".".join(parts[idx + 1:]))
        if not os.path.exists(os.path.join(path, "weight_config.json")):
            continue
        new = HLQLinear.from_export_dir(path, device, group_size)
        parent = model.get_submodule(".".join(parts[:-1])) if len(parts) > 1 else model
        setattr(parent, parts[-1], new)
        replaced += 1
    return replaced
