"""HLQ quantizer: fits W ~ z_g + sum_b s_{g,b} * B_b per group and emits the export arrays.

Counterpart of the reference's offline quantizer, restated on PyTorch tensors so it runs on
the GPU box (any device PyTorch-ROCm offers) without the reference:

  fit_alternating      find_optimal_params_alternating   GPTQ/quant.py:116-153
  assign_codes         quantize_with_scales              GPTQ/quant.py:154-174
  dequantize_codes     dequantize_with_scales            GPTQ/quant.py:176-183
  quantize_groups      pseudo_quantize_tensor(get_scale_zp=True, use_alternating_optimization=True)
                                                         GPTQ/quant.py:185-213
  gptq_hlq             HLQ.fasterquant (nn.Linear)       GPTQ/HLQ.py:63-173
  to_export_arrays     HLQ.export + Pack_T_MAC_Weight    GPTQ/HLQ.py:207-251

Only the alternating fit is mirrored; the Adam variant (quant.py:18-94) is not.  This is
offline tooling in front of the hot path: plain tensor algebra, no custom kernels.

The fit alternates two exact minimisations of sum (w - z - sum_b s_b c_b)^2 over a block:
codes for fixed (s, z) -- every element takes the nearest of the 2^bits levels -- and (s, z)
for fixed codes -- linear least squares on the design matrix [codes | 1] -- so the error
never grows from one round to the next.  Ties and enumeration orders follow the reference
(first minimum; the fit enumerates levels with code bit j = (i >> j) & 1, the final
assignment with the tuples of itertools.product([0, 1], repeat=bits), i.e. most significant
bit first), so that near-ties resolve the same way.
"""
from __future__ import annotations

import numpy as np
import torch

from .synth import pack_bits_lsb_first


def _codes_lsb_first(bits: int, device, dtype) -> torch.Tensor:
    """[2^bits, bits]: row i holds (i >> j) & 1."""
    i = torch.arange(2 ** bits, device=device)
    return torch.stack([(i >> j) & 1 for j in range(bits)], dim=1).to(dtype)


def _codes_msb_first(bits: int, device, dtype) -> torch.Tensor:
    """[2^bits, bits]: row i holds the binary digits of i, most significant first."""
    i = torch.arange(2 ** bits, device=device)
    return torch.stack([(i >> (bits - 1 - j)) & 1 for j in range(bits)], dim=1).to(dtype)


@torch.no_grad()
def fit_alternating(w: torch.Tensor, bits: int, iters: int = 10):
    """w [blocks, block_size] -> (scales [blocks, bits], zeros [blocks]) in fp32."""
    w = w.to(torch.float32)
    nb, _ = w.shape
    lo, hi = w.min(dim=1).values, w.max(dim=1).values
    step = (hi - lo) / (2 ** bits - 1)
    sol = torch.cat([step[:, None] * (2.0 ** torch.arange(bits, device=w.device, dtype=torch.float32)), lo[:, None]], dim=1)
    design = torch.cat([_codes_lsb_first(bits, w.device, torch.float32),
                        torch.ones(2 ** bits, 1, device=w.device)], dim=1)             # [2^bits, bits + 1]
    for _ in range(iters):
        levels = sol @ design.t()                                                     # [blocks, 2^bits]
        idx = (w[:, :, None] - levels[:, None, :]).abs().argmin(dim=2)                # nearest level, first on ties
        a = design[idx]                                                               # [blocks, block_size, bits + 1]
        at = a.transpose(1, 2)
        sol = (torch.linalg.pinv(at @ a) @ (at @ w[:, :, None])).squeeze(2)           # least squares, min-norm if singular
    return sol[:, :bits].contiguous(), sol[:, bits].contiguous()


@torch.no_grad()
def assign_codes(w: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor, bits: int) -> torch.Tensor:
    """Nearest level per element: uint8 codes [blocks, block_size, bits] (plane b pairs with scales[:, b])."""
    table = _codes_msb_first(bits, w.device, w.dtype)
    levels = scales.to(w.device) @ table.t()                                          # [blocks, 2^bits]
    idx = (levels[:, None, :] - (w - zeros.to(w.device)[:, None])[:, :, None]).abs().argmin(dim=2)
    return table[idx].to(torch.uint8)


@torch.no_grad()
def dequantize_codes(codes: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor) -> torch.Tensor:
    return (codes.float() * scales[:, None, :]).sum(dim=2) + zeros[:, None]


@torch.no_grad()
def quantize_groups(w: torch.Tensor, bits: int, group: int, iters: int = 10):
    """w [rows, cols] with cols % group == 0 -> (w_q [rows, cols] in w.dtype, codes uint8 [rows, cols, bits],
    scales fp32 [rows, cols/group, bits], zeros fp32 [rows, cols/group, 1])."""
    rows, cols = w.shape
    if cols % group:
        raise ValueError(f"{cols} columns are not a multiple of the group size {group}")
    blocks = w.reshape(-1, group)
    scales, zeros = fit_alternating(blocks, bits, iters)
    codes = assign_codes(blocks, scales.to(blocks.dtype), zeros.to(blocks.dtype), bits)
    wq = dequantize_codes(codes, scales, zeros).reshape(rows, cols).to(w.dtype)
    return (wq, codes.reshape(rows, cols, bits), scales.reshape(rows, cols // group, bits),
            zeros.reshape(rows, cols // group, 1))


@torch.no_grad()
def gptq_hlq(weight: torch.Tensor, hessian: torch.Tensor, bits: int, group: int, percdamp: float = 0.01,
             actorder: bool = False, iters: int = 10, quantizer=None):
    """GPTQ error compensation around the group-wise HLQ fit for one linear layer.

    weight [N, K]; hessian [K, K] = 2/n * sum x x^T over the calibration inputs (HLQ.add_batch,
    GPTQ/HLQ.py:36-60).  Each group of columns is quantized as a whole from the weights as
    compensated so far; its per-column errors, divided by the diagonal of the upper Cholesky
    factor of H^-1, are propagated to the later columns of the group and then to all later
    groups.  Returns (w_q fp32 [N, K], codes uint8 [N, K, bits], scales fp32 [N, K/group, bits],
    zeros fp32 [N, K/group, 1]); with actorder the codes / scales / zeros refer to the permuted
    column order, as in the reference.  `quantizer(w1, bits, group_size, iters)` stands in for
    quantize_groups (same arguments and results) where a test wants the loop alone."""
    quantizer = quantizer or quantize_groups
    w = weight.detach().clone().float()
    h = hessian.detach().clone().float()
    n, k = w.shape
    if h.shape != (k, k):
        raise ValueError("hessian must be [K, K]")
    if group == -1:
        group = k
    dead = torch.diag(h) == 0
    h[dead, dead] = 1
    w[:, dead] = 0
    if actorder:
        perm = torch.argsort(torch.diag(h), descending=True)
        w, h = w[:, perm], h[perm][:, perm]
    h = h + torch.eye(k, device=h.device) * (percdamp * torch.diag(h).mean())
    u = torch.linalg.cholesky(torch.cholesky_inverse(torch.linalg.cholesky(h)), upper=True)
    wq = torch.zeros_like(w)
    codes, scales, zeros = [], [], []
    for c0 in range(0, k, group):
        c1 = min(c0 + group, k)
        w1 = w[:, c0:c1].clone()
        q1, cd, sc, zp = quantizer(w1, bits, c1 - c0, iters)
        codes.append(cd); scales.append(sc); zeros.append(zp)
        u1 = u[c0:c1, c0:c1]
        err = torch.zeros_like(w1)
        for i in range(c1 - c0):
            e = (w1[:, i] - q1[:, i]) / u1[i, i]
            w1[:, i:] -= e[:, None] * u1[i, i:][None, :]
            err[:, i] = e
        wq[:, c0:c1] = q1
        w[:, c1:] -= err @ u[c0:c1, c1:]
    if actorder:
        wq = wq[:, torch.argsort(perm)]
    return wq, torch.cat(codes, dim=1), torch.cat(scales, dim=1), torch.cat(zeros, dim=1)


def to_export_arrays(codes: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor):
    """-> (w_quant uint8 [bits][N][K/8] LSB-first, w_scale fp16 [bits][N][K/G], w_zero fp16 [N][K/G]):
    the arrays of the export files (elutq_amd.export_io.write_export_dir)."""
    n, k, bits = codes.shape
    planes = codes.to(torch.uint8).permute(2, 0, 1).contiguous().cpu().numpy()
    w_scale = scales.to(torch.float16).permute(2, 0, 1).contiguous().cpu().numpy()
    w_zero = zeros.to(torch.float16).reshape(n, -1).contiguous().cpu().numpy()
    return pack_bits_lsb_first(planes), np.ascontiguousarray(w_scale), np.ascontiguousarray(w_zero)
