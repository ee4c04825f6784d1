"""Fused GEMV entry point (elutq_hlq_gemv_fused_f16): RMSNorm prologue, SiLU(gate)*up
prologue and residual epilogue against the unfused pipeline (PyTorch op + plain GEMV) and
the float64 oracle."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from elutq_amd import _lib
from elutq_amd.hlq_linear import HLQLinear
from elutq_amd.synth import make_layer
from oracle import hlq_oracle as O

pytestmark = pytest.mark.gpu


def build(k, n, bits, group, seed, dev):
    L = make_layer(k, n, bits=bits, group=group, seed=seed, bias=True)
    return L, HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, group, L.bias, dev)


@pytest.mark.parametrize("k,n,bits,group", [(1024, 256, 2, 128), (512, 100, 3, 64), (4096, 1024, 2, 128), (1088, 130, 2, 64)])
@pytest.mark.parametrize("ksplit,waves", [(0, 0), (1, 4), (2, 16), (_lib.GEMV_NARROW16, 0), (_lib.GEMV_NARROW32, 0),
                                          (_lib.GEMV_WIDE, 0)])
def test_rmsnorm_prologue_and_residual(cuda, k, n, bits, group, ksplit, waves):
    L, mod = build(k, n, bits, group, 5, cuda)
    mod.ksplit, mod.waves = ksplit, waves
    g = torch.Generator(device=cuda).manual_seed(1)
    x = (torch.randn(1, k, generator=g, device=cuda) * 3).half()
    w = (1 + 0.1 * torch.randn(k, generator=g, device=cuda)).half()
    res = torch.randn(1, n, generator=g, device=cuda).half()
    eps = 1e-5
    out = torch.empty(1, n, dtype=torch.float16, device=cuda)
    ws = torch.zeros(mod.workspace_bytes, dtype=torch.uint8, device=cuda)
    mod.gemv_fused(x, out, ws, prologue=1, norm_weight=w, eps=eps, residual=res)
    # unfused: fp32 RMSNorm rounded to fp16 (the reference's op boundary), then the oracle
    xf = x.float()
    h = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()).half()
    ref = O.gemv_f64(h.cpu().numpy()[0], L.w_quant, L.w_scale, L.w_zero, group, L.bias) + res.cpu().numpy()[0].astype(np.float64)
    assert O.rel_err(out.cpu().numpy()[0], ref) <= 1e-2
    # and the plain kernel on the same normalised input agrees to fp16 rounding of h
    y_plain = mod(h).float() + res.float()
    assert (out.float() - y_plain).abs().max() <= 2e-2 * y_plain.abs().max()


@pytest.mark.parametrize("k,n,bits,group", [(1024, 256, 2, 128), (1536, 192, 4, 64), (960, 100, 2, 64)])
@pytest.mark.parametrize("ksplit", [0, _lib.GEMV_NARROW16, _lib.GEMV_NARROW32, _lib.GEMV_WIDE])
def test_silu_mul_prologue(cuda, k, n, bits, group, ksplit):
    L, mod = build(k, n, bits, group, 7, cuda)
    mod.ksplit = ksplit
    g = torch.Generator(device=cuda).manual_seed(2)
    gu = torch.randn(1, 2 * k, generator=g, device=cuda).half()
    res = torch.randn(1, n, generator=g, device=cuda).half()
    out = torch.empty(1, n, dtype=torch.float16, device=cuda)
    ws = torch.zeros(mod.workspace_bytes, dtype=torch.uint8, device=cuda)
    mod.gemv_fused(gu, out, ws, prologue=2, residual=res)
    act = (F.silu(gu[:, :k].float()) * gu[:, k:].float()).half()
    ref = O.gemv_f64(act.cpu().numpy()[0], L.w_quant, L.w_scale, L.w_zero, group, L.bias) + res.cpu().numpy()[0].astype(np.float64)
    assert O.rel_err(out.cpu().numpy()[0], ref) <= 1e-2


def test_no_fusion_equals_plain_gemv_bitwise(cuda):
    L, mod = build(768, 130, 2, 128, 9, cuda)
    x = torch.from_numpy(L.x).to(cuda)
    out = torch.empty(1, 130, dtype=torch.float16, device=cuda)
    ws = torch.zeros(mod.workspace_bytes, dtype=torch.uint8, device=cuda)
    mod.gemv_fused(x, out, ws)
    assert torch.equal(out, mod(x))


def test_fusion_argument_errors(cuda):
    L, mod = build(256, 64, 2, 128, 3, cuda)
    x = torch.zeros(1, 256, dtype=torch.float16, device=cuda)
    out = torch.empty(1, 64, dtype=torch.float16, device=cuda)
    ws = torch.zeros(mod.workspace_bytes, dtype=torch.uint8, device=cuda)
    with pytest.raises(_lib.ElutqError):
        mod.gemv_fused(x, out, ws, prologue=1)            # RMSNorm without a weight
    with pytest.raises(_lib.ElutqError):
        mod.gemv_fused(x, out, ws, prologue=3)
