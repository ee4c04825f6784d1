"""Quantize on the device, export, load, run: the whole chain from an fp16 weight to the HIP
kernels without the reference (HLQ.fasterquant -> export files -> load_Parameter -> arm_gemm)."""
import numpy as np
import pytest
import torch

from elutq_amd import export_io as io
from elutq_amd import hlq_quantize as HQ
from elutq_amd.hlq_linear import HLQLinear

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bits,group", [(2, 128), (3, 128), (2, 64), (4, 128)])
def test_quantize_export_load_run(cuda, tmp_path, bits, group):
    g = torch.Generator(device=cuda).manual_seed(bits * 100 + group)
    k, n, m = 512, 192, 256
    w = torch.randn(n, k, generator=g, device=cuda) * 0.04
    x = torch.randn(m, k, generator=g, device=cuda)
    h = 2.0 / m * x.t() @ x
    wq, codes, scales, zeros = HQ.gptq_hlq(w, h, bits, group)
    assert wq.is_cuda and codes.is_cuda
    # the compensation lowers the error of the layer's outputs on the calibration inputs below that of
    # plain group-wise quantization, and more bits mean less of it
    out_err = lambda q: float((((w - q) @ x.t()) ** 2).mean() / ((w @ x.t()) ** 2).mean())
    assert out_err(wq) < out_err(HQ.quantize_groups(w, bits, group)[0])
    assert out_err(wq) < {2: 0.2, 3: 0.06, 4: 0.02}[bits]
    d = str(tmp_path / "q_proj")
    io.write_export_dir(d, *HQ.to_export_arrays(codes, scales, zeros))
    mod = HLQLinear.from_export_dir(d, cuda)
    assert (mod.in_features, mod.out_features, mod.bits, mod.group_size) == (k, n, bits, group)
    # the loaded layer is the quantizer's reconstruction up to the fp16 rounding of scales and zeros
    deq = mod.dequantize().float()
    assert (deq - wq).abs().max() <= 2.0 ** -9 * wq.abs().max()
    xv = x[:1].half()
    y = mod(xv).float()
    ref = xv.float() @ deq.t()
    assert (y - ref).abs().max() <= 1e-2 * ref.pow(2).mean().sqrt()
