"""Quantize on the device, export, load, run: the whole chain from an fp16 weight to the HIP
kernels without the reference (HLQ.fasterquant -> export files -> load_Parameter -> arm_gemm)."""
import os

import numpy as np
import pytest
import torch

from elutq_amd import export_io as io
from elutq_amd import hlq_quantize as HQ
from elutq_amd.hlq_linear import HLQLinear

pytestmark = pytest.mark.gpu

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hlq_quantizer_vectors.npz"))


@pytest.mark.parametrize("name,bits", [("b2_g128", 2), ("b3_g128", 3), ("b2_g64", 2), ("b4_g128", 4), ("b1_g64", 1)])
def test_fit_and_assignment_on_the_device_match_reference_vectors(cuda, name, bits):
    """The alternating fit and the nearest-level assignment run on device tensors against the vectors the
    reference's own GPTQ/quant.py wrote (tests/golden/make_quantizer_goldens.py): same bars as on the CPU."""
    w = torch.from_numpy(GOLD[f"{name}_w"]).to(cuda)
    scales, zeros = HQ.fit_alternating(w, bits)
    assert scales.is_cuda and zeros.is_cuda
    np.testing.assert_allclose(scales.cpu().numpy(), GOLD[f"{name}_scales"], rtol=2e-4, atol=1e-7)
    np.testing.assert_allclose(zeros.cpu().numpy(), GOLD[f"{name}_zeros"], rtol=2e-4, atol=1e-6)
    gs, gz = torch.from_numpy(GOLD[f"{name}_scales"]).to(cuda), torch.from_numpy(GOLD[f"{name}_zeros"]).to(cuda)
    codes = HQ.assign_codes(w, gs, gz, bits)
    assert codes.is_cuda and codes.dtype == torch.uint8
    # the device forms the levels with a library matrix product whose summation order is its own: an
    # element that sits within an ulp of the midpoint of two levels may land on the other one
    same = codes.cpu().numpy() == GOLD[f"{name}_codes"]
    assert (~same).mean() <= 1e-3
    deq = HQ.dequantize_codes(codes, gs, gz).cpu().numpy()
    keep = same.all(axis=-1)
    np.testing.assert_allclose(deq[keep], GOLD[f"{name}_deq"][keep], rtol=1e-6, atol=1e-8)
    own = HQ.assign_codes(w, scales, zeros, bits)
    assert (own.cpu().numpy() != GOLD[f"{name}_codes"]).mean() < 0.01
    mse = float(((HQ.dequantize_codes(own, scales, zeros) - w) ** 2).mean())
    assert mse == pytest.approx(float(((GOLD[f"{name}_deq"] - GOLD[f"{name}_w"]) ** 2).mean()), rel=1e-3)


def test_quantize_groups_on_the_device_matches_reference_slab(cuda):
    w = torch.from_numpy(GOLD["slab_w"]).to(cuda)
    wq, codes, scales, zeros = HQ.quantize_groups(w, 2, 128)
    assert wq.is_cuda and codes.shape == GOLD["slab_codes"].shape
    np.testing.assert_allclose(scales.cpu().numpy(), GOLD["slab_scales"], rtol=2e-4, atol=1e-7)
    np.testing.assert_allclose(zeros.cpu().numpy(), GOLD["slab_zeros"], rtol=2e-4, atol=1e-6)
    assert (codes.cpu().numpy() != GOLD["slab_codes"]).mean() < 0.01
    np.testing.assert_allclose(wq.cpu().numpy(), GOLD["slab_deq"], atol=2e-3 * np.abs(GOLD["slab_w"]).max())


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


@pytest.mark.parametrize("k,group,bits,actorder", [(32, 8, 2, False), (32, 16, 3, True), (24, 8, 2, True), (32, 32, 2, False)])
def test_gptq_loop_against_textbook_obq_on_the_device(cuda, k, group, bits, actorder):
    """gptq_hlq on device tensors against the textbook restatement of the error-feedback loop (tests/obq_reference.py:
    explicit float64 inverse Hessian, one column eliminated at a time), the same simple group quantizer injected into
    both; the reference's loop is GPTQ/HLQ.py:108-153."""
    import numpy as np
    from obq_reference import correlated_problem, obq_reference, uniform_group_quantizer
    for seed in range(3):
        w, h = correlated_problem(100 * k + seed, 12, k)
        want = obq_reference(w, h, bits, group, actorder=actorder)
        got = HQ.gptq_hlq(torch.from_numpy(w).float().to(cuda), torch.from_numpy(h).float().to(cuda), bits, group,
                          actorder=actorder, quantizer=uniform_group_quantizer)[0]
        assert got.is_cuda
        np.testing.assert_allclose(got.double().cpu().numpy(), want, atol=1e-5, rtol=0)
