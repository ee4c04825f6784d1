"""HLQ quantizer (elutq_amd/hlq_quantize.py) against the golden vectors written by
tests/golden/make_quantizer_goldens.py from the reference's GPTQ/quant.py, and against what the
mathematics fixes: each half-step of the alternating fit is an exact minimisation, data on a
uniform grid is reproduced exactly, a diagonal Hessian switches the GPTQ compensation off."""
import os

import numpy as np
import pytest
import torch

from elutq_amd import hlq_quantize as HQ
from oracle import hlq_oracle as O

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hlq_quantizer_vectors.npz"))
CASES = [("b2_g128", 2), ("b3_g128", 3), ("b2_g64", 2), ("b4_g128", 4), ("b1_g64", 1)]


def mse(w, codes, scales, zeros):
    return float(((HQ.dequantize_codes(codes, scales, zeros) - w) ** 2).mean())


@pytest.mark.parametrize("name,bits", CASES)
def test_fit_and_assignment_match_reference_vectors(name, bits):
    w = torch.from_numpy(GOLD[f"{name}_w"])
    scales, zeros = HQ.fit_alternating(w, bits)
    # same algorithm, fp32: equal up to the rounding of the least-squares solves
    np.testing.assert_allclose(scales.numpy(), GOLD[f"{name}_scales"], rtol=2e-4, atol=1e-7)
    np.testing.assert_allclose(zeros.numpy(), GOLD[f"{name}_zeros"], rtol=2e-4, atol=1e-6)
    # the assignment on the reference's own parameters is bit-identical (same enumeration, first minimum)
    gs, gz = torch.from_numpy(GOLD[f"{name}_scales"]), torch.from_numpy(GOLD[f"{name}_zeros"])
    codes = HQ.assign_codes(w, gs, gz, bits)
    assert codes.dtype == torch.uint8 and np.array_equal(codes.numpy(), GOLD[f"{name}_codes"])
    assert np.array_equal(HQ.dequantize_codes(codes, gs, gz).numpy(), GOLD[f"{name}_deq"])
    # and end to end the reconstruction error equals the reference's
    own = HQ.assign_codes(w, scales, zeros, bits)
    assert (own.numpy() != GOLD[f"{name}_codes"]).mean() < 0.01
    assert mse(w, own, scales, zeros) == pytest.approx(float(((GOLD[f"{name}_deq"] - GOLD[f"{name}_w"]) ** 2).mean()), rel=1e-3)


def test_quantize_groups_matches_reference_slab():
    w = torch.from_numpy(GOLD["slab_w"])
    wq, codes, scales, zeros = HQ.quantize_groups(w, 2, 128)
    assert codes.shape == GOLD["slab_codes"].shape and scales.shape == GOLD["slab_scales"].shape
    assert zeros.shape == GOLD["slab_zeros"].shape
    np.testing.assert_allclose(scales.numpy(), GOLD["slab_scales"], rtol=2e-4, atol=1e-7)
    np.testing.assert_allclose(zeros.numpy(), GOLD["slab_zeros"], rtol=2e-4, atol=1e-6)
    assert (codes.numpy() != GOLD["slab_codes"]).mean() < 0.01
    np.testing.assert_allclose(wq.numpy(), GOLD["slab_deq"], atol=2e-3 * np.abs(GOLD["slab_w"]).max())


@pytest.mark.parametrize("bits", [1, 2, 3, 4])
def test_each_half_step_is_a_minimisation(bits):
    g = torch.Generator().manual_seed(bits)
    w = torch.randn(9, 64, generator=g) * 0.1 + 0.03
    prev = None
    for iters in range(1, 8):
        s, z = HQ.fit_alternating(w, bits, iters=iters)
        codes = HQ.assign_codes(w, s, z, bits)
        e = mse(w, codes, s, z)
        assert prev is None or e <= prev * (1 + 1e-5)          # the error never grows with more rounds
        prev = e
        # codes are optimal for (s, z): no other level is nearer for any element (brute force)
        levels = (HQ._codes_msb_first(bits, w.device, torch.float32) @ s.t()).t() + z[:, None]     # [blocks, 2^bits]
        best = (w[:, :, None] - levels[:, None, :]).abs().min(dim=2).values
        got = (HQ.dequantize_codes(codes, s, z) - w).abs()
        assert torch.all(got <= best + 1e-7)
    # (s, z) are optimal for the codes of the last fit round: the normal equations hold
    s, z = HQ.fit_alternating(w, bits, iters=10)
    s9, z9 = HQ.fit_alternating(w, bits, iters=9)
    lv = torch.cat([HQ._codes_lsb_first(bits, w.device, torch.float32), torch.ones(2 ** bits, 1)], dim=1)
    idx = (w[:, :, None] - (torch.cat([s9, z9[:, None]], 1) @ lv.t())[:, None, :]).abs().argmin(2)
    a = lv[idx]
    r = w - (a @ torch.cat([s, z[:, None]], 1)[:, :, None]).squeeze(2)
    assert (a.transpose(1, 2) @ r[:, :, None]).abs().max() < 1e-4         # residual orthogonal to the design matrix


@pytest.mark.parametrize("bits", [2, 3])
def test_uniform_grid_is_reproduced(bits):
    r = np.random.default_rng(bits)
    q = r.integers(0, 2 ** bits, (5, 128))
    q[:, 0], q[:, 1] = 0, 2 ** bits - 1                       # both ends of the range occur
    step, zero = 0.0625, -0.25
    w = torch.from_numpy((zero + step * q).astype(np.float32))
    wq, codes, scales, zeros = HQ.quantize_groups(w, bits, 128)
    assert (wq - w).abs().max() <= 1e-6                      # exact up to the rounding of the least-squares solve
    np.testing.assert_allclose(scales.numpy()[:, 0], np.tile(step * 2.0 ** np.arange(bits), (5, 1)), rtol=1e-5)
    np.testing.assert_allclose(zeros.numpy().ravel(), zero, rtol=1e-5)
    assert np.array_equal((codes.numpy() * (1 << np.arange(bits))).sum(-1), q)


def test_export_arrays_round_trip_through_the_oracle():
    g = torch.Generator().manual_seed(5)
    w = torch.randn(24, 256, generator=g) * 0.05
    wq, codes, scales, zeros = HQ.quantize_groups(w, 2, 128)
    w_quant, w_scale, w_zero = HQ.to_export_arrays(codes, scales, zeros)
    assert w_quant.shape == (2, 24, 32) and w_scale.shape == (2, 24, 2) and w_zero.shape == (24, 2)
    assert w_quant.dtype == np.uint8 and w_scale.dtype == np.float16 and w_zero.dtype == np.float16
    assert np.array_equal(O.unpack_planes(w_quant), codes.permute(2, 0, 1).numpy())
    for a, b in zip((w_quant, w_scale, w_zero), O.export_arrays(codes.numpy(), scales.numpy(), zeros.numpy())):
        assert np.array_equal(a, b)                           # the oracle's restatement of HLQ.export
    deq = O.dequantize(w_quant, w_scale, w_zero, 128, np.float64)
    # the files hold fp16 parameters: equal to the fp32 reconstruction up to that rounding
    assert np.abs(deq - wq.numpy()).max() <= 3 * 2.0 ** -11 * np.abs(wq.numpy()).max()


def test_gptq_with_diagonal_hessian_is_plain_group_quantization():
    g = torch.Generator().manual_seed(11)
    w = torch.randn(16, 256, generator=g) * 0.04
    h = torch.diag(torch.rand(256, generator=g) + 0.5)
    wq, codes, scales, zeros = HQ.gptq_hlq(w, h, 2, 128)
    rq, rcodes, rscales, rzeros = HQ.quantize_groups(w, 2, 128)
    assert torch.equal(codes, rcodes) and torch.equal(scales, rscales) and torch.equal(wq, rq)
    h[3, 3] = 0                                               # a dead input column is zeroed first (HLQ.py:92-94)
    wq2, _, _, _ = HQ.gptq_hlq(w, h, 2, 128)
    w0 = w.clone(); w0[:, 3] = 0
    assert torch.equal(wq2, HQ.quantize_groups(w0, 2, 128)[0])


def test_gptq_lowers_the_output_error_on_correlated_inputs():
    g = torch.Generator().manual_seed(3)
    k, n, m = 256, 32, 512
    mix = torch.randn(k, k, generator=g) / k ** 0.5 + torch.eye(k)
    x = torch.randn(m, k, generator=g) @ mix                  # correlated calibration inputs
    w = torch.randn(n, k, generator=g) * 0.05
    h = 2.0 / m * x.t() @ x
    out_err = lambda q: float((((w - q) @ x.t()) ** 2).mean())
    plain = HQ.quantize_groups(w, 2, 128)[0]
    for actorder in (False, True):
        wq, codes, scales, zeros = HQ.gptq_hlq(w, h, 2, 128, actorder=actorder)
        assert codes.shape == (n, k, 2) and scales.shape == (n, 2, 2) and zeros.shape == (n, 2, 1)
        assert out_err(wq) < 0.9 * out_err(plain)
    with pytest.raises(ValueError):
        HQ.gptq_hlq(w, h[:10, :10], 2, 128)
    with pytest.raises(ValueError):
        HQ.quantize_groups(w[:, :100], 2, 128)


@pytest.mark.parametrize("k,group,bits,actorder", [(32, 8, 2, False), (32, 16, 3, False), (24, 8, 2, True), (32, 32, 2, False),
                                                   (20, 8, 3, True), (16, 16, 4, False)])
def test_gptq_loop_against_textbook_obq(k, group, bits, actorder):
    """The error-feedback loop itself (GPTQ/HLQ.py:108-153: per-group quantization, per-column error over the diagonal of
    the Cholesky factor, propagation inside the group and to the later groups; actorder = the same on columns sorted
    by the Hessian's diagonal) against tests/obq_reference.py -- an explicit inverse Hessian in float64 with one column
    eliminated at a time, no Cholesky factor, no blocks -- with the same simple group quantizer injected into both.
    A dropped propagation term, a wrong divisor, a transposed factor or a missed permutation changes the compensated
    weights the later groups are quantized from, hence w_q."""
    from obq_reference import correlated_problem, obq_reference, uniform_group_quantizer
    for seed in range(4):
        w, h = correlated_problem(100 * k + seed, 12, k)
        if seed == 3:
            h[5, :] = 0; h[:, 5] = 0                               # a dead input column (HLQ.py:92-94)
        want = obq_reference(w, h, bits, group, actorder=actorder)
        got = HQ.gptq_hlq(torch.from_numpy(w).float(), torch.from_numpy(h).float(), bits, group, actorder=actorder,
                          quantizer=uniform_group_quantizer)[0].double().numpy()
        np.testing.assert_allclose(got, want, atol=1e-5, rtol=0)
        # the loop is not a no-op on these inputs: plain group quantization gives other numbers
        if group < k:
            assert np.abs(got - np.concatenate([uniform_group_quantizer(torch.from_numpy(w[:, c:c + group]).float(), bits, group)[0].numpy()
                                                for c in range(0, k, group)], axis=1)).max() > 1e-3
