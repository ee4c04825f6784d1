"""GPU parity of the small-batch MFMA GEMM (C ABI elutq_hlq_gemm_f16) against the oracle.

The reference defines m > 1 as one GEMV per row (arm_gemm.cpp:380-385); the oracle for it
is the float64 dequantize-then-matmul, tolerance rel_err <= 1e-2 on fp16 outputs (the
kernel's error is fp32 accumulation plus the final fp16 rounding).  Rows must also agree
with the batch-1 LUT kernel to the same tolerance.
"""
import numpy as np
import pytest
import torch

from elutq_amd.hlq_linear import HLQLinear
from elutq_amd.synth import LLAMA2_13B_PREFILL_SHAPES, make_layer
from oracle import hlq_oracle as O

pytestmark = pytest.mark.gpu
TOL = 1e-2


def gemm(L, dev, x=None):
    mod = HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, L.group, L.bias, dev)
    y = mod(torch.from_numpy(np.ascontiguousarray(L.x if x is None else x)).to(dev))
    torch.cuda.synchronize()
    return mod, y.cpu().numpy()


@pytest.mark.parametrize("m", [2, 5, 16, 31, 32, 33, 64, 70, 130])
@pytest.mark.parametrize("k,n,bits,group", [(512, 128, 2, 128), (1024, 192, 3, 128), (640, 100, 2, 64),
                                             (384, 64, 4, 64), (2048, 64, 1, 128), (1216, 100, 2, 64), (192, 64, 3, 64)])
def test_gemm_matches_oracle(cuda, m, k, n, bits, group):
    L = make_layer(k, n, bits=bits, group=group, m=m, seed=m + k + bits, bias=(bits == 3))
    _, y = gemm(L, cuda)
    ref = O.gemm_f64(L.x, L.w_quant, L.w_scale, L.w_zero, group, L.bias)
    assert y.shape == (m, n) and y.dtype == np.float16
    assert O.rel_err(y, ref) <= TOL
    assert np.max(np.abs(y.astype(np.float64) - ref)) <= 2.0 ** -9 * max(1.0, np.max(np.abs(ref)))


@pytest.mark.parametrize("m", [3, 40])
def test_gemm_rows_do_not_leak_where_k_ends_inside_a_unit(cuda, m):
    """K = 64 mod 128 at group 64: the staging of a row's last unit must not take in the start of the next row.
    A NaN at the head of row 1 stays in row 1."""
    L = make_layer(704, 130, bits=2, group=64, m=m, seed=5)
    x = L.x.copy()
    x[1, :8] = np.nan
    _, y = gemm(L, cuda, x)
    ref = O.gemm_f64(L.x, L.w_quant, L.w_scale, L.w_zero, 64)
    keep = np.arange(m) != 1
    assert np.all(np.isnan(y[1].astype(np.float32))) and np.all(np.isfinite(y[keep].astype(np.float32)))
    assert O.rel_err(y[keep], ref[keep]) <= TOL


def test_gemm_rows_agree_with_gemv_and_are_deterministic(cuda):
    L = make_layer(1024, 256, bits=2, group=128, m=16, seed=3, bias=True)
    mod, y = gemm(L, cuda)
    _, y2 = gemm(L, cuda)
    assert np.array_equal(y, y2)
    for i in (0, 7, 15):
        yi = mod(torch.from_numpy(L.x[i:i + 1]).to(cuda)).cpu().numpy()[0]          # LUT GEMV path
        assert O.rel_err(y[i], yi.astype(np.float64)) <= 2e-3
    # rows are independent: permuting the rows of x permutes the rows of y exactly
    perm = np.random.default_rng(0).permutation(16)
    _, yp = gemm(L, cuda, L.x[perm])
    assert np.array_equal(yp, y[perm])


def test_gemm_exact_on_integer_inputs(cuda):
    r = np.random.default_rng(9)
    m, k, n, bits, group = 24, 768, 128, 2, 128
    x = r.integers(-2, 3, (m, k)).astype(np.float16)
    wq = O.pack_planes(r.integers(0, 2, (bits, n, k), dtype=np.uint8))
    ws = np.stack([np.full((n, k // group), 2.0 ** (b - 3), np.float16) for b in range(bits)])
    wz = (r.integers(-3, 1, (n, k // group)) / 4).astype(np.float16)
    mod = HLQLinear.from_export_arrays(wq, ws, wz, group, None, cuda)
    y = mod(torch.from_numpy(x).to(cuda)).cpu().numpy()
    assert np.array_equal(y.astype(np.float64), O.gemm_f64(x, wq, ws, wz, group))


@pytest.mark.parametrize("m", [16, 32, 64])
@pytest.mark.parametrize("k,n", LLAMA2_13B_PREFILL_SHAPES)
def test_llama2_13b_prefill_shapes(cuda, m, k, n):
    L = make_layer(k, n, bits=2, group=128, m=m, seed=11)
    _, y = gemm(L, cuda)
    w = O.dequantize(L.w_quant, L.w_scale, L.w_zero, 128, np.float32)
    ref = L.x.astype(np.float64) @ w.astype(np.float64).T
    assert O.rel_err(y, ref) <= TOL


@pytest.mark.parametrize("m", [16, 32, 64])
@pytest.mark.parametrize("bits,group", [(1, 128), (3, 128), (4, 64), (2, 64)])
def test_prefill_shape_other_formats(cuda, m, bits, group):
    """The instances of the other formats at a LLaMA-2-13B shape (5120 x 5120: 40 units per column, 80 column
    blocks, K cut into slices that meet through the workspace): every row count class x planes 1, 3, 4 and
    groups of 64, against the float64 oracle; bit-identical repeats."""
    k, n = 5120, 5120
    L = make_layer(k, n, bits=bits, group=group, m=m, seed=100 + bits + m)
    _, y = gemm(L, cuda)
    _, y2 = gemm(L, cuda)
    w = O.dequantize(L.w_quant, L.w_scale, L.w_zero, group, np.float32)
    ref = L.x.astype(np.float64) @ w.astype(np.float64).T
    assert O.rel_err(y, ref) <= TOL
    assert np.array_equal(y, y2)


@pytest.mark.parametrize("kparts", [0, 8])
@pytest.mark.parametrize("ksplit", [1, 2, 3, 0])
@pytest.mark.parametrize("m,k,n,bits,group", [(16, 1024, 100, 2, 128), (64, 1280, 320, 2, 128), (40, 1152, 576, 3, 64),
                                               (7, 896, 64, 4, 128), (33, 640, 200, 1, 64)])
def test_gemm_every_launch_shape(cuda, kparts, ksplit, m, k, n, bits, group):
    """Every cut of K into slices across workgroups, including a last column block past N, slices of
    unequal length, slices shorter than the eight waves of a workgroup and launches of two row tiles,
    against the float64 oracle; a second call on the same workspace
    must give the same bits (arrival counters are left at zero)."""
    from elutq_amd import _lib
    L = make_layer(k, n, bits=bits, group=group, m=m, seed=k + n + kparts, bias=True)
    mod = HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, L.group, L.bias, cuda)
    x = torch.from_numpy(L.x).to(cuda)
    ncb = -(-n // 64)
    ws = torch.zeros(64 * 1024 + (k // 128) * 64 * ncb * 64 * 4, dtype=torch.uint8, device=cuda)
    ref = O.gemm_f64(L.x, L.w_quant, L.w_scale, L.w_zero, group, L.bias)
    outs = []
    for _ in range(2):
        y = torch.full((m, n), float("nan"), dtype=torch.float16, device=cuda)
        rc = _lib.lib().elutq_hlq_gemm_f16_tuned(mod.planes.data_ptr(), mod.scales.data_ptr(), mod.zeros.data_ptr(),
                                                 mod.bias.data_ptr(), x.data_ptr(), y.data_ptr(), m, k, n, bits, group,
                                                 ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream,
                                                 kparts, ksplit)
        assert rc == 0
        torch.cuda.synchronize()
        outs.append(y.cpu().numpy())
    assert O.rel_err(outs[0], ref) <= TOL
    assert np.array_equal(outs[0], outs[1])


def test_gemm_tuned_rejects_bad_shapes(cuda):
    from elutq_amd import _lib
    L = make_layer(512, 64, bits=2, group=128, m=4, seed=1)
    mod = HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, L.group, None, cuda)
    x = torch.from_numpy(L.x).to(cuda)
    y = torch.empty(4, 64, dtype=torch.float16, device=cuda)
    ws = torch.zeros(64 * 1024, dtype=torch.uint8, device=cuda)
    call = lambda kp, ks, wsb: _lib.lib().elutq_hlq_gemm_f16_tuned(
        mod.planes.data_ptr(), mod.scales.data_ptr(), mod.zeros.data_ptr(), None, x.data_ptr(), y.data_ptr(), 4, 512, 64,
        2, 128, ws.data_ptr(), wsb, torch.cuda.current_stream().cuda_stream, kp, ks)
    assert call(3, 0, ws.numel()) == -7          # K parts: 8 (or 0 for the default, which is 8)
    assert call(4, 0, ws.numel()) == -7
    assert call(8, 5, ws.numel()) == -7          # more slices than units
    assert call(8, 2, ws.numel()) == -5          # two slices need room for partial sums
    assert call(8, 1, 0) == 0                    # one slice needs no workspace
    torch.cuda.synchronize()
