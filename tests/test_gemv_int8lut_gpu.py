"""GPU parity of the int8-LUT mode of the batch-1 GEMV (elutq_hlq_gemv_int8lut_f16) through the C ABI.

The tables the kernel builds must be the ones the oracle's lut_int8 builds (same fp16 sums, same scale, same
rounding), so against gemv_int8lut_f64 -- the exact evaluation on those tables -- only fp32 summation order and
the final fp16 rounding remain: the dense path's bars apply (rel_err <= 1e-2, and 2^-10 of the largest output).
Against the exact oracle the mode is lossy by design; that distance is only bounded loosely.
"""
import numpy as np
import pytest
import torch

from elutq_amd import _lib
from elutq_amd.hlq_linear import HLQLinear
from elutq_amd.synth import make_layer
from oracle import hlq_oracle as O

pytestmark = pytest.mark.gpu
TOL = 1e-2


def to_mod(L, dev):
    return HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, L.group, L.bias, dev)


def run8(mod, x, dev):
    y = mod.gemv_int8lut(torch.from_numpy(np.ascontiguousarray(x)).to(dev).reshape(-1))
    torch.cuda.synchronize()
    return y.cpu().numpy()[0]


@pytest.mark.parametrize("k,n,bits,group", [
    (256, 64, 2, 128), (384, 70, 2, 128), (1024, 192, 3, 64), (640, 100, 4, 64), (128, 1, 1, 128),
    (2048, 512, 4, 128), (4096, 1024, 2, 128), (4096, 4096, 2, 128), (8192, 128, 2, 64), (4224, 96, 2, 64),
    (6400, 64, 3, 128), (14336, 256, 2, 128),
])
def test_matches_the_exact_evaluation_on_int8_tables(cuda, k, n, bits, group):
    L = make_layer(k, n, bits=bits, group=group, seed=k + n + bits, bias=(n % 3 == 0))
    print(f"int8-lut gemv K={k} N={n} w{bits}g{group}", flush=True)
    y = run8(to_mod(L, cuda), L.x, cuda)
    ref = O.gemv_int8lut_f64(L.x[0], L.w_quant, L.w_scale, L.w_zero, group, L.bias)
    assert y.shape == (n,) and y.dtype == np.float16
    assert O.rel_err(y, ref) <= TOL
    assert np.max(np.abs(y.astype(np.float64) - ref)) <= 2.0 ** -10 * max(1.0, np.max(np.abs(ref)))
    # lossy against the exact sum, but near it
    exact = O.gemv_f64(L.x[0], L.w_quant, L.w_scale, L.w_zero, group, L.bias)
    assert np.sqrt(np.mean((y.astype(np.float64) - exact) ** 2)) <= 0.1 * np.sqrt(np.mean(exact ** 2))


@pytest.mark.parametrize("group,seed", [(128, 1), (64, 2), (128, 3)])
def test_every_table_entry_shows_in_an_output(cuda, group, seed):
    """Column n has plane bits on one chunk of four activations only, set as the subset m: with unit plane scale and
    no zero point its output is scale[group] * q[chunk][m], one product rounded once -- so all 64 x 15 entries of the
    kernel's tables and every group scale are compared with the oracle's exactly, on activations of mixed magnitude."""
    k, chunks = 256, 64
    r = np.random.default_rng(seed)
    x = (r.standard_normal((1, k)) * np.exp2(r.integers(-6, 3, (1, k)))).astype(np.float16)
    x[0, 8:12] = [0.5, -0.5, 0.25, 0]                          # ties and cancellations inside a chunk
    n = chunks * 15
    planes = np.zeros((1, n, k), np.uint8)
    for c in range(chunks):
        for m in range(1, 16):
            for i in range(4):
                planes[0, c * 15 + m - 1, 4 * c + i] = m >> i & 1
    wq = O.pack_planes(planes)
    ws = np.ones((1, n, k // group), np.float16)
    wz = np.zeros((n, k // group), np.float16)
    mod = HLQLinear.from_export_arrays(wq, ws, wz, group, None, cuda)
    y = run8(mod, x, cuda)
    q, sc = O.lut_int8(x[0], group)
    want = (q[:, 1:].astype(np.float64) * np.repeat(sc.astype(np.float64), group // 4)[:, None]).reshape(-1)
    assert np.array_equal(want, O.gemv_int8lut_f64(x[0], wq, ws, wz, group))
    assert np.array_equal(y, want.astype(np.float16))


@pytest.mark.parametrize("group", [64, 128])
def test_tables_that_lose_nothing_give_the_exact_gemv_bits(cuda, group):
    """Integer activations with a largest subset sum of 127 per group: scale 1, entries = the sums themselves, so
    the mode returns what the exact GEMV returns -- the float64 result, bit for bit."""
    k, n = 512, 130
    r = np.random.default_rng(group)
    x = r.integers(-3, 4, (1, k)).astype(np.float16)
    for g in range(k // group):
        x[0, g * group:g * group + 4] = [100, 27, 0, 0]
    wq = O.pack_planes(r.integers(0, 2, (2, n, k), dtype=np.uint8))
    ws = np.stack([np.full((n, k // group), 0.25), np.full((n, k // group), 0.5)]).astype(np.float16)
    wz = np.full((n, k // group), -0.5, np.float16)
    mod = HLQLinear.from_export_arrays(wq, ws, wz, group, None, cuda)
    want = O.gemv_f64(x[0], wq, ws, wz, group)
    y = run8(mod, x, cuda)
    assert np.array_equal(y.astype(np.float64), want)
    assert np.array_equal(mod(torch.from_numpy(x).to(cuda)).cpu().numpy()[0], y)


def test_zero_groups_scaling_and_negation(cuda):
    """A group of zeros has scale 0 and contributes its zero term only; activations times a power of two give
    the outputs times that power; negated activations give negated outputs (round-to-even is symmetric)."""
    L = make_layer(1024, 128, bits=2, group=128, seed=21)
    x = L.x.copy()
    x[0, 256:512] = 0
    mod = to_mod(L, cuda)
    y = run8(mod, x, cuda)
    ref = O.gemv_int8lut_f64(x[0], L.w_quant, L.w_scale, L.w_zero, 128)
    assert np.all(np.isfinite(y)) and O.rel_err(y, ref) <= TOL
    y4 = run8(mod, (x.astype(np.float32) * 4).astype(np.float16), cuda)
    assert np.array_equal(y4.astype(np.float32), y.astype(np.float32) * 4)
    yn = run8(mod, -x, cuda)
    assert np.array_equal(-yn, y)
    assert np.array_equal(run8(mod, x, cuda), y)                 # run-to-run determinism (K slices meet in order)


def test_uniform_format_against_the_reference_op_order(cuda):
    """The reference's own weight format for this variant -- one scale per (channel, group), planes weighted by
    powers of two, no zero point -- as the HLQ special case, against the op-for-op fp16 restatement of arm_gemv."""
    L = make_layer(1024, 128, bits=3, group=128, seed=23)
    ws = np.stack([L.w_scale[0].astype(np.float32) * 2 ** b for b in range(3)]).astype(np.float16)
    mod = HLQLinear.from_export_arrays(L.w_quant, ws, np.zeros_like(L.w_zero), 128, None, cuda)
    y = run8(mod, L.x, cuda)
    chain = O.gemv_int8lut_chain_uniform(L.x[0], L.w_quant, L.w_scale[0], 128)
    ref = O.gemv_int8lut_f64(L.x[0], L.w_quant, ws, np.zeros_like(L.w_zero), 128)
    assert O.rel_err(y, ref) <= TOL
    assert np.max(np.abs(y.astype(np.float64) - chain.astype(np.float64))) <= 2e-2 * np.sqrt(np.mean(ref ** 2))


def test_runs_on_the_lut_kernel_whatever_engine_is_selected(cuda):
    L = make_layer(1024, 128, bits=2, group=128, seed=25)
    mod = to_mod(L, cuda)
    y = run8(mod, L.x, cuda)
    lib = _lib.lib()
    assert lib.elutq_hlq_set_gemv_engine(2) == 0               # the matrix-core engine for the exact GEMV
    try:
        assert np.array_equal(run8(mod, L.x, cuda), y)
    finally:
        assert lib.elutq_hlq_set_gemv_engine(0) == 0


def test_argument_errors(cuda):
    L = make_layer(256, 64, bits=2, group=128, seed=27)
    mod = to_mod(L, cuda)
    lib = _lib.lib()
    x = torch.zeros(256, dtype=torch.float16, device=cuda)
    y = torch.zeros(64, dtype=torch.float16, device=cuda)
    ws = torch.zeros(mod.workspace_bytes, dtype=torch.uint8, device=cuda)
    args = lambda **kw: (mod.planes.data_ptr(), mod.scales.data_ptr(), mod.zeros.data_ptr(), None, kw.get("x", x.data_ptr()),
                         y.data_ptr(), kw.get("k", 256), 64, kw.get("bits", 2), kw.get("group", 128), ws.data_ptr(), ws.numel(), None)
    assert lib.elutq_hlq_gemv_int8lut_f16(*args()) == 0
    assert lib.elutq_hlq_gemv_int8lut_f16(*args(x=None)) == -1
    assert lib.elutq_hlq_gemv_int8lut_f16(*args(bits=5)) == -3
    assert lib.elutq_hlq_gemv_int8lut_f16(*args(group=32)) == -4
    assert lib.elutq_hlq_gemv_int8lut_f16(*args(k=200)) == -2
    with pytest.raises(ValueError):
        mod.gemv_int8lut(torch.zeros(255, dtype=torch.float16, device=cuda))
