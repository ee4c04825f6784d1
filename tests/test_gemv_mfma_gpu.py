"""The matrix-core GEMV kernel (ELUTQ_GEMV_ENGINE_MFMA: plane bits as fp4 operands of v_mfma_f32_32x32x64_f8f6f4
against fp4 base-7 digits of the activations) behind the same C-ABI entry points as the LUT kernel, to the same bars:
float64 oracle within rel_err <= 1e-2 (observed: the final fp16 rounding), bit-exact where the arithmetic is exact,
the fused prologues / epilogue and the hand-over of K slices bit for bit what the unfused calls give, and within an
fp16 rounding of the LUT kernel on the same inputs.  Reference path: arm_gemm (m = 1),
C++/ops/src/arm/arm_gemm.cpp:248-360, arm_t_mac_kernal.cpp:364-469."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from elutq_amd import _lib
from elutq_amd.hlq_linear import HLQLinear
from elutq_amd.synth import LLAMA3_8B_SHAPES, make_layer
from oracle import hlq_oracle as O

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.fixture(autouse=True)
def mfma_engine():
    _lib.set_gemv_engine("mfma")
    yield
    _lib.set_gemv_engine("auto")


def to_mod(L, dev, ksplit=0, waves=0):
    m = HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, L.group, L.bias, dev)
    m.ksplit, m.waves = ksplit, waves
    return m


def run(m, x, dev):
    y = m(torch.from_numpy(np.ascontiguousarray(x)).to(dev))
    torch.cuda.synchronize()
    return y.cpu().numpy()


@pytest.mark.parametrize("k,n,bits,group", [
    (256, 64, 2, 128), (512, 128, 2, 128), (1024, 256, 3, 128), (1024, 192, 2, 64), (384, 70, 2, 128), (128, 1, 1, 128),
    (640, 100, 4, 64), (2048, 512, 4, 128), (384, 64, 3, 64), (5120, 320, 2, 128), (8192, 128, 2, 128), (1152, 96, 1, 64),
])
@pytest.mark.parametrize("ksplit,waves", [(0, 0), (1, 0), (2, 0), (3, 16), (1, 8)])
def test_mfma_gemv_matches_oracle(cuda, k, n, bits, group, ksplit, waves):
    L = make_layer(k, n, bits=bits, group=group, seed=k + n + bits, bias=(n % 3 == 0))
    ks = min(ksplit, k // 128)
    m = to_mod(L, cuda, ks, waves)
    if m.slices == 0:
        pytest.skip("more than two unit pairs per wave: refused (covered below)")
    y = run(m, L.x, cuda)[0]
    ref = O.gemv_f64(L.x[0], L.w_quant, L.w_scale, L.w_zero, group, L.bias)
    assert y.shape == (n,) and y.dtype == np.float16
    assert O.rel_err(y, ref) <= TOL, (k, n, bits, group, ks, waves)
    assert np.max(np.abs(y.astype(np.float64) - ref)) <= 2.0 ** -10 * max(1.0, np.max(np.abs(ref)))
    assert np.array_equal(y, run(m, L.x, cuda)[0])


@pytest.mark.parametrize("k,n,bits,group,bias", [(4224, 16640, 2, 128, False), (8192, 16500, 3, 64, True), (4096, 16400, 1, 128, False)])
def test_mfma_wide_layers_stream_over_all_of_k(cuda, k, n, bits, group, bias):
    """A plain call on a layer with more column blocks than compute units runs on the streaming kernel (every workgroup an
    equal share of the column blocks over all of K; with the engine on its default only where K > 4096): an odd unit
    count, ragged N, bias, more pairs than waves; 4096 sampled columns against the float64 oracle evaluated on those
    columns, bit-identical repeats, y(-x) = -y(x) exactly, and a column slice of the layer gives the same columns."""
    L = make_layer(k, n, bits=bits, group=group, seed=k + n, bias=bias)
    for engine in ("mfma", "auto"):
        _lib.set_gemv_engine(engine)
        m = to_mod(L, cuda)
        print(f"wide layer K={k} N={n} engine {engine}", flush=True)
        y = run(m, L.x, cuda)[0]
        idx = np.sort(np.random.default_rng(n).choice(n, 4096, replace=False))
        idx[:3], idx[-3:] = (0, 1, 63), (n - 64, n - 2, n - 1)
        ref = O.gemv_f64(L.x[0], L.w_quant[:, idx], L.w_scale[:, idx], L.w_zero[idx], group, None if L.bias is None else L.bias[idx])
        assert O.rel_err(y[idx], ref) <= TOL
        assert np.max(np.abs(y[idx].astype(np.float64) - ref)) <= 2.0 ** -10 * max(1.0, np.max(np.abs(ref)))
        assert np.array_equal(y, run(m, L.x, cuda)[0])
        if not bias:
            assert np.array_equal(-run(m, (-L.x).astype(np.float16), cuda)[0], y)
        sub = HLQLinear.from_export_arrays(L.w_quant[:, 4096:8192], L.w_scale[:, 4096:8192], L.w_zero[4096:8192], group,
                                           None if L.bias is None else L.bias[4096:8192], cuda)
        ys = run(sub, L.x, cuda)[0]
        assert np.max(np.abs(ys.astype(np.float64) - y[4096:8192].astype(np.float64))) <= 2.0 ** -9 * max(1.0, np.max(np.abs(ref)))


def test_mfma_refuses_more_than_two_pairs_per_wave(cuda):
    L = make_layer(4096, 64, bits=2, group=128, seed=1)
    m = to_mod(L, cuda, 1, 2)                          # 16 pairs on 2 waves
    with pytest.raises(_lib.ElutqError):
        m(torch.from_numpy(L.x).to(cuda))


def test_mfma_takes_whole_units_only(cuda):
    """K that ends half way through the last unit of 128 (group 64) is the LUT kernels' business: the matrix-core
    kernel refuses it (the tests of this file run with the engine pinned to it)."""
    L = make_layer(320, 64, bits=2, group=64, seed=1)
    with pytest.raises(_lib.ElutqError):
        to_mod(L, cuda)(torch.from_numpy(L.x).to(cuda))


@pytest.mark.parametrize("bits,group,ksplit", [(2, 128, 1), (2, 128, 2), (3, 64, 0), (4, 128, 3), (1, 64, 0)])
def test_mfma_bit_exact_on_integer_inputs(cuda, lutref, bits, group, ksplit):
    """x in {-2..2}, power-of-two scales, quarter-integer zeros: every digit, product and partial sum is exactly
    representable, so GPU == float64 == the reference's fp16 chain, bit for bit."""
    r = np.random.default_rng(5)
    k, n = 768, 128
    x = r.integers(-2, 3, (1, k)).astype(np.float16)
    wq = O.pack_planes(r.integers(0, 2, (bits, n, k), dtype=np.uint8))
    ws = np.stack([np.full((n, k // group), 2.0 ** (b - 3), np.float16) for b in range(bits)])
    wz = (r.integers(-3, 1, (n, k // group)) / 4).astype(np.float16)
    y64 = O.gemv_f64(x[0], wq, ws, wz, group)
    m = HLQLinear.from_export_arrays(wq, ws, wz, group, None, cuda)
    m.ksplit = ksplit
    y = run(m, x, cuda)[0]
    assert np.array_equal(y.astype(np.float64), y64)
    yc = lutref.RefWeight(wq, ws, wz, group, 4).gemv(x[0])
    assert np.array_equal(y.view(np.uint16), yc.view(np.uint16))


def test_mfma_closed_forms_unit_vectors_and_range(cuda):
    L = make_layer(512, 128, bits=2, group=128, seed=31)
    x64 = L.x[0].astype(np.float64)
    xs = x64.reshape(-1, 128).sum(1)
    z, s = L.w_zero.astype(np.float64), L.w_scale.astype(np.float64)
    zero = HLQLinear.from_export_arrays(np.zeros_like(L.w_quant), L.w_scale, L.w_zero, 128, None, cuda)
    assert O.rel_err(run(zero, L.x, cuda)[0], z @ xs) <= 2e-3
    ones = HLQLinear.from_export_arrays(np.full_like(L.w_quant, 255), L.w_scale, L.w_zero, 128, None, cuda)
    assert O.rel_err(run(ones, L.x, cuda)[0], (s.sum(0) + z) @ xs) <= 2e-3
    # x = e_k returns column k of W, rounded once to fp16 -- for every position of a chunk and of a dword
    m = to_mod(L, cuda)
    w = O.dequantize(L.w_quant, L.w_scale, L.w_zero, 128)
    for kk in (0, 1, 2, 3, 28, 29, 30, 31, 32, 63, 64, 127, 128, 255, 256, 300, 510, 511):
        e = np.zeros((1, 512), np.float16)
        e[0, kk] = 1
        y = run(m, e, cuda)[0]
        assert np.array_equal(y, w[:, kk].astype(np.float32).astype(np.float16)), kk
    # the largest activation of a half unit is held exactly by its base-7 digits: against a one-plane layer with scale 0.5
    # and zero 0 a single activation of any magnitude and mantissa must come back as 0.5 * x where the plane bit is set,
    # bit for bit
    r = np.random.default_rng(3)
    one = r.integers(0, 2, (1, 128, 512), dtype=np.uint8)
    half = HLQLinear.from_export_arrays(O.pack_planes(one), np.full((1, 128, 4), 0.5, np.float16), np.zeros((128, 4), np.float16),
                                        128, None, cuda)
    for _ in range(32):
        kk = int(r.integers(512))
        val = np.float16(r.uniform(1, 2) * 2.0 ** r.integers(-11, 12) * r.choice([-1, 1]))
        e = np.zeros((1, 512), np.float16)
        e[0, kk] = val
        y = run(half, e, cuda)[0]
        assert np.array_equal(y, (one[0, :, kk].astype(np.float32) * np.float32(val) * np.float32(0.5)).astype(np.float16)), (kk, val)
        # beside a much larger activation in the same half unit the small one keeps the bits above 2^-18 of the large one
        if abs(float(val)) >= 512:
            continue
        e[0, kk ^ 1] = np.float16(float(val) * 64)
        y = run(half, e, cuda)[0].astype(np.float64)
        want = 0.5 * (one[0, :, kk] * np.float64(val) + one[0, :, kk ^ 1] * np.float64(e[0, kk ^ 1]))
        assert np.max(np.abs(y - want)) <= 2.0 ** -10 * np.max(np.abs(want)) + 1e-12, (kk, val)
    # power-of-two scaling of x, tiny and large activations, a unit of zeros, one activation 2^13 times the rest
    L = make_layer(1024, 256, bits=2, group=128, seed=41)
    m = to_mod(L, cuda)
    for f in (2.0 ** -10, 4.0, 2.0 ** 8):
        xf = (L.x.astype(np.float32) * f).astype(np.float16)
        assert O.rel_err(run(m, xf, cuda)[0], O.gemv_f64(xf[0], L.w_quant, L.w_scale, L.w_zero, 128)) <= 2e-3
    xz = L.x.copy()
    xz[0, 128:256] = 0
    assert O.rel_err(run(m, xz, cuda)[0], O.gemv_f64(xz[0], L.w_quant, L.w_scale, L.w_zero, 128)) <= 2e-3
    xw = (L.x.astype(np.float32) * 2.0 ** -6).astype(np.float16)
    xw[0, 5] = np.float16(64.0)
    assert O.rel_err(run(m, xw, cuda)[0], O.gemv_f64(xw[0], L.w_quant, L.w_scale, L.w_zero, 128)) <= 2e-3
    yn = run(m, (-L.x).astype(np.float16), cuda)[0]
    assert np.array_equal(-yn, run(m, L.x, cuda)[0])


@pytest.mark.parametrize("name", ["q_proj", "k_proj", "gate_proj", "down_proj"])
@pytest.mark.parametrize("bits,group", [(2, 128), (3, 128), (2, 64)])
def test_mfma_llama3_8b_shapes_and_the_lut_kernel(cuda, name, bits, group):
    k, n = LLAMA3_8B_SHAPES[name]
    L = make_layer(k, n, bits=bits, group=group, seed=7)
    m = to_mod(L, cuda)
    print(f"mfma {name} K={k} N={n} w{bits}g{group}", flush=True)
    y = run(m, L.x, cuda)[0]
    w = O.dequantize(L.w_quant, L.w_scale, L.w_zero, group, np.float32)
    ref = w.astype(np.float64) @ L.x[0].astype(np.float64)
    assert O.rel_err(y, ref) <= TOL
    assert np.max(np.abs(y.astype(np.float64) - ref)) <= 2.0 ** -10 * max(1.0, np.max(np.abs(ref)))
    _lib.set_gemv_engine("lut")
    y_lut = run(m, L.x, cuda)[0]
    assert np.max(np.abs(y.astype(np.float64) - y_lut.astype(np.float64))) <= 2.0 ** -9 * max(1.0, np.max(np.abs(ref)))


@pytest.mark.parametrize("n,bits,group", [(28672, 2, 128), (28672, 3, 64)])
def test_mfma_column_block_runs_with_the_rmsnorm_prologue(cuda, n, bits, group):
    k = 4096
    L = make_layer(k, n, bits=bits, group=group, seed=17)
    mod = HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, group, None, cuda)
    print(f"mfma fused run K={k} N={n} w{bits}g{group}", flush=True)
    g = torch.Generator(device=cuda).manual_seed(3)
    w = (1 + 0.1 * torch.randn(k, generator=g, device=cuda)).half()
    res = torch.randn(1, n, generator=g, device=cuda).half()
    ws = torch.zeros(mod.workspace_bytes, dtype=torch.uint8, device=cuda)
    idx = np.sort(np.random.default_rng(n).choice(n, 4096, replace=False))
    idx[:3], idx[-3:] = (0, 1, 63), (n - 64, n - 2, n - 1)
    x = (torch.randn(1, k, generator=g, device=cuda) * 3).half()
    xf = x.float()
    h = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5) * w.float()).half()
    ref = O.gemv_f64(h.cpu().numpy()[0], L.w_quant[:, idx], L.w_scale[:, idx], L.w_zero[idx], group)
    out = torch.empty(1, n, dtype=torch.float16, device=cuda)
    mod.gemv_fused(x, out, ws, prologue=1, norm_weight=w, eps=1e-5, residual=res)
    assert O.rel_err(out.cpu().numpy()[0, idx], ref + res.cpu().numpy()[0, idx].astype(np.float64)) <= TOL
    sign = torch.where(torch.rand(1, k, generator=g, device=cuda) < 0.5, -1.0, 1.0)
    h2 = (sign * w.float()).half()
    mod.gemv_fused((2 * sign).half(), out, ws, prologue=1, norm_weight=w, eps=0.0)
    assert torch.equal(out, mod(h2))                       # fp16(x * 0.5 * w) = +-w exactly: fused == plain, bit for bit


@pytest.mark.parametrize("k,n,bits,group", [(1024, 256, 2, 128), (1536, 192, 4, 64), (14336, 4096, 2, 128)])
def test_mfma_silu_prologue_residual_and_handed_over_slices(cuda, k, n, bits, group):
    L = make_layer(k, n, bits=bits, group=group, seed=7)
    mod = HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, group, None, cuda)
    g = torch.Generator(device=cuda).manual_seed(2)
    gu = torch.randn(1, 2 * k, generator=g, device=cuda).half()
    res = torch.randn(1, n, generator=g, device=cuda).half()
    out = torch.empty(1, n, dtype=torch.float16, device=cuda)
    ws = torch.zeros(mod.workspace_bytes, dtype=torch.uint8, device=cuda)
    mod.gemv_fused(gu, out, ws, prologue=2, residual=res)
    act = (F.silu(gu[:, :k].float()) * gu[:, k:].float()).half()
    if k * n <= 1 << 22:
        ref = O.gemv_f64(act.cpu().numpy()[0], L.w_quant, L.w_scale, L.w_zero, group) + res.cpu().numpy()[0].astype(np.float64)
        assert O.rel_err(out.cpu().numpy()[0], ref) <= TOL
    # the same call with its K slices left unsummed: slices + residual, summed in order and rounded once, is the output
    mod.ksplit = max(mod.slices, 2)
    n_s = mod.slices
    assert 2 <= n_s <= 4
    want = torch.empty_like(out)
    mod.gemv_fused(gu, want, ws, prologue=2, residual=res)
    slices = torch.zeros(n_s, n, dtype=torch.float32, device=cuda)
    mod.gemv_fused(gu, out, ws, prologue=2, slices_out=slices)
    acc = slices[0].clone()
    for i in range(1, n_s):
        acc = acc + slices[i]
    assert torch.equal((acc + res[0].float()).half(), want[0])
    # a consumer that takes them in its RMSNorm prologue forms that same x and writes it out
    if n % 128 == 0:
        Lc = make_layer(n, 320, bits=2, group=128, seed=9)
        cons = HLQLinear.from_export_arrays(Lc.w_quant, Lc.w_scale, Lc.w_zero, 128, None, cuda)
        nw = (1 + 0.1 * torch.randn(n, generator=g, device=cuda)).half()
        y_direct = torch.empty(1, 320, dtype=torch.float16, device=cuda)
        cons.gemv_fused(want, y_direct, ws, prologue=1, norm_weight=nw, eps=1e-5)
        y_handed = torch.empty_like(y_direct)
        x_out = torch.zeros(1, n, dtype=torch.float16, device=cuda)
        cons.gemv_fused(res, y_handed, ws, prologue=1, norm_weight=nw, eps=1e-5, slices_in=slices, x_out=x_out)
        assert torch.equal(x_out, want) and torch.equal(y_handed, y_direct)


@pytest.mark.parametrize("bad", [float("nan"), float("inf")])
def test_mfma_non_finite_activations_reach_the_output(cuda, bad):
    L = make_layer(1024, 192, bits=2, group=128, seed=41)
    m = to_mod(L, cuda)
    x = L.x.copy()
    x[0, 517] = bad
    y = run(m, x, cuda)[0]
    assert not np.any(np.isfinite(y.astype(np.float32)))


def test_engine_selector(cuda):
    L = _lib.lib()
    assert L.elutq_hlq_get_gemv_engine() == 2
    assert L.elutq_hlq_set_gemv_engine(7) == -7 and L.elutq_hlq_get_gemv_engine() == 2
    assert L.elutq_hlq_set_gemv_engine(1) == 0 and L.elutq_hlq_get_gemv_engine() == 1
    # slices start on a unit pair under the matrix-core kernel: 2 units are one slice, under the LUT kernel two
    assert L.elutq_hlq_gemv_slices(256, 64, 2, 128, 0, 0) == 2
    assert L.elutq_hlq_set_gemv_engine(2) == 0
    assert L.elutq_hlq_gemv_slices(256, 64, 2, 128, 0, 0) == 1
