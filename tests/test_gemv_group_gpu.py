"""Grouped launch of independent GEMVs (elutq_hlq_gemv_group_*).  On the LUT engine against the single-GEMV entry
point: same tiles, same K slicing, so the same bits.  On the matrix-core engine (the library's own choice for a group
whose layers have whole units of 128 k) a tile covers all of K, so the sums differ from the single-GEMV launch in
order only: the float64 oracle to the dense path's bars, bit-identical repeats, bit-exact where the arithmetic is
exact, and within an fp16 rounding of the LUT engine."""
import ctypes

import numpy as np
import pytest
import torch

from elutq_amd import _lib
from elutq_amd.hlq_linear import GemvGroup, HLQLinear
from elutq_amd.synth import LLAMA3_8B_SHAPES, make_device_layer, make_layer
from oracle import hlq_oracle as O

pytestmark = pytest.mark.gpu


def single(mod, x, ksplit):
    y = torch.empty(1, mod.out_features, dtype=torch.float16, device=x.device)
    ws = torch.zeros(mod.workspace_bytes, dtype=torch.uint8, device=x.device)
    rc = _lib.lib().elutq_hlq_gemv_f16_tuned(mod.planes.data_ptr(), mod.scales.data_ptr(), mod.zeros.data_ptr(),
                                             mod.bias.data_ptr() if mod.bias is not None else None, x.data_ptr(),
                                             y.data_ptr(), mod.in_features, mod.out_features, mod.bits, mod.group_size,
                                             ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream, ksplit, 16)
    assert rc == 0
    return y


@pytest.fixture
def lut_engine():
    _lib.set_gemv_engine("lut")
    yield
    _lib.set_gemv_engine("auto")


@pytest.mark.parametrize("bits,group", [(2, 128), (3, 128), (2, 64), (4, 64), (1, 128)])
def test_group_equals_single_calls(cuda, lut_engine, bits, group):
    shapes = [(512, 128), (1024, 70), (4096, 256), (8192, 64), (128, 1), (9216, 130), (640, 192)]
    if group == 64:
        shapes += [(704, 100), (4160, 64)]                        # K ends half way through the last unit of 128
    layers = [make_layer(k, n, bits=bits, group=group, seed=10 * i + bits, bias=(i % 2 == 0)) for i, (k, n) in enumerate(shapes)]
    mods = [HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, L.group, L.bias, cuda) for L in layers]
    xs = [torch.from_numpy(L.x).to(cuda) for L in layers]
    ys = [torch.full((1, L.n), float("nan"), dtype=torch.float16, device=cuda) for L in layers]
    grp = GemvGroup(mods, xs, ys)
    for rep in range(2):                                          # the second run finds the arrival counters at zero
        for y in ys:
            y.fill_(float("nan"))
        grp.run()
        torch.cuda.synchronize()
        for L, mod, x, y in zip(layers, mods, xs, ys):
            ref = O.gemv_f64(L.x[0], L.w_quant, L.w_scale, L.w_zero, L.group, L.bias)
            assert O.rel_err(y[0].cpu().numpy(), ref) <= 1e-2
            assert any(torch.equal(y, single(mod, x, ks)) for ks in range(1, 9)), (L.k, L.n, rep)   # same bits as one of the K slicings
    grp.close()


def test_group_of_a_whole_layer_at_full_size(cuda, lut_engine):
    names = list(LLAMA3_8B_SHAPES)
    mods = [make_device_layer(*LLAMA3_8B_SHAPES[n], 2, 128, seed=i, device=cuda) for i, n in enumerate(names)]
    xs = [torch.randn(1, m.in_features, device=cuda).half() for m in mods]
    ys = [torch.zeros(1, m.out_features, dtype=torch.float16, device=cuda) for m in mods]
    grp = GemvGroup(mods * 3, xs * 3, [y for y in ys] + [torch.zeros_like(y) for y in ys] + [torch.zeros_like(y) for y in ys])
    grp.run()
    torch.cuda.synchronize()
    for m, x, y in zip(mods, xs, ys):
        w = m.dequantize().float()
        ref = x.float() @ w.t()
        assert (y.float() - ref).abs().max() <= 1e-2 * ref.pow(2).mean().sqrt()
        assert torch.equal(y, single(m, x, -(-(m.in_features // 128) * 2 // 64)))
    # captured in a graph and replayed with eager work in between
    g = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        grp.run()
    s.synchronize()
    with torch.cuda.graph(g, stream=s):
        grp.run()
    want = [y.clone() for y in ys]
    for _ in range(3):
        for y in ys:
            y.zero_()
        g.replay()
        torch.cuda.synchronize()
        _ = torch.randn(32, 32, device=cuda) @ torch.randn(32, 32, device=cuda)
        assert all(torch.equal(a, b) for a, b in zip(ys, want))
    grp.close()


@pytest.mark.parametrize("engine", ["auto", "mfma"])
@pytest.mark.parametrize("bits,group", [(2, 128), (3, 128), (2, 64), (4, 64), (1, 128), (4, 128), (3, 64), (1, 64)])
def test_group_on_the_matrix_cores_matches_oracle(cuda, engine, bits, group):
    """Layers of every kind in one group -- one unit, an odd unit count, more pairs than waves, ragged N, a single
    column, more column blocks than a tile holds, bias -- against the float64 oracle; repeats give the same bits
    (the second run also finds the ring and the LDS tables as the first left them)."""
    _lib.set_gemv_engine(engine)
    try:
        shapes = [(512, 128), (1024, 70), (4096, 256), (8192, 64), (128, 1), (9216, 130), (640, 192), (384, 1100),
                  (14336, 192), (256, 64)]
        layers = [make_layer(k, n, bits=bits, group=group, seed=10 * i + bits, bias=(i % 2 == 0)) for i, (k, n) in enumerate(shapes)]
        mods = [HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, L.group, L.bias, cuda) for L in layers]
        xs = [torch.from_numpy(L.x).to(cuda) for L in layers]
        ys = [torch.full((1, L.n), float("nan"), dtype=torch.float16, device=cuda) for L in layers]
        grp = GemvGroup(mods, xs, ys)
        prev = None
        for rep in range(3):
            for y in ys:
                y.fill_(float("nan"))
            grp.run()
            torch.cuda.synchronize()
            outs = [y[0].cpu().numpy().copy() for y in ys]
            for L, o in zip(layers, outs):
                ref = O.gemv_f64(L.x[0], L.w_quant, L.w_scale, L.w_zero, L.group, L.bias)
                assert O.rel_err(o, ref) <= 1e-2, (L.k, L.n, rep)
                assert np.max(np.abs(o.astype(np.float64) - ref)) <= 2.0 ** -10 * max(1.0, np.max(np.abs(ref)))
            assert prev is None or all(np.array_equal(a, b) for a, b in zip(prev, outs))
            prev = outs
        grp.close()
    finally:
        _lib.set_gemv_engine("auto")


@pytest.mark.parametrize("bits,group", [(2, 128), (3, 64), (4, 128), (1, 64)])
def test_group_on_the_matrix_cores_is_exact_on_integer_inputs(cuda, bits, group):
    """x in {-2..2}, power-of-two scales, quarter-integer zeros: every digit, product and partial sum is exactly
    representable in fp32, so the grouped launch == the float64 result rounded once to fp16, bit for bit, whatever the
    order of its sums."""
    r = np.random.default_rng(7)
    layers = []
    for (k, n) in [(768, 128), (4096, 200), (9216, 64), (384, 520)]:
        L = make_layer(k, n, bits=bits, group=group, seed=k + n)
        L.x[:] = r.integers(-2, 3, (1, k)).astype(np.float16)
        L.w_scale[:] = (2.0 ** r.integers(-3, 1, L.w_scale.shape)).astype(np.float16)
        L.w_zero[:] = (r.integers(-8, 9, L.w_zero.shape) / 4.0).astype(np.float16)
        layers.append(L)
    mods = [HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, L.group, None, cuda) for L in layers]
    xs = [torch.from_numpy(L.x).to(cuda) for L in layers]
    ys = [torch.zeros(1, L.n, dtype=torch.float16, device=cuda) for L in layers]
    grp = GemvGroup(mods, xs, ys)
    grp.run()
    torch.cuda.synchronize()
    for L, y in zip(layers, ys):
        ref = O.gemv_f64(L.x[0], L.w_quant, L.w_scale, L.w_zero, L.group)
        assert np.array_equal(y[0].cpu().numpy(), ref.astype(np.float16))
    grp.close()


def test_group_of_whole_layers_on_both_engines(cuda):
    """Three LLaMA-3-8B layers' projections as one group on the library's choice of engine (the matrix cores)
    against the dense fp32 product and against the LUT engine's group: within an fp16 rounding; replayed from a
    captured graph with eager work in between, every replay the same bits."""
    names = list(LLAMA3_8B_SHAPES)
    mods = [make_device_layer(*LLAMA3_8B_SHAPES[n], 2, 128, seed=i, device=cuda) for i, n in enumerate(names)]
    xs = [torch.randn(1, m.in_features, device=cuda).half() for m in mods]
    out = {}
    for engine in ("auto", "lut"):
        _lib.set_gemv_engine(engine)
        try:
            ys = [torch.zeros(1, m.out_features, dtype=torch.float16, device=cuda) for m in mods * 3]
            grp = GemvGroup(mods * 3, xs * 3, ys)
            grp.run()
            torch.cuda.synchronize()
            for m, x, y in zip(mods, xs, ys):
                ref = x.float() @ m.dequantize().float().t()
                assert (y.float() - ref).abs().max() <= 1e-2 * ref.pow(2).mean().sqrt()
            for i in range(len(mods)):          # the copies of a layer: same sums, in an order that depends on where its tiles fall
                for j in (1, 2):
                    assert (ys[i].float() - ys[i + j * len(mods)].float()).abs().max() <= 2.0 ** -9 * max(1.0, ys[i].float().abs().max().item())
                    assert engine != "lut" or torch.equal(ys[i], ys[i + j * len(mods)])
            g = torch.cuda.CUDAGraph()
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                grp.run()
            s.synchronize()
            with torch.cuda.graph(g, stream=s):
                grp.run()
            want = [y.clone() for y in ys]
            for _ in range(3):
                for y in ys:
                    y.zero_()
                g.replay()
                torch.cuda.synchronize()
                _ = torch.randn(32, 32, device=cuda) @ torch.randn(32, 32, device=cuda)
                assert all(torch.equal(a, b) for a, b in zip(ys, want))
            out[engine] = want[:len(mods)]
            grp.close()
        finally:
            _lib.set_gemv_engine("auto")
    for a, b in zip(out["auto"], out["lut"]):
        assert (a.float() - b.float()).abs().max() <= 2.0 ** -9 * max(1.0, b.float().abs().max().item())


def test_group_rejects_bad_arguments(cuda, lut_engine):
    L = _lib.lib()
    m = make_device_layer(512, 64, 2, 128, seed=0, device=cuda)
    x = torch.zeros(1, 512, dtype=torch.float16, device=cuda)
    y = torch.zeros(1, 64, dtype=torch.float16, device=cuda)
    p = (_lib.GemvProblem * 1)()
    p[0].d_planes, p[0].d_scales, p[0].d_zeros = m.planes.data_ptr(), m.scales.data_ptr(), m.zeros.data_ptr()
    p[0].d_x, p[0].d_y, p[0].K, p[0].N = x.data_ptr(), y.data_ptr(), 512, 64
    plan = ctypes.c_void_p()
    assert L.elutq_hlq_gemv_group_create(ctypes.byref(p), 0, 2, 128, None, 0, ctypes.byref(plan)) == -2
    assert L.elutq_hlq_gemv_group_create(ctypes.byref(p), 1, 5, 128, None, 0, ctypes.byref(plan)) == -3
    p[0].K = 500
    assert L.elutq_hlq_gemv_group_create(ctypes.byref(p), 1, 2, 128, None, 0, ctypes.byref(plan)) == -2
    assert L.elutq_hlq_gemv_group_workspace_bytes(ctypes.byref(p), 1, 2, 128) == 0
    p[0].K, p[0].d_x = 512, None
    assert L.elutq_hlq_gemv_group_create(ctypes.byref(p), 1, 2, 128, None, 0, ctypes.byref(plan)) == -1
    p[0].d_x, p[0].K = x.data_ptr(), 8192                       # two slices need a workspace
    assert L.elutq_hlq_gemv_group_create(ctypes.byref(p), 1, 2, 128, None, 0, ctypes.byref(plan)) == -1
    assert L.elutq_hlq_gemv_group_run(None, None) == -1
    with pytest.raises(ValueError):
        GemvGroup([m], [x], [y, y])
