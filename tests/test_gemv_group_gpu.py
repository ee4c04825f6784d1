"""Grouped launch of independent GEMVs (elutq_hlq_gemv_group_*) against the single-GEMV entry
point: same tiles, same K slicing, so the same bits."""
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


@pytest.mark.parametrize("bits,group", [(2, 128), (3, 128), (2, 64), (4, 64), (1, 128)])
def test_group_equals_single_calls(cuda, bits, group):
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


def test_group_of_a_whole_layer_at_full_size(cuda):
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


def test_group_rejects_bad_arguments(cuda):
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
