"""elutq_hlq_gemv_f16_static, the batch-1 GEMV that allocates nothing and takes no workspace (its arrival
counters and partial sums live in a device array inside the library), against elutq_hlq_gemv_f16 on the
same inputs: bit for bit, on two calls in a row of which the second is the smaller one, with a K-sliced
launch first so that the second call meets the array as the first one left it."""
import ctypes

import numpy as np
import pytest
import torch

from elutq_amd import _lib
from elutq_amd.hlq_linear import HLQLinear
from elutq_amd.synth import make_layer
from oracle import hlq_oracle as O

pytestmark = pytest.mark.gpu


def static_gemv(mod: HLQLinear, x: torch.Tensor) -> torch.Tensor:
    y = torch.full((1, mod.out_features), float("nan"), dtype=torch.float16, device=x.device)
    rc = _lib.lib().elutq_hlq_gemv_f16_static(
        mod.planes.data_ptr(), mod.scales.data_ptr(), mod.zeros.data_ptr(),
        mod.bias.data_ptr() if mod.bias is not None else None, x.data_ptr(), y.data_ptr(), mod.in_features,
        mod.out_features, mod.bits, mod.group_size, torch.cuda.current_stream(x.device).cuda_stream)
    _lib.check(rc, "elutq_hlq_gemv_f16_static")
    return y


def test_static_gemv_equals_the_workspace_entry_point_on_two_calls_in_a_row(cuda):
    L = _lib.lib()
    assert L.elutq_hlq_static_init() == 0
    assert L.elutq_hlq_static_scratch_bytes() == (64 << 10) + (2 << 20)
    # first a K-sliced launch (14336 x 4096: four slices meet in the array), then a smaller one (4096 x 1024,
    # also sliced), then one without slices; every one against the entry point that takes a workspace
    # ... and 14336 x 8192, whose four slices of 128 column blocks do not fit the slots of the array's head: arrival
    # counters at its start (cleared by the call's fill kernel), partial sums behind the first 64 KiB
    shapes = [(14336, 4096, 2, 128, False), (4096, 1024, 3, 64, True), (1024, 200, 2, 128, True), (4096, 6144, 2, 128, False),
              (14336, 8192, 2, 128, False)]
    for rep in range(2):
        for k, n, bits, group, bias in shapes:
            print(f"static gemv K={k} N={n} w{bits}g{group} pass {rep}", flush=True)
            lay = make_layer(k, n, bits=bits, group=group, seed=k + n + rep, bias=bias)
            mod = HLQLinear.from_export_arrays(lay.w_quant, lay.w_scale, lay.w_zero, group, lay.bias, cuda)
            x = torch.from_numpy(lay.x).to(cuda)
            want = mod(x)
            got = static_gemv(mod, x)
            torch.cuda.synchronize()
            assert torch.equal(got, want), (k, n, bits, group)
            if k * n <= 4096 * 1024:
                ref = O.gemv_f64(lay.x[0], lay.w_quant, lay.w_scale, lay.w_zero, group, lay.bias)
                assert O.rel_err(got.cpu().numpy()[0], ref) <= 1e-2
            # and again at once on the same stream: the second call finds the counters where the first left them
            assert torch.equal(static_gemv(mod, x), want)


def test_static_gemv_in_a_graph_and_its_limits(cuda):
    L = _lib.lib()
    assert L.elutq_hlq_static_init() == 0
    lay = make_layer(4096, 1024, bits=2, group=128, seed=77)
    mod = HLQLinear.from_export_arrays(lay.w_quant, lay.w_scale, lay.w_zero, 128, None, cuda)
    assert mod.slices > 1
    x = torch.from_numpy(lay.x).to(cuda)
    want = mod(x)
    y = torch.zeros(1, 1024, dtype=torch.float16, device=cuda)
    s = torch.cuda.Stream()
    args = (mod.planes.data_ptr(), mod.scales.data_ptr(), mod.zeros.data_ptr(), None, x.data_ptr(), y.data_ptr(),
            4096, 1024, 2, 128)
    with torch.cuda.stream(s):
        assert L.elutq_hlq_gemv_f16_static(*args, s.cuda_stream) == 0
    s.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        assert L.elutq_hlq_gemv_f16_static(*args, torch.cuda.current_stream().cuda_stream) == 0
    for _ in range(3):
        y.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want)
        _ = mod(x)                       # eager work with a workspace of its own between the replays
    # the matrix-core engine chooses its own K slices (whole unit pairs): the call sizes its check from the launch it makes
    _lib.set_gemv_engine("mfma")
    try:
        for k, n in ((14336, 4096), (4096, 1024), (6144, 256)):
            lay2 = make_layer(k, n, bits=2, group=128, seed=k + n)
            mod2 = HLQLinear.from_export_arrays(lay2.w_quant, lay2.w_scale, lay2.w_zero, 128, None, cuda)
            x2 = torch.from_numpy(lay2.x).to(cuda)
            want2 = mod2(x2)
            for _ in range(2):
                assert torch.equal(static_gemv(mod2, x2), want2), (k, n)
    finally:
        _lib.set_gemv_engine("auto")
    # argument errors are those of the workspace entry point; a shape beyond the array's size is refused
    one = ctypes.c_void_p(1)
    assert L.elutq_hlq_gemv_f16_static(None, one, one, None, one, one, 4096, 64, 2, 128, None) == -1
    assert L.elutq_hlq_gemv_f16_static(one, one, one, None, one, one, 4000, 64, 2, 128, None) == -2
    assert L.elutq_hlq_gemv_f16_static(one, one, one, None, one, one, 4096, 64, 5, 128, None) == -3
    # 28672 x 131072 at two planes: five slices x 131072 columns x 4 bytes = 2.5 MiB of partial sums
    assert L.elutq_hlq_gemv_slices(28672, 131072, 2, 128, 0, 0) * 131072 * 4 > (2 << 20)
    assert L.elutq_hlq_gemv_f16_static(one, one, one, None, one, one, 28672, 131072, 2, 128, None) == -9
    assert "static buffer" in L.elutq_status_string(-9).decode()
