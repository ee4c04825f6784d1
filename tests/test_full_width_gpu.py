"""The launches the LLaMA-3-8B decode figure actually runs, at their real widths.

The fused GEMV instance that walks runs of column blocks with the RMSNorm in its prologue carries
gate|up (4096 x 28672) in every layer and, for a model whose lm_head is quantized, the 4096 x 128256
lm_head with the final norm in front; a decode step at hidden 4096 / FFN 14336 / vocab 128256 with a
512-token cache selects launch shapes (column-block runs, two K slices of q|k|v summed by the sliced
attention, the 64-workgroup argmax) that a small model never reaches.
Reference ops: launch_pre_rms_norm (C++/ops/src/arm/arm_rmsnorm.cpp:25-84) in front of arm_gemm
(C++/ops/src/arm/arm_gemm.cpp:871-924); llama::forward (C++/examples/models/llama.cpp:185-763).
"""
import numpy as np
import pytest
import torch

from elutq_amd.hlq_linear import HLQLinear
from elutq_amd.llama_decode import LlamaDecoder, LlamaShape
from torch_glue_decode import TorchGlueDecoder
from elutq_amd.synth import make_layer
from oracle import hlq_oracle as O
from test_decode_gpu import densify

pytestmark = pytest.mark.gpu
TOL = 1e-2


def sampled(n, count=4096):
    idx = np.sort(np.random.default_rng(n).choice(n, count, replace=False))
    idx[:3], idx[-3:] = (0, 1, 63), (n - 64, n - 2, n - 1)            # block edges, first and last
    return idx


def torch_rmsnorm(x, w, eps):
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()).half()


@pytest.mark.parametrize("n,bits,group", [(28672, 2, 128), (28672, 3, 128), (28672, 2, 64), (128256, 2, 128)])
def test_fused_column_block_run_instance(cuda, n, bits, group):
    k = 4096
    L = make_layer(k, n, bits=bits, group=group, seed=17)
    mod = HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, group, None, cuda)
    assert mod.slices == 1 and (n + 63) // 64 > 256            # what makes the launch walk runs of column blocks
    print(f"fused run instance K={k} N={n} w{bits}g{group}", flush=True)
    g = torch.Generator(device=cuda).manual_seed(3)
    w = (1 + 0.1 * torch.randn(k, generator=g, device=cuda)).half()
    res = torch.randn(1, n, generator=g, device=cuda).half()
    ws = torch.zeros(mod.workspace_bytes, dtype=torch.uint8, device=cuda)
    idx = sampled(n)
    sub = (L.w_quant[:, idx], L.w_scale[:, idx], L.w_zero[idx])

    # (1) random activations: sampled columns against the float64 oracle on the fp16-rounded normalised x,
    #     without and with the residual
    x = (torch.randn(1, k, generator=g, device=cuda) * 3).half()
    h = torch_rmsnorm(x, w, 1e-5)
    ref = O.gemv_f64(h.cpu().numpy()[0], *sub, group)
    out = torch.empty(1, n, dtype=torch.float16, device=cuda)
    mod.gemv_fused(x, out, ws, prologue=1, norm_weight=w, eps=1e-5)
    y = out.cpu().numpy()[0]
    assert O.rel_err(y[idx], ref) <= TOL
    out_r = torch.empty_like(out)
    mod.gemv_fused(x, out_r, ws, prologue=1, norm_weight=w, eps=1e-5, residual=res)
    ref_r = ref + res.cpu().numpy()[0, idx].astype(np.float64)
    assert O.rel_err(out_r.cpu().numpy()[0, idx], ref_r) <= TOL
    # run-to-run determinism, and the plain instance on the pre-normalised x to within the rounding of h
    out2 = torch.empty_like(out)
    mod.gemv_fused(x, out2, ws, prologue=1, norm_weight=w, eps=1e-5)
    assert torch.equal(out, out2)
    y_plain = mod(h)
    assert (out.float() - y_plain.float()).abs().max() <= 2e-2 * y_plain.float().abs().max()

    # (2) activations of one magnitude: x = +-2 and eps = 0 make 1/rms exactly 0.5, so the prologue forms
    #     fp16(x * 0.5 * w) = +-w without any rounding and the fused instance must equal the plain
    #     column-block-run instance fed that vector bit for bit
    sign = torch.where(torch.rand(1, k, generator=g, device=cuda) < 0.5, -1.0, 1.0)
    x2 = (2 * sign).half()
    h2 = (sign * w.float()).half()
    assert torch.equal(torch_rmsnorm(x2, w, 0.0), h2)
    mod.gemv_fused(x2, out, ws, prologue=1, norm_weight=w, eps=0.0)
    assert torch.equal(out, mod(h2))
    assert O.rel_err(out.cpu().numpy()[0, idx], O.gemv_f64(h2.cpu().numpy()[0], *sub, group)) <= TOL


FULL = LlamaShape(n_layers=2, hidden=4096, n_heads=32, n_kv_heads=8, ffn=14336, vocab=128256, max_seq=640)


def test_decode_step_at_full_llama3_8b_width(cuda):
    """Two layers of the LLaMA-3-8B shape with its vocabulary and a 512-token cache: the fused launches
    against the same HLQ model under PyTorch glue and against the dense fp32 model, eager steps and graph
    replays, with the K slices handed to the consuming launch and summed by the producer."""
    print("decode step at full width: building models", flush=True)
    hip = LlamaDecoder(FULL, device=cuda, seed=5)
    hip_nd = LlamaDecoder(FULL, device=cuda, seed=5)
    hip_nd.defer_slices = hip_nd.defer_qkv = False
    graph = LlamaDecoder(FULL, device=cuda, seed=5)
    glue = TorchGlueDecoder(FULL, device=cuda, seed=5)
    dense = densify(TorchGlueDecoder(FULL, device=cuda, seed=5))
    models = (hip, hip_nd, graph, glue, dense)
    for m in models:
        m.fill_cache(512, seed=9)
        m.token.fill_(4242)
    # the launch shapes this test is about
    assert hip.layers[0].gate_up.out_features == 28672 and hip.layers[0].qkv.slices == 2
    assert hip.layers[0].down_proj.slices >= 2
    graph.capture()
    for step in range(4):
        print(f"decode step at full width: step {step}", flush=True)
        lh = hip.step().float()
        ln = hip_nd.step().float()
        lg = glue.step().float()
        ld = dense.step().float()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(lh, ln), step                       # who sums the K slices changes no bit
        assert torch.equal(graph._logits.float(), lh), step    # nor does a graph replay
        rms = ld.pow(2).mean().sqrt()
        assert (lh - lg).abs().max() <= 1e-2 * lg.pow(2).mean().sqrt(), step
        assert (lh - ld).abs().max() <= 2e-2 * rms, step
        assert int(hip.token) == int(hip_nd.token) == int(graph.token)
        assert int(hip.pos) == 513 + step
        for m in (glue, dense):                                # keep every model on the same token sequence
            m.token.copy_(hip.token)
    for a, b in zip(hip.layers, glue.layers):
        assert torch.equal(a.k_cache[:512], b.k_cache[:512])
        assert (a.k_cache[512:516].float() - b.k_cache[512:516].float()).abs().max() <= 2e-2
        assert (a.v_cache[512:516].float() - b.v_cache[512:516].float()).abs().max() <= 2e-2
    for a, b in zip(hip.layers, graph.layers):
        assert torch.equal(a.k_cache, b.k_cache) and torch.equal(a.v_cache, b.v_cache)


def test_the_32_layer_step_the_benchmark_times(cuda):
    """The decode configuration itself: 32 layers at the LLaMA-3-8B shape, 512-token cache, one HIP graph per
    token (what `bench.py` times) against eager steps of the same fused path, bit for bit, and against the same
    HLQ model under PyTorch glue -- every projection through the C ABI one call at a time, norms, RoPE, attention
    and residual adds as PyTorch operators in fp32 -- to within 3e-2 of the logits' rms after 32 layers."""
    shape = LlamaShape(n_layers=32, hidden=4096, n_heads=32, n_kv_heads=8, ffn=14336, vocab=128256, max_seq=640)
    print("32-layer decode step: building models", flush=True)
    graph = LlamaDecoder(shape, device=cuda, seed=11)
    eager = LlamaDecoder(shape, device=cuda, seed=11)
    glue = TorchGlueDecoder(shape, device=cuda, seed=11)
    for m in (graph, eager, glue):
        m.fill_cache(512, seed=3)
        m.token.fill_(77)
    graph.capture()
    worst = 0.0
    for step in range(3):
        print(f"32-layer decode step: step {step}", flush=True)
        le = eager.step().float()
        lg = glue.step().float()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(graph._logits.float(), le), step
        assert int(graph.token) == int(eager.token) and int(graph.pos) == 513 + step
        assert torch.isfinite(le).all()
        d = float((le - lg).abs().max() / lg.pow(2).mean().sqrt())
        worst = max(worst, d)
        assert d <= 3e-2, (step, d)
        # the greedy pick of the fused path is among the glue path's best few (random weights give near ties)
        assert int(eager.token) in torch.topk(lg.flatten(), 5).indices.tolist(), step
        glue.token.copy_(eager.token)
    print(f"32-layer decode step: fused - glue, max over logits / rms = {worst:.3e}", flush=True)
    for a, b in zip(eager.layers, graph.layers):
        assert torch.equal(a.k_cache, b.k_cache) and torch.equal(a.v_cache, b.v_cache)
