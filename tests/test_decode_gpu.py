"""Decode step (the caller of the hot path): whole-step parity of the HLQ model against the
same model with every HLQLinear replaced by a dense fp32 F.linear over its dequantized
weight, and HIP-graph replays against eager steps."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from elutq_amd.hlq_linear import HLQLinear
from elutq_amd.llama_decode import LlamaDecoder, LlamaShape, fuse_along_n
from torch_glue_decode import TorchGlueDecoder, make_decoder, rms_norm, rope
from elutq_amd.synth import make_device_layer

pytestmark = pytest.mark.gpu

SMALL = LlamaShape(n_layers=2, hidden=512, n_heads=8, n_kv_heads=2, ffn=1024, vocab=1000, max_seq=48)


class DenseLinear(torch.nn.Module):
    def __init__(self, m: HLQLinear):
        super().__init__()
        self.w = m.dequantize().float()
        self.b = None if m.bias is None else m.bias.float()

    def forward(self, x):
        return F.linear(x.float(), self.w, self.b).to(torch.float16)


def densify(model):
    for layer in model.layers:
        for name, mod in list(layer.named_children()):
            if isinstance(mod, HLQLinear):
                setattr(layer, name, DenseLinear(mod))
    return model


def test_fuse_along_n_is_concatenation(cuda):
    a = make_device_layer(256, 128, 2, 128, seed=1, device=cuda)
    b = make_device_layer(256, 64, 2, 128, seed=2, device=cuda)
    c = make_device_layer(256, 70, 2, 128, seed=3, device=cuda, bias=True)
    x = torch.randn(1, 256, device=cuda).half()
    f = fuse_along_n([a, b, c])
    y = f(x)
    bias_free = torch.cat([a(x), b(x), c(x)], dim=-1)
    assert y.shape == (1, 262) and torch.equal(y, bias_free)
    assert torch.equal(f.dequantize(), torch.cat([a.dequantize(), b.dequantize(), c.dequantize()]))


@pytest.mark.parametrize("fuse,impl", [(True, "hip"), (True, "torch"), (False, "torch")])
def test_decode_step_matches_dense_model(cuda, fuse, impl):
    hlq = make_decoder(impl, SMALL, device=cuda, seed=3, fuse=fuse)
    ref = densify(TorchGlueDecoder(SMALL, device=cuda, seed=3, fuse=fuse))
    for m in (hlq, ref):
        m.fill_cache(20, seed=5)
        m.token.fill_(7)
    for step in range(4):
        lh = hlq.step().float()
        lr = ref.step().float()
        rms = lr.pow(2).mean().sqrt()
        assert (lh - lr).abs().max() <= 2e-2 * rms, step
        assert int(hlq.pos) == 21 + step
        ref.token.copy_(hlq.token)          # keep both on the same token sequence
    # the cache row written at position 20 is identical up to fp16 rounding of the projections
    k0, k1 = hlq.layers[0].k_cache[20].float(), ref.layers[0].k_cache[20].float()
    assert (k0 - k1).abs().max() <= 1e-2 * k1.abs().max()


def test_fused_launches_match_torch_glue(cuda):
    """The five fused launches per layer against the same HLQ model run with PyTorch glue:
    same tokens, logits within fp16 rounding of the intermediate activations."""
    a = LlamaDecoder(SMALL, device=cuda, seed=6)
    b = TorchGlueDecoder(SMALL, device=cuda, seed=6)
    for m in (a, b):
        m.fill_cache(33, seed=8)
        m.token.fill_(11)
    for step in range(5):
        la, lb = a.step().float(), b.step().float()
        assert (la - lb).abs().max() <= 1e-2 * lb.pow(2).mean().sqrt(), step
        assert int(a.token) == int(b.token)
    for la_, lb_ in zip(a.layers, b.layers):
        assert (la_.k_cache[33:38].float() - lb_.k_cache[33:38].float()).abs().max() <= 2e-2
        assert torch.equal(la_.k_cache[:33], lb_.k_cache[:33])


@pytest.mark.parametrize("impl", ["hip", "torch"])
def test_graph_replay_equals_eager(cuda, impl):
    eager = make_decoder(impl, SMALL, device=cuda, seed=4)
    graph = make_decoder(impl, SMALL, device=cuda, seed=4)
    for m in (eager, graph):
        m.fill_cache(10, seed=2)
        m.token.fill_(3)
    graph.capture()
    toks_e, toks_g = [], []
    for _ in range(6):
        le = eager.step()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(graph._logits, le)
        toks_e.append(int(eager.token))
        toks_g.append(int(graph.token))
        _ = torch.randn(64, 64, device=cuda) @ torch.randn(64, 64, device=cuda)    # unrelated eager work between replays
    assert toks_e == toks_g and int(graph.pos) == 16


@pytest.mark.parametrize("d,nq,nkv,splits", [(128, 8, 2, 1), (128, 4, 4, 1), (64, 8, 2, 1), (32, 4, 1, 1),
                                             (128, 8, 2, 2), (128, 8, 2, 8), (128, 32, 8, 0), (128, 4, 4, 3), (64, 8, 2, 4)])
@pytest.mark.parametrize("pos", [0, 1, 3, 4, 5, 37, 63, 64, 65, 192, 193, 255, 300, 513, 768, 769, 1030])
def test_rope_cache_attention_kernel(cuda, d, nq, nkv, splits, pos):
    """elutq_decode_rope_attn_f16 / _split_f16 (cached positions divided among `splits`
    workgroups per head, 0 = default) against the PyTorch restatement of the reference ops
    (half-split RoPE, cache append, fp32-softmax GQA attention); two calls in a row on one
    workspace (the second must find the arrival counters at zero)."""
    check_rope_cache_attention(cuda, d, nq, nkv, splits, pos, max_seq=1100)


@pytest.mark.parametrize("d,nq,nkv,splits", [(128, 32, 8, 0), (128, 8, 2, 1), (128, 8, 2, 8), (128, 4, 4, 3), (64, 8, 2, 4)])
@pytest.mark.parametrize("pos", [2047, 4096, 8191])
def test_rope_cache_attention_kernel_long_context(cuda, d, nq, nkv, splits, pos):
    """The same check at the context lengths of a LLaMA-3 model (cache of 8192 positions)."""
    check_rope_cache_attention(cuda, d, nq, nkv, splits, pos, max_seq=8192)


def check_rope_cache_attention(cuda, d, nq, nkv, splits, pos, max_seq):
    from elutq_amd import _lib
    g = torch.Generator(device=cuda).manual_seed(pos * 7 + d)
    base = 10000.0
    L = _lib.lib()
    qkv = torch.randn(1, (nq + 2 * nkv) * d, generator=g, device=cuda).half()
    kc = torch.randn(max_seq, nkv, d, generator=g, device=cuda).half()
    vc = torch.randn(max_seq, nkv, d, generator=g, device=cuda).half()
    kc0, vc0 = kc.clone(), vc.clone()
    pos_t = torch.tensor([pos], dtype=torch.long, device=cuda)
    stream = torch.cuda.current_stream().cuda_stream
    ws = torch.zeros(L.elutq_decode_attn_workspace_bytes(nq, d, 0), dtype=torch.uint8, device=cuda)
    outs = []
    for _ in range(2):
        out = torch.zeros(1, nq * d, dtype=torch.float16, device=cuda)
        if splits == 1:
            rc = L.elutq_decode_rope_attn_f16(qkv.data_ptr(), kc.data_ptr(), vc.data_ptr(), pos_t.data_ptr(),
                                              out.data_ptr(), nq, nkv, d, max_seq, base, stream)
        else:
            rc = L.elutq_decode_rope_attn_split_f16(qkv.data_ptr(), kc.data_ptr(), vc.data_ptr(), pos_t.data_ptr(),
                                                    out.data_ptr(), nq, nkv, d, max_seq, base, splits, ws.data_ptr(),
                                                    ws.numel(), stream)
        assert rc == 0
        torch.cuda.synchronize()
        outs.append(out)
    assert torch.equal(outs[0], outs[1])
    assert not ws[:64 * 1024].any()
    out = outs[0]
    # reference
    inv = base ** (-torch.arange(0, d, 2, device=cuda, dtype=torch.float32) / d)
    ang = pos * inv
    q, k, v = qkv[0].split([nq * d, nkv * d, nkv * d])
    qr = rope(q.view(nq, d), ang.cos(), ang.sin())
    kr = rope(k.view(nkv, d), ang.cos(), ang.sin())
    kref, vref = kc0.clone(), vc0.clone()
    kref[pos], vref[pos] = kr, v.view(nkv, d)
    assert (kc[pos].float() - kref[pos].float()).abs().max() <= 4e-3 * kref[pos].float().abs().max()
    assert torch.equal(vc[pos], vref[pos])
    keep = torch.ones(max_seq, dtype=torch.bool, device=cuda)
    keep[pos] = False
    assert torch.equal(kc[keep], kc0[keep]) and torch.equal(vc[keep], vc0[keep])      # nothing else touched
    qg = qr.view(nkv, nq // nkv, d).float()
    sc = torch.matmul(qg, kref[:pos + 1].permute(1, 2, 0).float()) * d ** -0.5
    ctx = torch.matmul(torch.softmax(sc, -1), vref[:pos + 1].permute(1, 0, 2).float()).reshape(1, nq * d)
    assert (out.float() - ctx).abs().max() <= 5e-3 * max(1.0, float(ctx.abs().max()))


def test_rope_attn_rejects_bad_arguments(cuda):
    from elutq_amd import _lib
    L = _lib.lib()
    t = torch.zeros(4096, dtype=torch.float16, device=cuda)
    p = torch.zeros(1, dtype=torch.long, device=cuda)
    s = torch.cuda.current_stream().cuda_stream
    args = lambda nq, nkv, d: (t.data_ptr(), t.data_ptr(), t.data_ptr(), p.data_ptr(), t.data_ptr(), nq, nkv, d, 8, 1e4, s)
    assert L.elutq_decode_rope_attn_f16(*args(8, 3, 64)) == -2       # heads not a multiple of kv heads
    assert L.elutq_decode_rope_attn_f16(*args(8, 2, 256)) == -2      # head_dim > 128
    assert L.elutq_decode_rope_attn_f16(None, t.data_ptr(), t.data_ptr(), p.data_ptr(), t.data_ptr(), 8, 2, 64, 8, 1e4, s) == -1
    # a position outside the cache: the caches stay as they are and the output is NaN throughout, so that a step
    # beyond the cache shows in the logits (general kernel, and the head_dim 128 kernel with and without splits)
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device=cuda)
    for d, pos in ((64, 8), (128, 8), (128, -1)):
        out = torch.full((1, 4 * d), 7.0, dtype=torch.float16, device=cuda)
        kc = torch.full((8, 1, d), 3.0, dtype=torch.float16, device=cuda)
        vc = kc.clone()
        p.fill_(pos)
        assert L.elutq_decode_rope_attn_f16(t.data_ptr(), kc.data_ptr(), vc.data_ptr(), p.data_ptr(), out.data_ptr(), 4, 1, d, 8, 1e4, s) == 0
        torch.cuda.synchronize()
        assert bool(out.isnan().all()) and bool((kc == 3).all()) and bool((vc == 3).all())
        out.fill_(7.0)
        assert L.elutq_decode_rope_attn_split_f16(t.data_ptr(), kc.data_ptr(), vc.data_ptr(), p.data_ptr(), out.data_ptr(), 4, 1, d, 8,
                                                  1e4, 0, ws.data_ptr(), ws.numel(), s) == 0
        torch.cuda.synchronize()
        assert bool(out.isnan().all()) and bool((kc == 3).all()) and int(ws.count_nonzero()) == 0


@pytest.mark.parametrize("split", [False, True])
@pytest.mark.parametrize("n", [1, 7, 8, 4096, 65536, 128256, 128259])
def test_argmax_kernel(cuda, n, split):
    """elutq_decode_argmax_f16 / _ws_f16 (64 workgroups that meet in a workspace; two calls in a row must
    find its counter at zero): first index of the strict maximum (arm_argmax.cpp:3-30), also
    with the maximum repeated, at either end, in the unaligned tail, and with NaNs present;
    the position counter is advanced by one."""
    from elutq_amd import _lib
    lib = _lib.lib()
    ws = torch.zeros(65536 + 512, dtype=torch.uint8, device=cuda)

    class L:              # the entry point under test, with the single-workgroup signature
        @staticmethod
        def elutq_decode_argmax_f16(logits, count, token, position, st):
            if split:
                return lib.elutq_decode_argmax_ws_f16(logits, count, token, position, ws.data_ptr(), ws.numel(), st)
            return lib.elutq_decode_argmax_f16(logits, count, token, position, st)
    g = torch.Generator(device=cuda).manual_seed(n)
    stream = torch.cuda.current_stream().cuda_stream
    tok = torch.full((1,), -5, dtype=torch.long, device=cuda)
    pos = torch.tensor([41], dtype=torch.long, device=cuda)
    cases = [torch.randn(n, generator=g, device=cuda).half() for _ in range(3)]
    t = cases[0].clone(); t[n - 1] = 60000.0; cases.append(t)                    # last element
    t = cases[1].clone(); t[0] = 60000.0; cases.append(t)                        # first element
    t = cases[2].clone(); t[n // 2:] = t.max(); cases.append(t)                  # a run of equal maxima
    t = cases[0].clone(); t[::3] = float("nan"); cases.append(t)                 # NaNs never win
    cases.append(torch.full((n,), float("-inf"), dtype=torch.float16, device=cuda))
    for i, c in enumerate(cases):
        assert L.elutq_decode_argmax_f16(c.data_ptr(), n, tok.data_ptr(), pos.data_ptr(), stream) == 0
        torch.cuda.synchronize()
        v = c.float().cpu().numpy()
        best, want = float("-inf"), 0
        for j in range(n):                                                       # the reference's loop
            if v[j] > best:
                best, want = v[j], j
        assert int(tok) == want, (i, n)
        assert int(pos) == 42 + i
    # unaligned pointer: same answer through the scalar path
    if n > 9:
        c = cases[0]
        assert L.elutq_decode_argmax_f16(c.data_ptr() + 2, n - 1, tok.data_ptr(), None, stream) == 0
        torch.cuda.synchronize()
        assert int(tok) == int(c[1:].float().argmax())
    assert L.elutq_decode_argmax_f16(None, n, tok.data_ptr(), None, stream) == -1
    assert L.elutq_decode_argmax_f16(cases[0].data_ptr(), 0, tok.data_ptr(), None, stream) == -2
    if split:
        assert not bool(ws[:4].any())                    # the arrival counter is back at zero
        if n >= 65536:
            small = torch.zeros(1024, dtype=torch.uint8, device=cuda)
            assert _lib.lib().elutq_decode_argmax_ws_f16(cases[0].data_ptr(), n, tok.data_ptr(), None, small.data_ptr(),
                                                         small.numel(), stream) == -5


@pytest.mark.parametrize("n", [64, 4096, 5120, 1000])
def test_final_rmsnorm_kernel(cuda, n):
    """elutq_decode_rmsnorm_f16 against the fp32 restatement of arm_rmsnorm.cpp:25-84."""
    from elutq_amd import _lib
    g = torch.Generator(device=cuda).manual_seed(n)
    x = (torch.randn(1, n, generator=g, device=cuda) * 3).half()
    w = (1 + 0.1 * torch.randn(n, generator=g, device=cuda)).half()
    out = torch.zeros(1, n, dtype=torch.float16, device=cuda)
    rc = _lib.lib().elutq_decode_rmsnorm_f16(x.data_ptr(), w.data_ptr(), out.data_ptr(), n, 1e-5,
                                             torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    ref = rms_norm(x, w, 1e-5)
    # same formula, different fp32 summation order: at most one fp16 ulp apart
    assert (out.float() - ref.float()).abs().max() <= 2.0 ** -10 * ref.float().abs().max()
    assert (out != ref).float().mean() < 0.02


def test_embedding_gather_follows_the_device_token(cuda):
    """elutq_decode_embed_f16: the row of the token held in device memory (arm_embedding.cpp:4-20); a token
    outside the table gives a zero row instead of a read outside it."""
    from elutq_amd import _lib
    g = torch.Generator(device=cuda).manual_seed(3)
    for vocab, hidden in ((1000, 512), (37, 4096), (5, 24)):
        embed = torch.randn(vocab, hidden, generator=g, device=cuda).half()
        out = torch.full((1, hidden), 7.0, dtype=torch.float16, device=cuda)
        token = torch.zeros(1, dtype=torch.long, device=cuda)
        for t in (0, vocab // 2, vocab - 1):
            token.fill_(t)
            _lib.check(_lib.lib().elutq_decode_embed_f16(embed.data_ptr(), token.data_ptr(), out.data_ptr(), hidden, vocab,
                                                         torch.cuda.current_stream().cuda_stream), "embed")
            assert torch.equal(out[0], embed[t])
        for t in (-1, vocab, 1 << 40):
            token.fill_(t)
            out.fill_(7.0)
            _lib.check(_lib.lib().elutq_decode_embed_f16(embed.data_ptr(), token.data_ptr(), out.data_ptr(), hidden, vocab,
                                                         torch.cuda.current_stream().cuda_stream), "embed")
            assert torch.count_nonzero(out) == 0
    assert _lib.lib().elutq_decode_embed_f16(None, token.data_ptr(), out.data_ptr(), 512, 10, None) == -1
    assert _lib.lib().elutq_decode_embed_f16(embed.data_ptr(), token.data_ptr(), out.data_ptr(), 12, 10, None) == -2
