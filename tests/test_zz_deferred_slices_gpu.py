"""K slices of a projection left to the launch that reads its output (elutq_gemv_fusion.d_slices_out /
d_slices_in): the consumer must see, bit for bit, the activations the producer's own output stage
would have written, and a decode step must not change by a bit.  (The file name sorts last on
purpose: the newest entry-point mode is tested after everything it builds on.)"""
import pytest
import torch

from elutq_amd import _lib
from elutq_amd.hlq_linear import HLQLinear
from elutq_amd.llama_decode import LlamaDecoder, LlamaShape
from elutq_amd.synth import make_layer

pytestmark = pytest.mark.gpu


def build(k, n, seed, dev, bits=2, group=128):
    L = make_layer(k, n, bits=bits, group=group, seed=seed, bias=False)
    return HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, group, None, dev)


@pytest.mark.parametrize("ffn,hidden,n_next,bits,group", [(1024, 512, 768, 2, 128), (14336, 4096, 6144, 2, 128),
                                                          (1024, 512, 768, 3, 64), (1024, 512, 768, 4, 128),
                                                          (2048, 1024, 1536, 2, 64), (1088, 576, 768, 2, 64)])
@pytest.mark.parametrize("consumer", [_lib.GEMV_WIDE, 0, _lib.GEMV_NARROW32])
def test_consumer_sees_what_the_producer_would_have_written(cuda, ffn, hidden, n_next, bits, group, consumer):
    """down (SiLU*up prologue, K slices) -> next q|k|v (RMSNorm prologue), at the shapes of the small test
    model and of LLaMA-3-8B, and at the other plane counts / group size; the consumer on the wide-tile kernel,
    on the library's choice (narrow tiles at these widths) and on 32-column tiles."""
    down, qkv = build(ffn, hidden, 1, cuda, bits, group), build(hidden, n_next, 2, cuda, bits, group)
    qkv.ksplit = consumer                # the reference call below runs on the same kernel
    S = down.slices
    assert 2 <= S <= 4
    g = torch.Generator(device=cuda).manual_seed(3)
    gu = torch.randn(1, 2 * ffn, generator=g, device=cuda).half()
    res = torch.randn(1, hidden, generator=g, device=cuda).half()
    w = (1 + 0.1 * torch.randn(hidden, generator=g, device=cuda)).half()
    ws = torch.zeros(max(down.workspace_bytes, qkv.workspace_bytes), dtype=torch.uint8, device=cuda)
    f16 = dict(dtype=torch.float16, device=cuda)
    # the producer sums its own slices
    h_ref, y_ref = torch.empty(1, hidden, **f16), torch.empty(1, n_next, **f16)
    down.gemv_fused(gu, h_ref, ws, prologue=2, residual=res)
    qkv.gemv_fused(h_ref, y_ref, ws, prologue=1, norm_weight=w, eps=1e-5)
    # the consumer does
    slices = torch.full((4, hidden), float("nan"), dtype=torch.float32, device=cuda)
    untouched = torch.full((1, hidden), 7.0, **f16)
    h, y = torch.zeros(1, hidden, **f16), torch.empty(1, n_next, **f16)
    for _ in range(2):                                   # twice: nothing may be left behind in the workspace
        down.gemv_fused(gu, untouched, ws, prologue=2, slices_out=slices)
        qkv.gemv_fused(res, y, ws, prologue=1, norm_weight=w, eps=1e-5, slices_in=slices[:S], x_out=h)
        torch.cuda.synchronize()
        assert torch.equal(h, h_ref) and torch.equal(y, y_ref)
    assert torch.all(untouched == 7.0)                   # the producer's output vector is not written
    assert not torch.isnan(slices[:S]).any() and torch.isnan(slices[S:]).all()
    # the slices are what they say: their sum in order plus the residual, rounded once
    tot = slices[0].clone()
    for s in range(1, S):
        tot += slices[s]
    assert torch.equal((tot + res[0].float()).half(), h_ref[0])
    # without x_out the projection is the same
    y2 = torch.empty(1, n_next, **f16)
    qkv.gemv_fused(res, y2, ws, prologue=1, norm_weight=w, eps=1e-5, slices_in=slices[:S])
    assert torch.equal(y2, y_ref)


def test_deferred_slices_argument_errors(cuda):
    down, qkv, wide = build(1024, 512, 1, cuda), build(512, 768, 2, cuda), build(512, 8192, 4, cuda)
    f16 = dict(dtype=torch.float16, device=cuda)
    gu, res = torch.zeros(1, 2048, **f16), torch.zeros(1, 512, **f16)
    out, y = torch.zeros(1, 512, **f16), torch.zeros(1, 768, **f16)
    w = torch.ones(512, **f16)
    ws = torch.zeros(max(down.workspace_bytes, wide.workspace_bytes), dtype=torch.uint8, device=cuda)
    slices = torch.zeros(4, 512, dtype=torch.float32, device=cuda)
    with pytest.raises(_lib.ElutqError):                 # the consumer adds the residual, not the producer
        down.gemv_fused(gu, out, ws, prologue=2, residual=res, slices_out=slices)
    assert wide.slices == 1
    with pytest.raises(_lib.ElutqError):                 # a launch without K slices has nothing to defer
        wide.gemv_fused(res, torch.zeros(1, 8192, **f16), ws, slices_out=torch.zeros(4, 8192, dtype=torch.float32, device=cuda))
    with pytest.raises(_lib.ElutqError):                 # slices come with the RMSNorm prologue only
        qkv.gemv_fused(res, y, ws, slices_in=slices)
    with pytest.raises(_lib.ElutqError):                 # the combined x may not overwrite its own base
        qkv.gemv_fused(res, y, ws, prologue=1, norm_weight=w, eps=1e-5, slices_in=slices, x_out=res)
    with pytest.raises(_lib.ElutqError):                 # at most four slices
        qkv.gemv_fused(res, y, ws, prologue=1, norm_weight=w, eps=1e-5,
                       slices_in=torch.zeros(5, 512, dtype=torch.float32, device=cuda))


@pytest.mark.parametrize("graph", [False, True])
def test_decode_step_is_bit_identical_with_deferred_slices(cuda, graph):
    shape = LlamaShape(n_layers=3, hidden=512, n_heads=8, n_kv_heads=2, ffn=1024, vocab=1000, max_seq=64)
    runs = {}
    for defer in (False, True):
        m = LlamaDecoder(shape, device=cuda, seed=3)
        m.defer_slices = defer
        m.fill_cache(20)
        m.token.fill_(5)
        if graph:
            m.capture()
        logits, toks = [], []
        for _ in range(5):
            if graph:
                m.replay()
                logits.append(m._buf.logits.clone())
            else:
                logits.append(m.step().clone())
            toks.append(int(m.token))
        runs[defer] = (logits, toks, m.layers[0].k_cache.clone())
    assert runs[False][1] == runs[True][1]
    assert all(torch.equal(a, b) for a, b in zip(runs[False][0], runs[True][0]))
    assert torch.equal(runs[False][2], runs[True][2])


@pytest.mark.parametrize("n_slices", [1, 2, 4])
@pytest.mark.parametrize("pos,splits", [(0, 0), (37, 0), (250, 0), (900, 0), (250, 1), (600, 3)])
def test_attention_reads_unsummed_qkv_slices(cuda, n_slices, pos, splits):
    """elutq_decode_rope_attn_sliced_f16 on fp32 slices == elutq_decode_rope_attn_split_f16 on the fp16
    vector a projection would have stored (slices summed in order, rounded once): output and appended
    cache rows bit for bit."""
    L = _lib.lib()
    nq, nkv, d, max_seq, base = 8, 2, 128, 1024, 500000.0
    g = torch.Generator(device=cuda).manual_seed(pos + n_slices)
    width = (nq + 2 * nkv) * d
    stride = width + 64                                   # rows may be longer than the vector
    slices = torch.randn(n_slices, stride, generator=g, device=cuda)
    tot = slices[0, :width].clone()
    for s in range(1, n_slices):
        tot += slices[s, :width]
    qkv = tot.half().view(1, width)
    kc0 = torch.randn(max_seq, nkv, d, generator=g, device=cuda).half()
    vc0 = torch.randn(max_seq, nkv, d, generator=g, device=cuda).half()
    pos_t = torch.tensor([pos], dtype=torch.long, device=cuda)
    ws = torch.zeros(L.elutq_decode_attn_workspace_bytes(nq, d, 0), dtype=torch.uint8, device=cuda)
    stream = torch.cuda.current_stream().cuda_stream
    res = []
    for sliced in (False, True):
        kc, vc = kc0.clone(), vc0.clone()
        out = torch.zeros(1, nq * d, dtype=torch.float16, device=cuda)
        if sliced:
            rc = L.elutq_decode_rope_attn_sliced_f16(slices.data_ptr(), n_slices, stride, kc.data_ptr(), vc.data_ptr(),
                                                     pos_t.data_ptr(), out.data_ptr(), nq, nkv, d, max_seq, base, splits,
                                                     ws.data_ptr(), ws.numel(), stream)
        else:
            rc = L.elutq_decode_rope_attn_split_f16(qkv.data_ptr(), kc.data_ptr(), vc.data_ptr(), pos_t.data_ptr(),
                                                    out.data_ptr(), nq, nkv, d, max_seq, base, splits, ws.data_ptr(),
                                                    ws.numel(), stream)
        assert rc == 0
        torch.cuda.synchronize()
        res.append((out, kc, vc))
    assert torch.equal(res[0][0], res[1][0]) and torch.equal(res[0][1], res[1][1]) and torch.equal(res[0][2], res[1][2])
    assert not ws[:64 * 1024].any()


def test_sliced_attention_argument_errors(cuda):
    L = _lib.lib()
    nq, nkv, max_seq = 4, 2, 64
    buf = torch.zeros(8, 2048, device=cuda)
    kc = torch.zeros(max_seq, nkv, 128, dtype=torch.float16, device=cuda)
    pos_t = torch.zeros(1, dtype=torch.long, device=cuda)
    out = torch.zeros(1, nq * 128, dtype=torch.float16, device=cuda)
    stream = torch.cuda.current_stream().cuda_stream

    def call(n_slices, stride, d=128, slices=buf):
        return L.elutq_decode_rope_attn_sliced_f16(slices.data_ptr() if slices is not None else None, n_slices, stride,
                                                   kc.data_ptr(), kc.data_ptr(), pos_t.data_ptr(), out.data_ptr(), nq, nkv, d,
                                                   max_seq, 10000.0, 1, None, 0, stream)
    assert call(2, 2048) == 0
    assert call(0, 2048) != 0 and call(5, 2048) != 0      # 1..4 slices
    assert call(2, 1000) != 0                             # rows shorter than q|k|v
    assert call(2, 2048, d=64) != 0                       # head_dim 128 only
    assert call(2, 2048, slices=None) != 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("graph", [False, True])
def test_decode_step_is_bit_identical_with_qkv_slices_left_to_attention(cuda, graph):
    """head_dim 128, a context long enough for several attention splits; the q|k|v projection keeps
    its K slices either way, so only where they are summed differs."""
    shape = LlamaShape(n_layers=2, hidden=1024, n_heads=8, n_kv_heads=2, ffn=2048, vocab=2000, max_seq=320)
    runs = {}
    for defer in (False, True):
        m = LlamaDecoder(shape, device=cuda, seed=3)
        m.defer_qkv = defer
        assert 2 <= m.layers[0].qkv.slices <= 4
        m.fill_cache(250)
        m.token.fill_(5)
        if graph:
            m.capture()
        logits, toks = [], []
        for _ in range(4):
            if graph:
                m.replay()
                logits.append(m._buf.logits.clone())
            else:
                logits.append(m.step().clone())
            toks.append(int(m.token))
        runs[defer] = (logits, toks, m.layers[1].k_cache[250:254].clone())
    assert runs[False][1] == runs[True][1]
    assert all(torch.equal(a, b) for a, b in zip(runs[False][0], runs[True][0]))
    assert torch.equal(runs[False][2], runs[True][2])
