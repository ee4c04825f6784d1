"""LlamaDecoder over an exported model tree: the reference's layout, the same tree after the
offline repack, and the in-memory construction must decode the same tokens."""
import numpy as np
import pytest
import torch

from elutq_amd.hlq_linear import HLQLinear
from elutq_amd.llama_decode import LlamaDecoder
from torch_glue_decode import TorchGlueDecoder, decoder_from_export, make_decoder
from elutq_amd.repack import repack_tree

from model_export_fixture import TINY, write_tiny_export

pytestmark = pytest.mark.gpu


def in_memory_parts(arrays, dev):
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    layers = []
    for lay in arrays["layers"]:
        lin = {name: HLQLinear.from_export_arrays(L.w_quant, L.w_scale, L.w_zero, L.group, L.bias, dev)
               for name, L in lay.items() if not name.endswith(".bin")}
        layers.append((lin, (t(lay["input_layernorm_weight.bin"]), t(lay["post_attention_layernorm_weight.bin"]))))
    head = arrays.get("lm_head")
    if head is not None and not isinstance(head, np.ndarray):
        head = HLQLinear.from_export_arrays(head.w_quant, head.w_scale, head.w_zero, head.group, None, dev)
    elif head is not None:
        head = t(head)
    return {"layers": layers, "embed": t(arrays["embed"]), "lm_head": head, "norm": t(arrays["norm"])}


@pytest.mark.parametrize("kind", ["fp16", "hlq", "tied"])
@pytest.mark.parametrize("impl", ["hip", "torch"])
def test_decoder_from_export_tree(cuda, tmp_path, kind, impl):
    src, dst = str(tmp_path / "export"), str(tmp_path / "repacked")
    arrays = write_tiny_export(src, lm_head=kind)
    repack_tree(src, dst)
    models = [decoder_from_export(impl, src, TINY, device=cuda),
              decoder_from_export(impl, dst, TINY, device=cuda),
              make_decoder(impl, TINY, device=cuda, parts=in_memory_parts(arrays, cuda))]
    assert (models[0].lm_head_q is not None) == (kind == "hlq")
    if kind == "tied":
        assert torch.equal(models[0].lm_head, models[0].embed)
    outs = []
    for m in models:
        m.fill_cache(9, seed=3)
        m.token.fill_(5)
        toks, logits = [], []
        for _ in range(4):
            logits.append(m.step().clone())
            toks.append(int(m.token))
        outs.append((toks, torch.cat(logits)))
    for toks, logits in outs[1:]:
        assert toks == outs[0][0] and torch.equal(logits, outs[0][1])
    assert all(0 <= t < TINY.vocab for t in outs[0][0]) and int(models[0].pos) == 13
    if impl == "hip":
        # the fused step (with an HLQ lm_head: final norm inside its GEMV) against the PyTorch-glue step
        glue = TorchGlueDecoder.from_export(src, TINY, device=cuda, fuse=False)
        glue.fill_cache(9, seed=3)
        glue.token.fill_(5)
        first = glue.step().float()
        assert float((outs[0][1][:1].float() - first).abs().max()) <= 2e-2 * float(first.abs().max())


def test_decoder_with_sparse_extra_planes(cuda, tmp_path):
    """Layers with a sparse extra plane: by default the plane is written out as one more dense plane at load, so the
    fused step runs them (q carries three planes, k and v two: the concatenation lifts k and v); held as blocks they
    run through the plain HLQLinear calls of the PyTorch-glue step, or through the fused step with a launch of the
    plane in front of each such projection (q|k|v: the block lists concatenated like the dense buffers)."""
    src, dst, plain = str(tmp_path / "export"), str(tmp_path / "repacked"), str(tmp_path / "plain")
    write_tiny_export(src, sparse_on=("down_proj", "q_proj"))
    write_tiny_export(plain)
    repack_tree(src, dst)
    outs = []
    for root, impl, kw in ((src, "hip", {}), (dst, "hip", {}), (src, "torch", dict(fuse=False, sparse_mode="blocks")),
                           (plain, "hip", {}), (src, "hip", dict(sparse_mode="blocks"))):
        m = decoder_from_export(impl, root, TINY, device=cuda, **kw)
        m.fill_cache(9, seed=3)
        m.token.fill_(5)
        logits = torch.cat([m.step().clone() for _ in range(3)])
        outs.append((m, logits))
    assert outs[0][0].layers[0].down_proj.bits == 3 and outs[0][0].layers[0].qkv.bits == 3
    assert outs[2][0].layers[0].down_proj.sparse_count > 0 and outs[3][0].layers[0].down_proj.bits == 2
    assert torch.equal(outs[0][1], outs[1][1])                  # export tree == repacked tree
    assert not torch.equal(outs[0][1], outs[3][1])              # the planes do take part
    # fused step on dense planes against the glue step on blocks: the first step's logits
    a, b = outs[0][1][:1].float(), outs[2][1][:1].float()
    assert float((a - b).abs().max()) <= 2e-2 * float(b.abs().max())
    # the fused step on blocks: against the glue step on the same blocks and against the fused step on dense planes
    fb = outs[4][0]
    assert fb.layers[0].down_proj.sparse_count > 0 and fb.layers[0].qkv.sparse_count > 0 and fb.layers[0].qkv.bits == 2
    assert fb.layers[0].qkv.sparse_count == outs[2][0].layers[0].q_proj.sparse_count
    c = outs[4][1][:1].float()
    assert float((c - b).abs().max()) <= 2e-2 * float(b.abs().max())
    assert float((c - a).abs().max()) <= 2e-2 * float(a.abs().max())
    assert not torch.equal(outs[4][1], outs[3][1])
    # ... and replayed from a graph: the same logits as its eager steps
    fb.fill_cache(9, seed=3)
    fb.token.fill_(5)
    fb.capture()
    for i in range(3):
        fb.replay()
        torch.cuda.synchronize()
        assert torch.equal(fb._logits, outs[4][1][i:i + 1])
    # every layer held as blocks equals its own dequantized weight applied densely
    x = torch.randn(3, TINY.ffn, device=cuda).to(torch.float16)
    mod = outs[2][0].layers[1].down_proj
    want = x.float() @ mod.dequantize().float().T + (mod.bias.float() if mod.bias is not None else 0)
    got = mod(x).float()
    assert float((got - want).abs().max()) <= 2e-2 * float(want.pow(2).mean().sqrt())


def test_from_export_rejects_wrong_shape(cuda, tmp_path):
    import dataclasses
    src = str(tmp_path / "export")
    write_tiny_export(src)
    with pytest.raises(ValueError, match="the shape needs"):
        LlamaDecoder.from_export(src, dataclasses.replace(TINY, ffn=512), device=cuda)
    with pytest.raises(ValueError, match="fp16 values"):
        LlamaDecoder.from_export(src, dataclasses.replace(TINY, vocab=301), device=cuda)
