"""A tiny synthetic model export tree in the reference's layout (GPTQ/llama.py:285-343),
written with the package's own writers; shared by the CPU and GPU tests of the loader."""
import os

import numpy as np

from elutq_amd import export_io as io
from elutq_amd.llama_decode import PROJ_DIRS, LlamaShape, proj_shapes
from elutq_amd.synth import make_layer, make_sparse_plane, pack_bits_lsb_first

TINY = LlamaShape(n_layers=2, hidden=256, n_heads=2, n_kv_heads=1, ffn=384, vocab=300, max_seq=48, bits=2, group=128)


def write_tiny_export(root: str, lm_head: str = "fp16", with_groupsize: bool = False, sparse_on=()) -> dict:
    """lm_head: 'fp16' (lm_head.bin), 'hlq' (lm_head/lm_head: the reference quantizes the lm_head like any other layer unless
    told to skip it, GPTQ/llama.py:143-176; 4 bits here, so that one tree holds two formats)
    or 'tied' (shared_embed_lm_head.bin only).  Projections named in `sparse_on` get a block-sparse
    extra plane on half of their blocks.  Returns the arrays that were written."""
    s = TINY
    r = np.random.default_rng(7)
    out = {"layers": []}
    seed = 1000
    for i in range(s.n_layers):
        lay = {}
        for name, (k, n) in proj_shapes(s).items():
            L = make_layer(k, n, bits=s.bits, group=s.group, seed=seed, bias=(name == "o_proj"))
            seed += 1
            sp = None
            if name in sparse_on:
                b, sc, mk = make_sparse_plane(k, n, s.group, 0.5, seed=seed)
                sp = io.SparseBlocks(pack_bits_lsb_first(b), sc, mk)
            io.write_export_dir(os.path.join(root, str(i), PROJ_DIRS[name]), L.w_quant, L.w_scale, L.w_zero, L.bias,
                                groupsize=s.group if with_groupsize else None, sparse=sp)
            lay[name] = L
        for f in io.LAYER_NORMS:
            lay[f] = (1 + 0.1 * r.standard_normal(s.hidden)).astype(np.float16)
            io.write_fp16_bin(os.path.join(root, str(i), f), lay[f])
        out["layers"].append(lay)
    out["embed"] = (0.5 * r.standard_normal((s.vocab, s.hidden))).astype(np.float16)
    out["norm"] = (1 + 0.1 * r.standard_normal(s.hidden)).astype(np.float16)
    io.write_fp16_bin(os.path.join(root, "final_rmsnorm_weight.bin"), out["norm"])
    if lm_head == "tied":
        io.write_fp16_bin(os.path.join(root, "shared_embed_lm_head.bin"), out["embed"])
    else:
        io.write_fp16_bin(os.path.join(root, "embed_tokens.bin"), out["embed"])
    if lm_head == "fp16":
        out["lm_head"] = (0.05 * r.standard_normal((s.vocab, s.hidden))).astype(np.float16)
        io.write_fp16_bin(os.path.join(root, "lm_head.bin"), out["lm_head"])
    elif lm_head == "hlq":
        L = make_layer(s.hidden, s.vocab, bits=4, group=128, seed=999)
        io.write_export_dir(os.path.join(root, "lm_head", "lm_head"), L.w_quant, L.w_scale, L.w_zero)
        out["lm_head"] = L
    return out
