"""Whole-model export tree and the offline repack CLI (CPU only: the repack is the host
function of the C ABI).  Layout per GPTQ/llama.py:285-343 and C++/examples/models/llama.cpp:59-115."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from elutq_amd import export_io as io
from elutq_amd.hlq_linear import repack_export_arrays, unpack_to_export_arrays
from elutq_amd.llama_decode import PROJ_DIRS
from elutq_amd.repack import main as repack_main, repack_tree

from model_export_fixture import TINY, write_tiny_export


def test_repack_cli_rewrites_linears_and_copies_the_rest(tmp_path):
    src, dst = str(tmp_path / "export"), str(tmp_path / "repacked")
    arrays = write_tiny_export(src, lm_head="hlq")
    rc = subprocess.run([sys.executable, "-m", "elutq_amd.repack", src, dst], capture_output=True, text=True,
                        cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    assert rc.returncode == 0, rc.stderr
    assert "repacked 15 linear layers" in rc.stdout          # 2 layers x 7 + the HLQ lm_head
    for i, lay in enumerate(arrays["layers"]):
        for name, d in PROJ_DIRS.items():
            L = lay[name]
            k, n, bits, group, planes, scales, zeros, bias = io.read_repacked_dir(os.path.join(dst, str(i), d))
            assert (k, n, bits, group) == (L.k, L.n, L.bits, L.group)
            want = repack_export_arrays(L.w_quant, L.w_scale, L.w_zero, L.group)
            for got, w in zip((planes, scales, zeros), want):
                assert np.array_equal(got, w)
            # and back: the repacked files still hold the export bit for bit
            q, s, z = unpack_to_export_arrays(planes, scales, zeros, k, n, bits, group)
            assert np.array_equal(q, L.w_quant) and np.array_equal(s, L.w_scale) and np.array_equal(z, L.w_zero)
            assert (bias is None) == (L.bias is None) and (bias is None or np.array_equal(bias, L.bias))
            assert not os.path.exists(os.path.join(dst, str(i), d, "w_quant.bin"))
        for f in io.LAYER_NORMS:
            assert np.array_equal(io.read_fp16_bin(os.path.join(dst, str(i), f)), lay[f])
    assert np.array_equal(io.read_fp16_bin(os.path.join(dst, "embed_tokens.bin")).reshape(TINY.vocab, -1), arrays["embed"])
    assert np.array_equal(io.read_fp16_bin(os.path.join(dst, "final_rmsnorm_weight.bin")), arrays["norm"])
    assert io.lm_head_kind(dst) == "hlq" and io.is_repacked_dir(os.path.join(dst, "lm_head", "lm_head"))


def test_lm_head_kinds_and_embedding_names(tmp_path):
    for kind in ("fp16", "hlq", "tied"):
        root = str(tmp_path / kind)
        write_tiny_export(root, lm_head=kind)
        assert io.lm_head_kind(root) == kind
        assert os.path.basename(io.embedding_file(root)) == ("shared_embed_lm_head.bin" if kind == "tied" else "embed_tokens.bin")
    with pytest.raises(FileNotFoundError):
        io.embedding_file(str(tmp_path))


def test_repack_errors(tmp_path):
    assert repack_main([str(tmp_path / "missing"), str(tmp_path / "out")]) == 2
    os.makedirs(tmp_path / "empty")
    assert repack_main([str(tmp_path / "empty"), str(tmp_path / "out2")]) == 1          # nothing to repack
    src = str(tmp_path / "export")
    write_tiny_export(src, lm_head="tied", with_groupsize=True)
    assert repack_tree(src, str(tmp_path / "out3")) == 14
    d = os.path.join(str(tmp_path / "out3"), "0", "mlp.down_proj")
    cfg = json.load(open(os.path.join(d, io.REPACKED_JSON)))
    cfg["layout_version"] = 99
    json.dump(cfg, open(os.path.join(d, io.REPACKED_JSON), "w"))
    with pytest.raises(ValueError, match="layout version"):
        io.read_repacked_dir(d)
    with pytest.raises(ValueError, match="fp16 values"):
        io.read_fp16_bin(os.path.join(src, "final_rmsnorm_weight.bin"), 7)
