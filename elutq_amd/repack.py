"""Offline repack of a reference export tree into the kernel layout.

    python -m elutq_amd.repack <export root> <output root>

Every linear directory (weight_config.json + w_quant/w_scale/w_zero[/bias].bin) under the
export root is rewritten as planes.bin / scales.bin / zeros.bin [/ bias.bin] + repacked.json;
every other file (embeddings, norms, fp16 lm_head) is copied.  The output tree loads with
plain file-to-device copies (HLQLinear.from_export_dir and LlamaDecoder.from_export accept
either form).  Counterpart of the rearrangement the reference performs at every model load
(t_mac_g4_rearrange_weight_impl from load_Parameter, C++/ops/src/arm/parameters.cpp:8-70);
runs on the CPU (elutq_hlq_repack_host), no GPU needed.
"""
from __future__ import annotations

import argparse
import os
import shutil
import sys

from .export_io import densify_sparse, read_export_dir, write_repacked_dir


def repack_tree(src: str, dst: str, group_size: int | None = None, verbose: bool = False,
                sparse_mode: str = "auto") -> int:
    """Returns the number of linear layers repacked.  `sparse_mode` as in HLQLinear.from_export_arrays:
    "auto" / "dense" write a block-sparse extra plane out as one more dense plane where that is possible,
    "blocks" keeps its file form beside the dense planes."""
    from .hlq_linear import repack_export_arrays
    count = 0
    for cur, dirs, files in os.walk(src):
        rel = os.path.relpath(cur, src)
        out = os.path.join(dst, rel) if rel != "." else dst
        if "weight_config.json" in files:
            e = read_export_dir(cur, group_size)
            w_quant, w_scale, sparse, bits = e.w_quant, e.w_scale, e.sparse, e.bits
            if sparse is not None:
                from .hlq_linear import sparse_index
                sparse_index(sparse.mask, e.k, e.n, e.group)        # validates the block list
                dense = densify_sparse(w_quant, w_scale, sparse, e.group) if sparse_mode != "blocks" else None
                if dense is not None:
                    (w_quant, w_scale), sparse, bits = dense, None, e.bits + 1
                elif sparse_mode == "dense":
                    raise ValueError(f"{cur}: the sparse extra plane cannot be written as a dense plane")
            planes, scales, zeros = repack_export_arrays(w_quant, w_scale, e.w_zero, e.group)
            write_repacked_dir(out, e.k, e.n, bits, e.group, planes, scales, zeros, e.bias, sparse)
            count += 1
            dirs[:] = []
            if verbose:
                extra = ""
                if e.sparse is not None:
                    extra = f" + {e.sparse.mask.shape[0]} sparse blocks" + (" as a dense plane" if sparse is None else "")
                print(f"{rel}: K={e.k} N={e.n} w{e.bits}g{e.group}{extra}", file=sys.stderr)
            continue
        os.makedirs(out, exist_ok=True)
        for name in files:
            shutil.copyfile(os.path.join(cur, name), os.path.join(out, name))
    return count


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("src")
    ap.add_argument("dst")
    ap.add_argument("--groupsize", type=int, default=None,
                    help="only needed if neither the json nor the size of w_zero.bin determines it")
    ap.add_argument("--sparse", choices=["auto", "dense", "blocks"], default="auto",
                    help="how a block-sparse extra plane is stored: as one more dense plane where possible "
                         "(auto, the default; dense insists), or in its file form (blocks)")
    ap.add_argument("-v", "--verbose", action="store_true")
    a = ap.parse_args(argv)
    if not os.path.isdir(a.src):
        print(f"{a.src}: not a directory", file=sys.stderr)
        return 2
    n = repack_tree(a.src, a.dst, a.groupsize, a.verbose, a.sparse)
    print(f"repacked {n} linear layers into {a.dst}")
    return 0 if n else 1


if __name__ == "__main__":
    sys.exit(main())
