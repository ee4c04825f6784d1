"""Writes tests/golden/hlq_quantizer_vectors.npz: input/output vectors of the reference's
HLQ parameter fitting (GPTQ/quant.py: find_optimal_params_alternating, quantize_with_scales,
dequantize_with_scales, pseudo_quantize_tensor), which nothing but the reference itself pins
(an iterative fit with data-dependent argmin ties and a pseudo-inverse).

Run once, in the container that has the reference checked out:

    python tests/golden/make_quantizer_goldens.py /root/reference

CPU, float32, seeded inputs; the fixture holds data only.
"""
import os
import sys

import numpy as np
import torch


def main(ref_root: str) -> None:
    sys.path.insert(0, os.path.join(ref_root, "GPTQ"))
    import quant as Q          # the reference module, imported read-only

    torch.manual_seed(0)
    out = {}
    cases = [("b2_g128", 2, 6, 128), ("b3_g128", 3, 5, 128), ("b2_g64", 2, 7, 64), ("b4_g128", 4, 3, 128), ("b1_g64", 1, 4, 64)]
    for name, bits, nblocks, gs in cases:
        g = torch.Generator().manual_seed(100 + bits * 10 + gs)
        w = torch.randn(nblocks, gs, generator=g) * 0.05 + torch.randn(nblocks, 1, generator=g) * 0.01
        scales, zeros = Q.find_optimal_params_alternating(w.clone(), bits=bits)
        codes = Q.quantize_with_scales(w.clone(), scales, zeros, bits)
        deq = Q.dequantize_with_scales(codes, scales, zeros)
        out[f"{name}_w"] = w.numpy()
        out[f"{name}_scales"] = scales.numpy()
        out[f"{name}_zeros"] = zeros.numpy()
        out[f"{name}_codes"] = codes.numpy()
        out[f"{name}_deq"] = deq.numpy()
    # the entry point the GPTQ driver calls, on a [rows, group] slab (HLQ.py:127-128)
    g = torch.Generator().manual_seed(7)
    W1 = torch.randn(12, 128, generator=g) * 0.03
    wq, codes, sc, zp = Q.pseudo_quantize_tensor(W1, 2, True, 128, False, True, use_alternating_optimization=True)
    out["slab_w"] = W1.numpy(); out["slab_deq"] = wq.numpy(); out["slab_codes"] = codes.numpy()
    out["slab_scales"] = sc.numpy(); out["slab_zeros"] = zp.numpy()
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hlq_quantizer_vectors.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst, {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
