"""Seeded synthetic HLQ layers with the distributions the benchmark configs name.

All tensors are drawn on the CPU from ``torch.Generator().manual_seed(seed)`` and
rounded to fp16 before anything uses them, so every machine sees the same bits:

  x       randn(M, K)                                            -> fp16
  planes  randint(0, 2, [B, N, K])  (i.i.d. Bernoulli 0.5)
  w2      s0 ~ U(0.005, 0.02) per (n, group);  s1 = 2*s0*U(0.8, 1.2)
  w3/w4   s0 ~ U(0.003, 0.01);                 s_b = 2^b*s0*U(0.8, 1.2), b >= 1
  zero    z = -(sum_b s_b)/2 * U(0.9, 1.1)

The arrays come back in the reference's export layout (GPTQ/HLQ.py:207-251):
w_quant uint8 [B, N, K/8] packed LSB-first along K, w_scale fp16 [B, N, K/G],
w_zero fp16 [N, K/G].
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch


@dataclass
class SynthLayer:
    k: int
    n: int
    bits: int
    group: int
    w_quant: np.ndarray     # uint8 [B, N, K/8]
    w_scale: np.ndarray     # fp16  [B, N, K/G]
    w_zero: np.ndarray      # fp16  [N, K/G]
    bias: np.ndarray | None  # fp16 [N]
    x: np.ndarray           # fp16  [M, K]


def pack_bits_lsb_first(planes: np.ndarray) -> np.ndarray:
    """0/1 uint8 [..., K] -> uint8 [..., K/8]; bit j of byte i is element 8*i+j
    (the order Pack_T_MAC_Weight writes, GPTQ/HLQ.py:239-251)."""
    return np.packbits(np.asarray(planes, dtype=np.uint8), axis=-1, bitorder="little")


def make_layer(k: int, n: int, bits: int = 2, group: int = 128, m: int = 1, seed: int = 0,
               bias: bool = False) -> SynthLayer:
    assert k % group == 0 and k % 8 == 0
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g).to(torch.float16)
    planes = torch.randint(0, 2, (bits, n, k), generator=g, dtype=torch.uint8)
    ng = k // group

    def uni(lo, hi):
        return torch.rand(n, ng, generator=g) * (hi - lo) + lo

    s0 = uni(0.005, 0.02) if bits == 2 else uni(0.003, 0.01)
    scales = [s0]
    for b in range(1, bits):
        scales.append((2.0 ** b) * s0 * uni(0.8, 1.2))
    s = torch.stack(scales, 0)                                   # [B, N, K/G] fp32
    z = -(s.sum(0)) / 2 * uni(0.9, 1.1)
    bvec = None
    if bias:
        bvec = (torch.randn(n, generator=g) * 0.1).to(torch.float16).numpy()
    return SynthLayer(k=k, n=n, bits=bits, group=group,
                      w_quant=pack_bits_lsb_first(planes.numpy()),
                      w_scale=s.to(torch.float16).numpy(),
                      w_zero=z.to(torch.float16).numpy(),
                      bias=bvec, x=x.numpy())


def make_sparse_plane(k: int, n: int, group: int = 128, density: float = 0.25, seed: int = 0,
                      scale_range=(0.02, 0.08)):
    """A seeded block-sparse extra plane in the form the reference's loader consumes
    (C++/ops/src/arm/parameters.cpp:19-64): every (32-channel tile, group) pair is a block with
    probability `density`; blocks are listed by ascending channel start, then ascending k start.
    Returns (bits uint8 0/1 [nblk, 32, G], scale fp16 [nblk, 32], mask uint32 [nblk, 2])."""
    assert n % 32 == 0 and k % group == 0
    g = torch.Generator().manual_seed(seed)
    pick = torch.rand(n // 32, k // group, generator=g) < density
    idx = pick.nonzero()                                           # row-major: tile, then group
    mask = torch.stack([idx[:, 0] * 32, idx[:, 1] * group], 1).to(torch.int64).numpy().astype(np.uint32)
    nblk = mask.shape[0]
    bits = torch.randint(0, 2, (nblk, 32, group), generator=g, dtype=torch.uint8).numpy()
    lo, hi = scale_range
    scale = (torch.rand(nblk, 32, generator=g) * (hi - lo) + lo).to(torch.float16).numpy()
    return bits, scale, mask


def with_device_sparse_plane(mod, density: float = 0.1, seed: int = 0):
    """`mod` (an HLQLinear on the GPU) with a random block-sparse extra plane held as blocks, drawn on the device:
    every (32-channel tile, group) pair is a block with probability `density`, in the list order the kernels expect
    (ascending tile, then ascending k start).  The dense buffers are shared with `mod`."""
    import torch

    from .hlq_linear import HLQLinear, sparse_index

    dev = mod.planes.device
    g = torch.Generator(device=dev).manual_seed(seed)
    k, n, group = mod.in_features, mod.out_features, mod.group_size
    tiles = (n + 31) // 32
    pick = torch.rand(tiles, k // group, generator=g, device=dev) < density
    where = pick.nonzero()                                          # row-major: tile, then group
    nblk = where.shape[0]
    mask = torch.stack([where[:, 0] * 32, where[:, 1] * group], 1).cpu().numpy().astype(np.uint32)
    index = torch.from_numpy(sparse_index(mask, k, n, group)).to(dev)
    blocks = torch.randint(0, 256, (nblk, 32, group // 8), generator=g, device=dev, dtype=torch.uint8)
    scales = (torch.rand(nblk, 32, generator=g, device=dev) * 0.004 + 0.001).to(torch.float16)
    return HLQLinear(k, n, mod.bits, group, mod.planes, mod.scales, mod.zeros, mod.bias, (blocks, scales, index))


# (K, N) of the LLaMA-3-8B projections and of the LLaMA-2-13B prefill shapes.
LLAMA3_8B_SHAPES = {
    "q_proj": (4096, 4096), "k_proj": (4096, 1024), "v_proj": (4096, 1024), "o_proj": (4096, 4096),
    "gate_proj": (4096, 14336), "up_proj": (4096, 14336), "down_proj": (14336, 4096),
}
LLAMA2_13B_PREFILL_SHAPES = [(5120, 5120), (5120, 13824), (13824, 5120)]


def algorithmic_bytes(k: int, n: int, bits: int, group: int, m: int = 1) -> int:
    """planes + fp16 per-plane scales + fp16 zeros + x + y."""
    return k * n * bits // 8 + 2 * bits * n * (k // group) + 2 * n * (k // group) + 2 * m * k + 2 * m * n


def make_device_layer(k: int, n: int, bits: int = 2, group: int = 128, seed: int = 0, device="cuda",
                      bias: bool = False):
    """Random HLQLinear drawn on the GPU directly in the kernel layout, for benchmarks.

    Planes are uniform random bytes (i.i.d. Bernoulli(0.5) bits in any bit order); scales and
    zeros follow the same per-(column, group) distributions as make_layer.  The values are
    not those of make_layer(seed): use make_layer when a CPU oracle must see the same bits.
    """
    import torch

    from . import _lib
    from .hlq_linear import HLQLinear

    L = _lib.lib()
    dev = torch.device(device)
    g = torch.Generator(device=dev).manual_seed(seed)
    pb, sb, zb = (L.elutq_hlq_planes_bytes(k, n, bits), L.elutq_hlq_scales_bytes(k, n, bits, group),
                  L.elutq_hlq_zeros_bytes(k, n, group))
    if not pb or not sb:
        raise ValueError(f"unsupported HLQ shape K={k} N={n} bits={bits} group={group}")
    planes = torch.randint(0, 256, (pb,), generator=g, dtype=torch.uint8, device=dev)
    ncb, nt = (n + 63) // 64, (k // group + 1) // 2

    def uni(lo, hi):
        return torch.rand(ncb, nt, 64, 2, generator=g, device=dev) * (hi - lo) + lo

    s0 = uni(0.005, 0.02) if bits == 2 else uni(0.003, 0.01)
    sc = [s0] + [(2.0 ** b) * s0 * uni(0.8, 1.2) for b in range(1, bits)]
    s = torch.stack(sc, 2)                                    # [ncb, nt, bits, 64, 2]
    z = -(s.sum(2)) / 2 * uni(0.9, 1.1)                       # [ncb, nt, 64, 2]
    scales = s.to(torch.float16).contiguous().view(torch.uint8).reshape(-1)
    zeros = z.to(torch.float16).contiguous().view(torch.uint8).reshape(-1)
    assert scales.numel() == sb and zeros.numel() == zb
    b = (torch.randn(n, generator=g, device=dev) * 0.1).to(torch.float16) if bias else None
    return HLQLinear(k, n, bits, group, planes, scales, zeros, b)
