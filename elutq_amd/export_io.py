"""Reader / writer of the reference's per-layer export directory.

One quantized linear layer is a directory `<root>/<layer id>/<module name>/`
(GPTQ/HLQ.py:73, read back by C++/examples/models/llama.cpp:92-111) holding

  weight_config.json  weight_data_len, base_bit, use_sparse, in_channel, out_channel,
                      has_bias                                   (GPTQ/HLQ.py:175-193)
  w_quant.bin         uint8 [bits][N][K/8], LSB-first along K    (GPTQ/HLQ.py:230-251)
  w_scale.bin         fp16  [bits][N][K/G]                       (GPTQ/HLQ.py:223-228)
  w_zero.bin          fp16  [N][K/G]                             (GPTQ/HLQ.py:218-221)
  bias.bin            fp16  [N], only if has_bias                (GPTQ/HLQ.py:184-191)

A layer whose json says `use_sparse: true` (read by C++/ops/src/arm/parameters.cpp:19-64; the
reference's exporter never writes one) has `base_bit` dense planes and a block-sparse extra plane:

  weight_mask.bin     uint32 [sparse_mask_len]: pairs (channel start, k start) of blocks of
                      32 channels x G inputs
  w_quant.bin         dense planes, then every block as uint8 [32][G/8]
  w_scale.bin         dense scales, then every block's fp16 [32]

The reference exporter never writes the `groupsize` key its own loader reads
(C++/ops/src/arm/parameters.cpp:17), so the reader takes it from the json when
present and otherwise derives it from the size of w_zero.bin.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass

import numpy as np


@dataclass
class ExportedLinear:
    k: int
    n: int
    bits: int
    group: int
    w_quant: np.ndarray          # uint8 [bits, N, K/8]
    w_scale: np.ndarray          # fp16  [bits, N, K/G]
    w_zero: np.ndarray           # fp16  [N, K/G]
    bias: np.ndarray | None      # fp16  [N]
    sparse: "SparseBlocks | None" = None


@dataclass
class SparseBlocks:
    """Block-sparse extra plane as the files hold it."""
    blocks: np.ndarray           # uint8  [nblk, 32, G/8], LSB-first along K
    scale: np.ndarray            # fp16   [nblk, 32]
    mask: np.ndarray             # uint32 [nblk, 2] = (channel start, k start)


def densify_sparse(w_quant, w_scale, sparse: SparseBlocks, group: int):
    """The block-sparse extra plane written out as one more dense plane: the blocks' bits where a block
    exists and zero bits elsewhere, the blocks' scales where a block exists and scale 0 elsewhere -- the
    same W, term for term (a scale of 0 contributes exactly 0), in the form every dense kernel reads.
    Returns (w_quant [bits+1, N, K/8], w_scale [bits+1, N, K/G]), or None if the plane does not fit that
    form: more than four planes in all, a block that does not start at a group boundary, or two blocks on
    the same (channel tile, group).  Rows of a last, partial channel tile beyond N are dropped."""
    w_quant = np.ascontiguousarray(w_quant, dtype=np.uint8)
    w_scale = np.ascontiguousarray(w_scale, dtype=np.float16)
    bits, n, k8 = w_quant.shape
    k, ng = k8 * 8, k8 * 8 // group
    mask = np.ascontiguousarray(sparse.mask, dtype=np.uint32).reshape(-1, 2).astype(np.int64)
    nblk = mask.shape[0]
    blocks = np.ascontiguousarray(sparse.blocks, dtype=np.uint8).reshape(nblk, 32, group // 8)
    scale = np.ascontiguousarray(sparse.scale, dtype=np.float16).reshape(nblk, 32)
    if bits + 1 > 4:
        return None
    c0, k0 = mask[:, 0], mask[:, 1]
    if nblk and (np.any(k0 % group) or np.any(c0 % 32) or np.any(c0 >= n) or np.any(k0 + group > k)):
        return None
    if nblk and np.unique(c0 // 32 * ng + k0 // group).size != nblk:
        return None
    npad = (n + 31) // 32 * 32
    plane = np.zeros((npad // 32, 32, ng, group // 8), dtype=np.uint8)       # [tile][ch][group][byte]
    sc = np.zeros((npad // 32, 32, ng), dtype=np.float16)
    plane[c0 // 32, :, k0 // group, :] = blocks
    sc[c0 // 32, :, k0 // group] = scale
    plane = plane.reshape(npad, k8)[:n]
    sc = sc.reshape(npad, ng)[:n]
    return np.concatenate([w_quant, plane[None]]), np.concatenate([w_scale, sc[None]])


def write_export_dir(path: str, w_quant, w_scale, w_zero, bias=None, groupsize: int | None = None,
                     sparse: SparseBlocks | None = None) -> None:
    """Writes the five files exactly as the reference exporter does.  `groupsize`
    adds the key the reference forgets; leave None to reproduce its output.  `sparse` appends a
    block-sparse extra plane in the form the reference's loader reads."""
    w_quant = np.ascontiguousarray(w_quant, dtype=np.uint8)
    w_scale = np.ascontiguousarray(w_scale, dtype=np.float16)
    w_zero = np.ascontiguousarray(w_zero, dtype=np.float16)
    bits, n, k8 = w_quant.shape
    k = k8 * 8
    os.makedirs(path, exist_ok=True)
    cfg = {
        "weight_data_len": int(k * n * bits // 8),
        "base_bit": int(bits),
        "use_sparse": False,
        "in_channel": int(k),
        "out_channel": int(n),
        "has_bias": bias is not None,
    }
    if groupsize is not None:
        cfg["groupsize"] = int(groupsize)
    quant_tail = scale_tail = b""
    if sparse is not None:
        blocks = np.ascontiguousarray(sparse.blocks, dtype=np.uint8)
        mask = np.ascontiguousarray(sparse.mask, dtype=np.uint32).reshape(-1, 2)
        sp_scale = np.ascontiguousarray(sparse.scale, dtype=np.float16)
        nblk = mask.shape[0]
        if blocks.ndim != 3 or blocks.shape[:2] != (nblk, 32) or sp_scale.shape != (nblk, 32):
            raise ValueError("sparse blocks must be uint8 [nblk, 32, G/8] with fp16 scales [nblk, 32]")
        quant_tail, scale_tail = blocks.tobytes(), sp_scale.tobytes()
        cfg["use_sparse"] = True
        cfg["sparse_mask_len"] = int(mask.size)
        cfg["weight_data_len"] += len(quant_tail)
        with open(os.path.join(path, "weight_mask.bin"), "wb") as f:
            f.write(mask.tobytes())
    if bias is not None:
        with open(os.path.join(path, "bias.bin"), "wb") as f:
            f.write(np.ascontiguousarray(bias, dtype=np.float16).tobytes())
    with open(os.path.join(path, "w_zero.bin"), "wb") as f:
        f.write(w_zero.tobytes())
    with open(os.path.join(path, "w_scale.bin"), "wb") as f:
        f.write(w_scale.tobytes() + scale_tail)
    with open(os.path.join(path, "w_quant.bin"), "wb") as f:
        f.write(w_quant.tobytes() + quant_tail)
    with open(os.path.join(path, "weight_config.json"), "w") as f:
        json.dump(cfg, f, indent=4)


def read_export_dir(path: str, groupsize: int | None = None) -> ExportedLinear:
    with open(os.path.join(path, "weight_config.json")) as f:
        cfg = json.load(f)
    k, n, bits = int(cfg["in_channel"]), int(cfg["out_channel"]), int(cfg["base_bit"])
    use_sparse = bool(cfg.get("use_sparse", False))
    mask_len = int(cfg["sparse_mask_len"]) if use_sparse else 0
    if mask_len < 0 or mask_len % 2:
        raise ValueError(f"{path}: sparse_mask_len {mask_len} is not an even, non-negative count")
    nblk = mask_len // 2
    dense_bytes = k * n * bits // 8
    w_quant = np.fromfile(os.path.join(path, "w_quant.bin"), dtype=np.uint8)
    if w_quant.size != int(cfg["weight_data_len"]) or w_quant.size < dense_bytes:
        raise ValueError(f"{path}: w_quant.bin has {w_quant.size} bytes, config says {cfg['weight_data_len']}")
    w_zero = np.fromfile(os.path.join(path, "w_zero.bin"), dtype=np.float16)
    group = int(cfg.get("groupsize", 0)) or groupsize
    if not group:
        if w_zero.size == 0 or (k * n) % w_zero.size:
            raise ValueError(f"{path}: cannot derive groupsize from w_zero.bin ({w_zero.size} values)")
        group = k * n // w_zero.size
    if w_zero.size * group != k * n:
        raise ValueError(f"{path}: w_zero.bin has {w_zero.size} values, expected {k * n // group}")
    if w_quant.size != dense_bytes + nblk * 32 * group // 8:
        raise ValueError(f"{path}: w_quant.bin has {w_quant.size} bytes, expected {dense_bytes} for the dense planes "
                         f"and {nblk * 32 * group // 8} for {nblk} sparse blocks")
    w_scale = np.fromfile(os.path.join(path, "w_scale.bin"), dtype=np.float16)
    dense_scales = bits * n * (k // group)
    if w_scale.size != dense_scales + nblk * 32:
        raise ValueError(f"{path}: w_scale.bin has {w_scale.size} values, expected {dense_scales + nblk * 32}")
    sparse = None
    if use_sparse:
        mask = np.fromfile(os.path.join(path, "weight_mask.bin"), dtype=np.uint32)
        if mask.size != mask_len:
            raise ValueError(f"{path}: weight_mask.bin has {mask.size} values, config says {mask_len}")
        sparse = SparseBlocks(blocks=w_quant[dense_bytes:].reshape(nblk, 32, group // 8),
                              scale=w_scale[dense_scales:].reshape(nblk, 32), mask=mask.reshape(nblk, 2))
        w_quant, w_scale = w_quant[:dense_bytes], w_scale[:dense_scales]
    bias = None
    if cfg.get("has_bias", False):
        bias = np.fromfile(os.path.join(path, "bias.bin"), dtype=np.float16)
        if bias.size != n:
            raise ValueError(f"{path}: bias.bin has {bias.size} values, expected {n}")
    return ExportedLinear(k=k, n=n, bits=bits, group=int(group),
                          w_quant=w_quant.reshape(bits, n, k // 8),
                          w_scale=w_scale.reshape(bits, n, k // group),
                          w_zero=w_zero.reshape(n, k // group), bias=bias, sparse=sparse)


# ---------------------------------------------------------------------------------------
# Whole-model export tree (GPTQ/llama.py:285-343 writes it, C++/examples/models/llama.cpp:59-115
# reads it): fp16 raw binaries next to the per-layer linear directories.
#
#   <root>/embed_tokens.bin               fp16 [vocab][hidden]   (shared_embed_lm_head.bin when the
#                                                                 exporter found tied embeddings)
#   <root>/lm_head.bin                    fp16 [vocab][hidden]   or <root>/lm_head/lm_head/ (HLQ)
#   <root>/final_rmsnorm_weight.bin       fp16 [hidden]
#   <root>/<i>/input_layernorm_weight.bin, post_attention_layernorm_weight.bin   fp16 [hidden]
#   <root>/<i>/self_attn.{q,k,v,o}_proj/, mlp.{gate,up,down}_proj/               linear directories
# ---------------------------------------------------------------------------------------
LAYER_LINEARS = ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj",
                 "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj")
LAYER_NORMS = ("input_layernorm_weight.bin", "post_attention_layernorm_weight.bin")
REPACKED_JSON = "repacked.json"
REPACK_LAYOUT_VERSION = 1


def write_fp16_bin(path: str, a) -> None:
    os.makedirs(os.path.dirname(path) or ".", exist_ok=True)
    with open(path, "wb") as f:
        f.write(np.ascontiguousarray(a, dtype=np.float16).tobytes())


def read_fp16_bin(path: str, count: int | None = None) -> np.ndarray:
    a = np.fromfile(path, dtype=np.float16)
    if count is not None and a.size != count:
        raise ValueError(f"{path}: {a.size} fp16 values, expected {count}")
    return a


def embedding_file(root: str) -> str:
    """embed_tokens.bin, or the name the exporter uses for tied embeddings."""
    for name in ("embed_tokens.bin", "shared_embed_lm_head.bin"):
        if os.path.exists(os.path.join(root, name)):
            return os.path.join(root, name)
    raise FileNotFoundError(f"{root}: neither embed_tokens.bin nor shared_embed_lm_head.bin")


def lm_head_kind(root: str) -> str:
    """'hlq' (lm_head/lm_head directory), 'fp16' (lm_head.bin) or 'tied' (llama.cpp:70-80)."""
    if os.path.isdir(os.path.join(root, "lm_head", "lm_head")):
        return "hlq"
    if os.path.exists(os.path.join(root, "lm_head.bin")):
        return "fp16"
    return "tied"


def is_repacked_dir(path: str) -> bool:
    return os.path.exists(os.path.join(path, REPACKED_JSON))


def write_repacked_dir(path: str, k: int, n: int, bits: int, group: int, planes, scales, zeros, bias=None,
                       sparse: SparseBlocks | None = None) -> None:
    """Kernel-layout buffers of one linear layer as files that load with a plain copy.  A sparse
    extra plane keeps its file form (the kernels read that form) under names of its own."""
    os.makedirs(path, exist_ok=True)
    for name, a in (("planes.bin", planes), ("scales.bin", scales), ("zeros.bin", zeros)):
        with open(os.path.join(path, name), "wb") as f:
            f.write(np.ascontiguousarray(a, dtype=np.uint8).tobytes())
    if bias is not None:
        write_fp16_bin(os.path.join(path, "bias.bin"), bias)
    cfg = {"layout_version": REPACK_LAYOUT_VERSION, "in_channel": int(k), "out_channel": int(n),
           "base_bit": int(bits), "groupsize": int(group), "has_bias": bias is not None}
    if sparse is not None:
        mask = np.ascontiguousarray(sparse.mask, dtype=np.uint32)
        cfg["use_sparse"], cfg["sparse_mask_len"] = True, int(mask.size)
        for name, a in (("sparse_blocks.bin", np.ascontiguousarray(sparse.blocks, dtype=np.uint8)),
                        ("sparse_scales.bin", np.ascontiguousarray(sparse.scale, dtype=np.float16)),
                        ("weight_mask.bin", mask)):
            with open(os.path.join(path, name), "wb") as f:
                f.write(a.tobytes())
    with open(os.path.join(path, REPACKED_JSON), "w") as f:
        json.dump(cfg, f, indent=4)


def read_repacked_sparse(path: str) -> SparseBlocks | None:
    """The sparse extra plane of a repacked directory, or None."""
    with open(os.path.join(path, REPACKED_JSON)) as f:
        cfg = json.load(f)
    if not cfg.get("use_sparse", False):
        return None
    mask_len, group = int(cfg["sparse_mask_len"]), int(cfg["groupsize"])
    nblk = mask_len // 2
    mask = np.fromfile(os.path.join(path, "weight_mask.bin"), dtype=np.uint32)
    blocks = np.fromfile(os.path.join(path, "sparse_blocks.bin"), dtype=np.uint8)
    scale = np.fromfile(os.path.join(path, "sparse_scales.bin"), dtype=np.float16)
    if mask_len % 2 or mask.size != mask_len or blocks.size != nblk * 32 * group // 8 or scale.size != nblk * 32:
        raise ValueError(f"{path}: sparse files do not match sparse_mask_len = {mask_len}")
    return SparseBlocks(blocks.reshape(nblk, 32, group // 8), scale.reshape(nblk, 32), mask.reshape(nblk, 2))


def read_repacked_dir(path: str):
    """-> (k, n, bits, group, planes, scales, zeros, bias) with uint8 buffers (bias fp16 or None)."""
    with open(os.path.join(path, REPACKED_JSON)) as f:
        cfg = json.load(f)
    if cfg.get("layout_version") != REPACK_LAYOUT_VERSION:
        raise ValueError(f"{path}: layout version {cfg.get('layout_version')}, this build reads {REPACK_LAYOUT_VERSION}")
    k, n, bits, group = int(cfg["in_channel"]), int(cfg["out_channel"]), int(cfg["base_bit"]), int(cfg["groupsize"])
    bufs = [np.fromfile(os.path.join(path, name), dtype=np.uint8) for name in ("planes.bin", "scales.bin", "zeros.bin")]
    bias = read_fp16_bin(os.path.join(path, "bias.bin"), n) if cfg.get("has_bias") else None
    return (k, n, bits, group, *bufs, bias)
