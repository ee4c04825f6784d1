"""Reader / writer of the reference's per-layer export directory.

One quantized linear layer is a directory `<root>/<layer id>/<module name>/`
(GPTQ/HLQ.py:73, read back by C++/examples/models/llama.cpp:92-111) holding

  weight_config.json  weight_data_len, base_bit, use_sparse, in_channel, out_channel,
                      has_bias                                   (GPTQ/HLQ.py:175-193)
  w_quant.bin         uint8 [bits][N][K/8], LSB-first along K    (GPTQ/HLQ.py:230-251)
  w_scale.bin         fp16  [bits][N][K/G]                       (GPTQ/HLQ.py:223-228)
  w_zero.bin          fp16  [N][K/G]                             (GPTQ/HLQ.py:218-221)
  bias.bin            fp16  [N], only if has_bias                (GPTQ/HLQ.py:184-191)

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


def write_export_dir(path: str, w_quant, w_scale, w_zero, bias=None, groupsize: int | None = None) -> None:
    """Writes the five files exactly as the reference exporter does.  `groupsize`
    adds the key the reference forgets; leave None to reproduce its output."""
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
    if bias is not None:
        with open(os.path.join(path, "bias.bin"), "wb") as f:
            f.write(np.ascontiguousarray(bias, dtype=np.float16).tobytes())
    with open(os.path.join(path, "w_zero.bin"), "wb") as f:
        f.write(w_zero.tobytes())
    with open(os.path.join(path, "w_scale.bin"), "wb") as f:
        f.write(w_scale.tobytes())
    with open(os.path.join(path, "w_quant.bin"), "wb") as f:
        f.write(w_quant.tobytes())
    with open(os.path.join(path, "weight_config.json"), "w") as f:
        json.dump(cfg, f, indent=4)


def read_export_dir(path: str, groupsize: int | None = None) -> ExportedLinear:
    with open(os.path.join(path, "weight_config.json")) as f:
        cfg = json.load(f)
    if cfg.get("use_sparse", False):
        raise NotImplementedError("sparse extra-plane exports are not supported")
    k, n, bits = int(cfg["in_channel"]), int(cfg["out_channel"]), int(cfg["base_bit"])
    w_quant = np.fromfile(os.path.join(path, "w_quant.bin"), dtype=np.uint8)
    if w_quant.size != int(cfg["weight_data_len"]) or w_quant.size != k * n * bits // 8:
        raise ValueError(f"{path}: w_quant.bin has {w_quant.size} bytes, config says {cfg['weight_data_len']}")
    w_zero = np.fromfile(os.path.join(path, "w_zero.bin"), dtype=np.float16)
    group = int(cfg.get("groupsize", 0)) or groupsize
    if not group:
        if w_zero.size == 0 or (k * n) % w_zero.size:
            raise ValueError(f"{path}: cannot derive groupsize from w_zero.bin ({w_zero.size} values)")
        group = k * n // w_zero.size
    if w_zero.size * group != k * n:
        raise ValueError(f"{path}: w_zero.bin has {w_zero.size} values, expected {k * n // group}")
    w_scale = np.fromfile(os.path.join(path, "w_scale.bin"), dtype=np.float16)
    if w_scale.size != bits * n * (k // group):
        raise ValueError(f"{path}: w_scale.bin has {w_scale.size} values, expected {bits * n * (k // group)}")
    bias = None
    if cfg.get("has_bias", False):
        bias = np.fromfile(os.path.join(path, "bias.bin"), dtype=np.float16)
        if bias.size != n:
            raise ValueError(f"{path}: bias.bin has {bias.size} values, expected {n}")
    return ExportedLinear(k=k, n=n, bits=bits, group=int(group),
                          w_quant=w_quant.reshape(bits, n, k // 8),
                          w_scale=w_scale.reshape(bits, n, k // group),
                          w_zero=w_zero.reshape(n, k // group), bias=bias)
