"""Batch-1 decode step of a LLaMA-shaped model whose linear layers are HLQLinear.

Counterpart of the caller of the hot path in the reference runtime, ``llama::forward`` +
the decode loop of ``main.cpp`` (C++/examples/models/llama.cpp:150-774,
C++/examples/main.cpp:81-110): embedding, then per layer RMSNorm -> q/k/v -> RoPE -> KV-cache
append -> single-token GQA attention -> o -> residual -> RMSNorm -> gate/up -> SiLU*up ->
down -> residual, final RMSNorm, fp16 lm_head, greedy argmax.  Semantics follow the
reference ops: RMSNorm in fp32 with fp16 output (arm_rmsnorm.cpp:25-84), half-split RoPE
pairs (j, j + d/2) with theta = pos * base^(-2j/d) and no frequency rescaling
(arm_rotary.cpp:31-46), fp32 softmax, GQA map h_kv = h * n_kv / n_q
(arm_attention.cpp:199-274), SiLU*up in fp32 (arm_activation.cpp:36-49).

Five fused launches per layer, embedding gather, final norm, lm_head and greedy pick as kernels
of the library.  The step is captured in a HIP graph (token id and position live in device
tensors), so one replay = one token.  q|k|v and gate|up are fused along N, which in the kernel
layout is a concatenation of the packed buffers.  (The same step written with PyTorch ops around
plain HLQLinear calls, the parity partner of this path, lives with the tests:
tests/torch_glue_decode.py.)
"""
from __future__ import annotations

import os
import time
from dataclasses import dataclass

import torch
from torch import nn

from . import _lib
from .hlq_linear import HLQLinear
from .synth import make_device_layer


@dataclass
class LlamaShape:
    n_layers: int = 32
    hidden: int = 4096
    n_heads: int = 32
    n_kv_heads: int = 8
    ffn: int = 14336
    vocab: int = 128256
    rms_eps: float = 1e-5
    rope_base: float = 500000.0
    max_seq: int = 640
    bits: int = 2
    group: int = 128

    @property
    def head_dim(self) -> int:
        return self.hidden // self.n_heads


def fuse_along_n(mods: list[HLQLinear]) -> HLQLinear:
    """One HLQLinear computing the concatenation of the outputs.  The kernel layout is
    column-block major, so this is a concatenation of the packed buffers (every N but the
    last must be a multiple of 64)."""
    k, group = mods[0].in_features, mods[0].group_size
    bits = max(m.bits for m in mods)                 # a layer that carries an extra plane lifts the others
    mods = [m.with_bits(bits) for m in mods]
    for m in mods:
        assert (m.in_features, m.group_size) == (k, group)
    for m in mods[:-1]:
        assert m.out_features % 64 == 0
    bias = None
    if any(m.bias is not None for m in mods):
        bias = torch.cat([m.bias if m.bias is not None else
                          torch.zeros(m.out_features, dtype=torch.float16, device=m.planes.device) for m in mods])
    return HLQLinear(k, sum(m.out_features for m in mods), bits, group,
                     torch.cat([m.planes for m in mods]), torch.cat([m.scales for m in mods]),
                     torch.cat([m.zeros for m in mods]), bias, concat_sparse(mods))


def concat_sparse(mods: list[HLQLinear]):
    """The sparse extra planes (held as blocks) of layers concatenated along N as one plane: the block
    lists one after the other, every layer's channels behind those of the layers before it; the index is
    made anew from the (channel start, k start) pairs."""
    if not any(m.sparse_count for m in mods):
        return None
    import numpy as np

    from .hlq_linear import sparse_index
    dev = mods[0].planes.device
    k, group = mods[0].in_features, mods[0].group_size
    blocks, scales, pairs = [], [], []
    n0 = 0
    for m in mods:
        if m.sparse_count:
            blocks.append(m.sparse_blocks.reshape(-1))
            scales.append(m.sparse_scales)
            pairs.append(m.sparse_pairs() + np.array([[n0, 0]], dtype=np.uint32))
        n0 += m.out_features
    nblk = sum(p.shape[0] for p in pairs)
    index = torch.from_numpy(sparse_index(np.concatenate(pairs), k, n0, group)).to(dev)
    return (torch.cat(blocks).view(nblk, 32, group // 8), torch.cat(scales), index)


class DecoderLayer(nn.Module):
    def __init__(self, s: LlamaShape, linears: dict, norms: tuple, fuse: bool = True):
        super().__init__()
        self.s = s
        self.fused = fuse
        if fuse:
            self.qkv = fuse_along_n([linears["q_proj"], linears["k_proj"], linears["v_proj"]])
            self.gate_up = fuse_along_n([linears["gate_proj"], linears["up_proj"]])
        else:
            self.q_proj, self.k_proj, self.v_proj = linears["q_proj"], linears["k_proj"], linears["v_proj"]
            self.gate_proj, self.up_proj = linears["gate_proj"], linears["up_proj"]
        self.o_proj, self.down_proj = linears["o_proj"], linears["down_proj"]
        self.register_buffer("ln1", norms[0])
        self.register_buffer("ln2", norms[1])
        self.register_buffer("k_cache", torch.zeros(s.max_seq, s.n_kv_heads, s.head_dim, dtype=torch.float16,
                                                    device=norms[0].device))
        self.register_buffer("v_cache", torch.zeros_like(self.k_cache))


class FusedBuffers:
    """Static activations of the fused decode path (nothing is allocated per token)."""

    def __init__(self, s: LlamaShape, ws_bytes: int, device):
        d = s.head_dim
        f16 = dict(dtype=torch.float16, device=device)
        self.xa = torch.zeros(1, s.hidden, **f16)
        self.xb = torch.zeros(1, s.hidden, **f16)
        self.qkv = torch.zeros(1, (s.n_heads + 2 * s.n_kv_heads) * d, **f16)
        self.attn = torch.zeros(1, s.n_heads * d, **f16)
        self.gu = torch.zeros(1, 2 * s.ffn, **f16)
        self.ws = torch.zeros(ws_bytes, dtype=torch.uint8, device=device)
        self.logits = torch.zeros(1, s.vocab, **f16)
        # unsummed K slices of a q|k|v projection, read by the attention launch
        self.sq = torch.zeros(MAX_DEFERRED_SLICES, self.qkv.shape[1], dtype=torch.float32, device=device)
        # unsummed K slices of a down projection, read by the next layer's first launch
        self.sd = torch.zeros(MAX_DEFERRED_SLICES, s.hidden, dtype=torch.float32, device=device)


MAX_DEFERRED_SLICES = 4        # what a consuming launch accepts (elutq_gemv_fusion.n_slices_in)


def deferred_layer_step(layer: "DecoderLayer", b: FusedBuffers, pos: torch.Tensor, cur: torch.Tensor,
                        other: torch.Tensor, pending: int, last: bool, defer_qkv: bool = True,
                        defer_down: bool = True):
    """The same five launches with the K slices of the down projection left unsummed for the launch
    that reads them (the next layer's q|k|v), which forms fp16(slices + residual) itself, bit for
    bit what the producer's own output stage writes, and stores it for the later residual add.
    `cur` holds the residual stream, `other` is free; `pending` = slices of the previous layer's
    down waiting in b.sd (0 = none).  Returns (cur, other, pending).  `defer_qkv`: the q|k|v
    projection's K slices go to the attention launch the same way (head_dim 128), where a
    workgroup only sums the 3 x 128 elements of its own head.  `defer_down` = False: the launch that
    would read down's slices cannot take them (LlamaDecoder decides that per layer when it is built), so
    down sums them itself."""
    s = layer.s
    n_q = layer.qkv.slices
    defer_qkv = (defer_qkv and s.head_dim == 128 and 2 <= n_q <= MAX_DEFERRED_SLICES and layer.qkv.bias is None
                 and not layer.qkv.sparse_own_launch)
    layer.qkv.gemv_fused(cur, b.qkv, b.ws, prologue=1, norm_weight=layer.ln1, eps=s.rms_eps,
                         slices_in=b.sd[:pending] if pending else None, x_out=other if pending else None,
                         slices_out=b.sq if defer_qkv else None)
    if pending:
        cur, other = other, cur
    L, stream = _lib.lib(), torch.cuda.current_stream().cuda_stream
    if defer_qkv:
        rc = L.elutq_decode_rope_attn_sliced_f16(
            b.sq.data_ptr(), n_q, b.sq.shape[1], layer.k_cache.data_ptr(), layer.v_cache.data_ptr(), pos.data_ptr(),
            b.attn.data_ptr(), s.n_heads, s.n_kv_heads, s.head_dim, s.max_seq, s.rope_base, 0, b.ws.data_ptr(),
            b.ws.numel(), stream)
        _lib.check(rc, "elutq_decode_rope_attn_sliced_f16")
    else:
        rc = L.elutq_decode_rope_attn_split_f16(
            b.qkv.data_ptr(), layer.k_cache.data_ptr(), layer.v_cache.data_ptr(), pos.data_ptr(), b.attn.data_ptr(),
            s.n_heads, s.n_kv_heads, s.head_dim, s.max_seq, s.rope_base, 0, b.ws.data_ptr(), b.ws.numel(), stream)
        _lib.check(rc, "elutq_decode_rope_attn_split_f16")
    layer.o_proj.gemv_fused(b.attn, other, b.ws, residual=cur)
    layer.gate_up.gemv_fused(other, b.gu, b.ws, prologue=1, norm_weight=layer.ln2, eps=s.rms_eps)
    cur, other = other, cur
    n_d = layer.down_proj.slices
    if (not last and defer_down and 2 <= n_d <= MAX_DEFERRED_SLICES and layer.down_proj.bias is None
            and not layer.down_proj.sparse_own_launch):
        layer.down_proj.gemv_fused(b.gu, other, b.ws, prologue=2, slices_out=b.sd)
        return cur, other, n_d
    layer.down_proj.gemv_fused(b.gu, other, b.ws, prologue=2, residual=cur)
    return other, cur, 0


def fused_layer_step(layer: "DecoderLayer", b: FusedBuffers, pos: torch.Tensor) -> None:
    """One decoder layer in five launches: rmsnorm+qkv | rope+cache+attention | o+residual |
    rmsnorm+gate|up | silu*up+down+residual.  The residual stream enters and leaves in b.xa."""
    s = layer.s
    layer.qkv.gemv_fused(b.xa, b.qkv, b.ws, prologue=1, norm_weight=layer.ln1, eps=s.rms_eps)
    rc = _lib.lib().elutq_decode_rope_attn_split_f16(
        b.qkv.data_ptr(), layer.k_cache.data_ptr(), layer.v_cache.data_ptr(), pos.data_ptr(), b.attn.data_ptr(),
        s.n_heads, s.n_kv_heads, s.head_dim, s.max_seq, s.rope_base, 0, b.ws.data_ptr(), b.ws.numel(),
        torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "elutq_decode_rope_attn_split_f16")
    layer.o_proj.gemv_fused(b.attn, b.xb, b.ws, residual=b.xa)
    layer.gate_up.gemv_fused(b.xb, b.gu, b.ws, prologue=1, norm_weight=layer.ln2, eps=s.rms_eps)
    layer.down_proj.gemv_fused(b.gu, b.xa, b.ws, prologue=2, residual=b.xb)


PROJ_DIRS = {"q_proj": "self_attn.q_proj", "k_proj": "self_attn.k_proj", "v_proj": "self_attn.v_proj",
             "o_proj": "self_attn.o_proj", "gate_proj": "mlp.gate_proj", "up_proj": "mlp.up_proj",
             "down_proj": "mlp.down_proj"}


def proj_shapes(s: LlamaShape) -> dict:
    d = s.head_dim
    return {"q_proj": (s.hidden, s.n_heads * d), "k_proj": (s.hidden, s.n_kv_heads * d),
            "v_proj": (s.hidden, s.n_kv_heads * d), "o_proj": (s.n_heads * d, s.hidden),
            "gate_proj": (s.hidden, s.ffn), "up_proj": (s.hidden, s.ffn), "down_proj": (s.ffn, s.hidden)}


def random_parts(s: LlamaShape, dev, seed: int, hlq_lm_head: bool = False) -> dict:
    """Random-init weights of the shape (generated on the device).  `hlq_lm_head`: the lm_head is an HLQ
    layer of the model's bits and group size -- what the reference's exporter produces unless told to
    skip the lm_head (GPTQ/llama.py:143-176) -- instead of an fp16 matrix."""
    g = torch.Generator(device=dev).manual_seed(seed)
    layers = []
    sd = seed * 100_003
    for _ in range(s.n_layers):
        lin = {}
        for name, (k, n) in proj_shapes(s).items():
            lin[name] = make_device_layer(k, n, s.bits, s.group, seed=sd, device=dev)
            sd += 1
        norms = tuple((1.0 + 0.1 * torch.randn(s.hidden, generator=g, device=dev)).to(torch.float16) for _ in range(2))
        layers.append((lin, norms))
    embed = (torch.randn(s.vocab, s.hidden, generator=g, device=dev) * 0.5).to(torch.float16)
    if hlq_lm_head:
        lm_head = make_device_layer(s.hidden, s.vocab, s.bits, s.group, seed=sd, device=dev)
    else:
        lm_head = (torch.randn(s.vocab, s.hidden, generator=g, device=dev) * 0.02).to(torch.float16)
    norm = (1.0 + 0.1 * torch.randn(s.hidden, generator=g, device=dev)).to(torch.float16)
    return {"layers": layers, "embed": embed, "lm_head": lm_head, "norm": norm}


def parts_from_export(root: str, s: LlamaShape, dev, sparse_mode: str = "auto") -> dict:
    """Reads the reference's model export tree (written by GPTQ/llama.py:285-343, read by
    C++/examples/models/llama.cpp:59-115), or the same tree after `python -m elutq_amd.repack`.
    The lm_head is the HLQ layer in lm_head/lm_head if that directory exists, else lm_head.bin,
    else the (tied) embedding, in the order of llama.cpp:68-80."""
    import os
    from . import export_io as io

    def vec(path, n):
        return torch.from_numpy(io.read_fp16_bin(path, n)).to(dev)

    layers = []
    for i in range(s.n_layers):
        base = os.path.join(root, str(i))
        lin = {}
        for name, (k, n) in proj_shapes(s).items():
            m = HLQLinear.from_export_dir(os.path.join(base, PROJ_DIRS[name]), dev, sparse_mode=sparse_mode)
            if (m.in_features, m.out_features) != (k, n):
                raise ValueError(f"{base}/{PROJ_DIRS[name]}: {m.in_features}x{m.out_features}, the shape needs {k}x{n}")
            lin[name] = m
        layers.append((lin, tuple(vec(os.path.join(base, f), s.hidden) for f in io.LAYER_NORMS)))
    embed = vec(io.embedding_file(root), s.vocab * s.hidden).view(s.vocab, s.hidden)
    kind = io.lm_head_kind(root)
    if kind == "hlq":
        lm_head = HLQLinear.from_export_dir(os.path.join(root, "lm_head", "lm_head"), dev, sparse_mode=sparse_mode)
        if (lm_head.in_features, lm_head.out_features) != (s.hidden, s.vocab):
            raise ValueError("lm_head/lm_head does not match hidden x vocab")
    elif kind == "fp16":
        lm_head = vec(os.path.join(root, "lm_head.bin"), s.vocab * s.hidden).view(s.vocab, s.hidden)
    else:
        lm_head = None
    return {"layers": layers, "embed": embed, "lm_head": lm_head,
            "norm": vec(os.path.join(root, "final_rmsnorm_weight.bin"), s.hidden)}


class LlamaDecoder(nn.Module):
    """Random-init LLaMA-shaped decoder for the decode benchmark and its parity test."""

    FUSED_LAUNCHES = True      # (a subclass that steps through other operators sets this to False: no launch buffers)

    def __init__(self, s: LlamaShape, device="cuda", seed: int = 0, fuse: bool = True,
                 parts: dict | None = None, qkv_to_attention: bool = True):
        """Five fused launches per layer through the C ABI (q|k|v and gate|up fused along N: fuse=True).
        qkv_to_attention: run q|k|v in two K slices that the attention launch sums (head_dim 128) rather than
        on the narrow-tile kernel (measured on MI355X at the LLaMA-3-8B shape: 835 against 817 tokens/s)."""
        super().__init__()
        assert fuse or not self.FUSED_LAUNCHES
        self.s = s
        dev = torch.device(device)
        d = s.head_dim
        if parts is None:
            parts = random_parts(s, dev, seed)
        self.layers = nn.ModuleList([DecoderLayer(s, lin, norms, fuse) for lin, norms in parts["layers"]])
        self.register_buffer("embed", parts["embed"])
        self.register_buffer("norm", parts["norm"])
        # lm_head: fp16 [vocab, hidden] (lm_head.bin, or the embedding when tied) or an HLQ layer
        head = parts["lm_head"] if parts["lm_head"] is not None else parts["embed"]
        self.lm_head_q = head if isinstance(head, HLQLinear) else None
        self.register_buffer("lm_head", None if isinstance(head, HLQLinear) else head)
        inv = s.rope_base ** (-torch.arange(0, d, 2, device=dev, dtype=torch.float32) / d)
        ang = torch.arange(s.max_seq, device=dev, dtype=torch.float32)[:, None] * inv[None, :]
        self.register_buffer("cos_t", ang.cos())
        self.register_buffer("sin_t", ang.sin())
        self.register_buffer("arange", torch.arange(s.max_seq, device=dev))
        # state of the decode loop (device resident so a captured step can advance it)
        self.register_buffer("token", torch.zeros(1, dtype=torch.long, device=dev))
        self.register_buffer("pos", torch.zeros(1, dtype=torch.long, device=dev))
        self._graph = None
        self._buf = None
        # leave the K slices of down to the launch that reads them (deferred_layer_step); the
        # logits are bit for bit those of fused_layer_step.  Set before capture().
        self.defer_slices = True
        self.defer_qkv = False             # likewise q|k|v -> attention (set by the constructor, see qkv_to_attention)
        if self.FUSED_LAUNCHES:
            ws = max(m.workspace_bytes for m in self.modules() if isinstance(m, HLQLinear))
            ws = max(ws, _lib.lib().elutq_decode_attn_workspace_bytes(s.n_heads, s.head_dim, 0))
            self._buf = FusedBuffers(s, ws, dev)
            # q|k|v in two K slices where that still leaves at most one workgroup per compute unit: the
            # attention launch sums the slices of its own head for free, so the projection gets twice
            # the workgroups without the meeting that otherwise makes the split a loss
            # (LLaMA-3-8B: 96 -> 192 workgroups, 6.7 -> 5.7 us).  The alternative: narrow tiles (two
            # workgroups per column block, all of K each), nothing for the attention to sum.
            self.defer_qkv = bool(qkv_to_attention) and d == 128
            if self.defer_qkv:
                for layer in self.layers:
                    q = layer.qkv
                    if q.sparse_own_launch:
                        continue                         # its plane's launch reads the stored input: no slices
                    if q.bias is None and q.slices == 1 and 2 * ((q.out_features + 63) // 64) <= 256:
                        q.ksplit, q.waves = 2, 16
                    elif q.ksplit == 0:
                        q.ksplit = _lib.GEMV_WIDE        # a launch that leaves K slices runs on the wide-tile kernel
            # down leaves its K slices unsummed only where the next layer's q|k|v launch takes them (a q|k|v
            # with more tiles than compute units, or tables that leave no room for the staged activations,
            # does not): decided here, once, so that a step never meets a refusing launch
            self._defer_down = [i + 1 < len(self.layers) and 2 <= layer.down_proj.slices <= MAX_DEFERRED_SLICES
                                and not layer.down_proj.sparse_own_launch and not self.layers[i + 1].qkv.sparse_own_launch
                                and self.layers[i + 1].qkv.accepts_slices(layer.down_proj.slices)
                                for i, layer in enumerate(self.layers)]
            # a launch that leaves its K slices to the next one runs on the wide-tile kernel: a down that may do so
            # is pinned to it, so that the step computes the same bits whether or not the slices are handed over
            for i, layer in enumerate(self.layers):
                if self._defer_down[i] and layer.down_proj.ksplit == 0:
                    layer.down_proj.ksplit = _lib.GEMV_WIDE

    @classmethod
    def from_export(cls, root: str, s: LlamaShape, device="cuda", fuse: bool = True,
                    sparse_mode: str = "auto") -> "LlamaDecoder":
        """A decoder over a genuinely exported model (bits and group size come from the files)."""
        return cls(s, device=device, fuse=fuse, parts=parts_from_export(root, s, torch.device(device), sparse_mode))

    @torch.no_grad()
    def fill_cache(self, n_tokens: int, seed: int = 1) -> None:
        """Random fp16 KV entries for positions [0, n_tokens): the 'context already decoded'."""
        g = torch.Generator(device=self.embed.device).manual_seed(seed)
        for layer in self.layers:
            layer.k_cache[:n_tokens] = torch.randn(n_tokens, self.s.n_kv_heads, self.s.head_dim, generator=g,
                                                   device=self.embed.device).to(torch.float16)
            layer.v_cache[:n_tokens] = torch.randn(n_tokens, self.s.n_kv_heads, self.s.head_dim, generator=g,
                                                   device=self.embed.device).to(torch.float16)
        self.pos.fill_(n_tokens)

    @torch.no_grad()
    def step(self) -> torch.Tensor:
        """One decode step from the device-resident (token, pos); stores the greedy next token
        and pos + 1 back.  Returns the logits [1, vocab] (fp16)."""
        b = self._buf
        _lib.check(_lib.lib().elutq_decode_embed_f16(self.embed.data_ptr(), self.token.data_ptr(), b.xa.data_ptr(),
                                                     self.s.hidden, self.s.vocab,
                                                     torch.cuda.current_stream().cuda_stream), "elutq_decode_embed_f16")
        if self.defer_slices:
            x, free, pending = b.xa, b.xb, 0
            for i, layer in enumerate(self.layers):
                x, free, pending = deferred_layer_step(layer, b, self.pos, x, free, pending,
                                                       last=i == len(self.layers) - 1, defer_qkv=self.defer_qkv,
                                                       defer_down=self._defer_down[i])
        else:
            for layer in self.layers:
                fused_layer_step(layer, b, self.pos)
            x, free = b.xa, b.xb
        L, stream = _lib.lib(), torch.cuda.current_stream().cuda_stream
        if self.lm_head_q is not None:       # the final norm rides in the GEMV's prologue
            logits = self.lm_head_q.gemv_fused(x, b.logits, b.ws, prologue=1, norm_weight=self.norm,
                                               eps=self.s.rms_eps)
        elif self.s.hidden % 8 == 0 and self.s.hidden <= 32768 and self.lm_head.data_ptr() % 16 == 0:
            # the unquantized lm_head: the library's dense fp16 GEMV, the final norm in the same launch
            logits = b.logits
            _lib.check(L.elutq_fp16_gemv_f16(self.lm_head.data_ptr(), None, x.data_ptr(), logits.data_ptr(), self.s.hidden,
                                             self.s.vocab, self.norm.data_ptr(), self.s.rms_eps, stream),
                       "elutq_fp16_gemv_f16")
        else:
            _lib.check(L.elutq_decode_rmsnorm_f16(x.data_ptr(), self.norm.data_ptr(), free.data_ptr(),
                                                  self.s.hidden, self.s.rms_eps, stream), "elutq_decode_rmsnorm_f16")
            logits = torch.mm(free, self.lm_head.t(), out=b.logits)
        _lib.check(L.elutq_decode_argmax_ws_f16(logits.data_ptr(), self.s.vocab, self.token.data_ptr(),
                                                self.pos.data_ptr(), b.ws.data_ptr(), b.ws.numel(), stream),
                   "elutq_decode_argmax_ws_f16")
        return logits

    @torch.no_grad()
    def capture(self) -> None:
        """Captures step() in a HIP graph (after eager warm-up steps that size the scratch)."""
        state = (self.token.clone(), self.pos.clone())
        s = torch.cuda.Stream()
        with torch.cuda.stream(s):
            for _ in range(2):
                self.step()
        s.synchronize()
        self.token.copy_(state[0])
        self.pos.copy_(state[1])
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            self._logits = self.step()
        self._graph = g
        self.token.copy_(state[0])
        self.pos.copy_(state[1])
        torch.cuda.synchronize()

    def replay(self) -> None:
        self._graph.replay()


def bench_decode(device, n_ctx: int = 512, n_gen: int = 50, shape: LlamaShape | None = None,
                 hlq_lm_head: bool = False) -> dict:
    """Decode tokens/s of the random-init model: n_gen greedy tokens after an n_ctx-token
    cache; the first generated token is excluded, as in the reference
    ((generate_num - 1) / elapsed, main.cpp:110).  `hlq_lm_head`: see random_parts."""
    s = shape or LlamaShape()
    if n_ctx + n_gen > s.max_seq:
        # the attention launch of a position beyond the cache returns at once (NaN output): such tokens must not be timed
        raise ValueError(f"n_ctx + n_gen = {n_ctx + n_gen} exceeds the cache of {s.max_seq} positions")
    dev = torch.device(device)
    model = LlamaDecoder(s, device=dev, seed=0, parts=random_parts(s, dev, 0, hlq_lm_head))
    model.fill_cache(n_ctx)
    model.token.fill_(1)
    model.capture()
    # one untimed pass over the same n_gen tokens (the GPU's clocks follow the load with a delay of some tens of
    # milliseconds, about the length of the whole measurement), then the same tokens again, timed: the cache rows the
    # pass wrote are written again with the same values
    for _ in range(n_gen):
        model.replay()
    model.pos.fill_(n_ctx)
    model.token.fill_(1)
    model.replay()                           # token 1 (excluded)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n_gen - 1):
        model.replay()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    hlq_bytes = sum(m.planes.numel() + m.scales.numel() + m.zeros.numel()
                    for m in model.modules() if isinstance(m, HLQLinear))
    lm_bytes = model.lm_head.numel() * 2 if model.lm_head is not None else 0
    kv_bytes = 2 * s.n_layers * n_ctx * s.n_kv_heads * s.head_dim * 2
    ms = dt / (n_gen - 1) * 1e3
    return {"tokens_per_s": (n_gen - 1) / dt, "ms_per_token": ms, "n_ctx": n_ctx, "n_gen": n_gen,
            "bytes_per_token": hlq_bytes + lm_bytes + kv_bytes,
            "GBps": (hlq_bytes + lm_bytes + kv_bytes) / (ms * 1e-3) / 1e9,
            "model": f"LLaMA-3-8B-shaped random init, {s.n_layers} layers, HLQ w{s.bits}g{s.group}, "
                     + (f"HLQ w{s.bits}g{s.group} lm_head" if hlq_lm_head else "fp16 lm_head"),
            "glue": "5 launches per layer (rmsnorm+qkv | rope+cache+attention | o+residual | rmsnorm+gate|up | "
                    "silu*up+down+residual; the K slices of q|k|v and of down are summed by the launch that reads "
                    "them), own embedding gather and argmax kernels, "
                    + ("HLQ GEMV lm_head, " if hlq_lm_head else "own dense fp16 GEMV lm_head, ") + "the final norm inside the lm_head launch, "
                    + "one HIP graph per token"}
