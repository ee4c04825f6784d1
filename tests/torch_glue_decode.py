"""The decode step of elutq_amd.llama_decode written with PyTorch-ROCm operators around plain HLQLinear calls: the parity
partner of the fused HIP path in the decode tests (it does not touch the oracle: every projection is still the library's
GEMV; what differs is everything around the projections).  Same reference semantics as the fused launches restate:
RMSNorm in fp32 with fp16 output (C++/ops/src/arm/arm_rmsnorm.cpp:25-84), half-split RoPE (arm_rotary.cpp:31-46), fp32
softmax and the GQA head map (arm_attention.cpp:199-274), SiLU * up in fp32 (arm_activation.cpp:36-49), greedy argmax
(arm_argmax.cpp:21-29)."""
import torch
import torch.nn.functional as F

from elutq_amd.llama_decode import LlamaDecoder


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(torch.float16)


def rope(t: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Half-split rotation: pairs (j, j + d/2)."""
    d2 = t.shape[-1] // 2
    a, b = t[..., :d2].float(), t[..., d2:].float()
    return torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1).to(torch.float16)


def layer_forward(layer, x, pos, cos, sin, mask):
    """x [1, hidden] fp16; pos int64 [1] (device); cos/sin [1, head_dim/2] fp32 at pos;
    mask [1, 1, max_seq] additive fp32 (0 up to pos, -inf beyond)."""
    s = layer.s
    d, nq, nkv = s.head_dim, s.n_heads, s.n_kv_heads
    h = rms_norm(x, layer.ln1, s.rms_eps)
    if layer.fused:
        qkv = layer.qkv(h)
        q, k, v = qkv.split([nq * d, nkv * d, nkv * d], dim=-1)
    else:
        q, k, v = layer.q_proj(h), layer.k_proj(h), layer.v_proj(h)
    q = rope(q.view(nq, d), cos, sin)
    k = rope(k.view(nkv, d), cos, sin)
    layer.k_cache.index_copy_(0, pos, k.unsqueeze(0))
    layer.v_cache.index_copy_(0, pos, v.reshape(1, nkv, d))
    # single-token GQA attention over the whole cache buffer, masked beyond pos
    qg = q.view(nkv, nq // nkv, d).float()
    kc = layer.k_cache.permute(1, 2, 0).float()                 # [nkv, d, L]
    scores = torch.matmul(qg, kc) * (d ** -0.5) + mask          # [nkv, nq/nkv, L]
    p = torch.softmax(scores, dim=-1)
    ctx = torch.matmul(p, layer.v_cache.permute(1, 0, 2).float())   # [nkv, nq/nkv, d]
    attn = ctx.to(torch.float16).reshape(1, nq * d)
    x = x + layer.o_proj(attn)
    h = rms_norm(x, layer.ln2, s.rms_eps)
    if layer.fused:
        g, u = layer.gate_up(h).split([s.ffn, s.ffn], dim=-1)
    else:
        g, u = layer.gate_proj(h), layer.up_proj(h)
    act = (F.silu(g.float()) * u.float()).to(torch.float16)
    return x + layer.down_proj(act)


class TorchGlueDecoder(LlamaDecoder):
    """LlamaDecoder whose step runs PyTorch operators around the HLQ projections (fused along N or not)."""
    FUSED_LAUNCHES = False

    @torch.no_grad()
    def step(self) -> torch.Tensor:
        x = self.embed.index_select(0, self.token)
        cos = self.cos_t.index_select(0, self.pos)
        sin = self.sin_t.index_select(0, self.pos)
        mask = torch.where(self.arange <= self.pos, 0.0, float("-inf")).view(1, 1, -1)
        for layer in self.layers:
            x = layer_forward(layer, x, self.pos, cos, sin, mask)
        xn = rms_norm(x, self.norm, self.s.rms_eps)
        logits = self.lm_head_q(xn) if self.lm_head_q is not None else F.linear(xn, self.lm_head)
        self.token.copy_(logits.argmax(-1))
        self.pos.add_(1)
        return logits


def make_decoder(impl: str, *args, **kw):
    """impl "hip": the library's fused decode step; "torch": the PyTorch-glue step."""
    return (LlamaDecoder if impl == "hip" else TorchGlueDecoder)(*args, **kw)


def decoder_from_export(impl: str, *args, **kw):
    return (LlamaDecoder if impl == "hip" else TorchGlueDecoder).from_export(*args, **kw)
