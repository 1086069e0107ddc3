"""Llama-style decoder layer for the attention-beside-MLP schedule.

The layer is written so that dynamo attributes every traced node to exactly one
of two blocks (weights are plain ``nn.Parameter``s used through ``F.linear``;
there are no ``nn.Linear`` sub-modules whose nodes would be attributed one level
deeper), which lets a single ``Mod`` rule cut the graph:

    AttentionBlock   x + o_proj(attention(rope(q), rope(k), v)) on rms_norm(x)
    MLPBlock         x + down(silu(gate(h)) * up(h)),  h = rms_norm(x)

Tokens are flattened, ``x[T, H]`` with ``T = B * seq_len``; ``seq_len`` is a
constructor constant, so a nano-batch (a whole number of sequences) keeps the
layout.  Everything is plain PyTorch and also runs on the CPU; on the GPU the
lowering pass moves the projections, SiLU*mul, RMSNorm, RoPE and (at head_dim
128 and sequence lengths that are multiples of 64) the causal attention onto the
HIP operators; other attention shapes stay on PyTorch's fused attention kernel.

In the reference the layer is host-model code: the decoder layer of the HF Llama
that examples/ae/scripts/bench_hf_transformers.py:206-210 loads and traces.
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn
import torch.nn.functional as F


def rope_tables(seq_len: int, head_dim: int, theta: float, dtype=torch.float32, device=None):
    """cos / sin of shape [seq_len, head_dim / 2] for positions 0 .. seq_len-1."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float64, device=device) / head_dim))
    angles = torch.arange(seq_len, dtype=torch.float64, device=device)[:, None] * inv_freq[None, :]
    return torch.cos(angles).to(dtype), torch.sin(angles).to(dtype)


@torch._dynamo.allow_in_graph
def apply_rope(t: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Rotate pairs (t[..., i], t[..., i + d/2]) - the half-split convention of Llama checkpoints.

    ``t`` is [B, S, heads, d]; cos / sin are [S, d/2].  Arithmetic in fp32, one rounding.
    Dynamo keeps a call of this function as ONE graph node (it does not trace into it), which the
    HIP lowering replaces with the fused ``dynaflow_hip.rope`` kernel.
    """
    d2 = t.shape[-1] // 2
    tf = t.float()
    lo, hi = tf[..., :d2], tf[..., d2:]
    c, s = cos[None, :, None, :], sin[None, :, None, :]
    return torch.cat((lo * c - hi * s, hi * c + lo * s), dim=-1).to(t.dtype)


@torch._dynamo.allow_in_graph
def causal_gqa_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """Causal grouped-query attention: q [B, S, Hq, d], k / v [B, S, Hkv, d] -> [B, S, Hq, d].

    ONE graph node for dynamo (it does not trace into it); the HIP lowering replaces it with the
    ``dynaflow_hip.causal_attention`` kernel, this body is the definition in plain tensor operations.
    """
    out = F.scaled_dot_product_attention(
        q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), is_causal=True, enable_gqa=True
    )
    return out.transpose(1, 2)


class AttentionBlock(nn.Module):
    def __init__(self, hidden: int, heads: int, kv_heads: int, head_dim: int, seq_len: int, theta: float,
                 eps: float, dtype, device=None) -> None:
        super().__init__()
        self.heads, self.kv_heads, self.head_dim, self.seq_len, self.eps = heads, kv_heads, head_dim, seq_len, eps
        kw = dict(dtype=dtype, device=device)
        self.norm_weight = nn.Parameter(torch.ones(hidden, **kw))
        self.wq = nn.Parameter(torch.empty(heads * head_dim, hidden, **kw))
        self.wk = nn.Parameter(torch.empty(kv_heads * head_dim, hidden, **kw))
        self.wv = nn.Parameter(torch.empty(kv_heads * head_dim, hidden, **kw))
        self.wo = nn.Parameter(torch.empty(hidden, heads * head_dim, **kw))
        cos, sin = rope_tables(seq_len, head_dim, theta, torch.float32, device)
        self.register_buffer("cos", cos, persistent=False)
        self.register_buffer("sin", sin, persistent=False)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        h = F.rms_norm(x, (x.shape[-1],), self.norm_weight, self.eps)
        q = F.linear(h, self.wq).view(-1, self.seq_len, self.heads, self.head_dim)
        k = F.linear(h, self.wk).view(-1, self.seq_len, self.kv_heads, self.head_dim)
        v = F.linear(h, self.wv).view(-1, self.seq_len, self.kv_heads, self.head_dim)
        q = apply_rope(q, self.cos, self.sin)
        k = apply_rope(k, self.cos, self.sin)
        attn = causal_gqa_attention(q, k, v).reshape(-1, self.heads * self.head_dim)
        return x + F.linear(attn, self.wo)


class MLPBlock(nn.Module):
    def __init__(self, hidden: int, inter: int, eps: float, dtype, device=None) -> None:
        super().__init__()
        self.eps = eps
        kw = dict(dtype=dtype, device=device)
        self.norm_weight = nn.Parameter(torch.ones(hidden, **kw))
        self.w_gate = nn.Parameter(torch.empty(inter, hidden, **kw))
        self.w_up = nn.Parameter(torch.empty(inter, hidden, **kw))
        self.w_down = nn.Parameter(torch.empty(hidden, inter, **kw))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        h = F.rms_norm(x, (x.shape[-1],), self.norm_weight, self.eps)
        g = F.linear(h, self.w_gate)
        u = F.linear(h, self.w_up)
        return x + F.linear(F.silu(g) * u, self.w_down)


class DecoderLayer(nn.Module):
    """Token embedding + one decoder layer; input is a flat vector of token ids."""

    def __init__(self, vocab: int = 128256, hidden: int = 4096, heads: int = 32, kv_heads: int = 8,
                 head_dim: int = 128, inter: int = 14336, seq_len: int = 2048, theta: float = 500000.0,
                 eps: float = 1e-5, dtype=torch.bfloat16, device=None) -> None:
        super().__init__()
        self.embed = nn.Parameter(torch.empty(vocab, hidden, dtype=dtype, device=device))
        self.attn = AttentionBlock(hidden, heads, kv_heads, head_dim, seq_len, theta, eps, dtype, device)
        self.mlp = MLPBlock(hidden, inter, eps, dtype, device)

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        x = F.embedding(token_ids, self.embed)
        return self.mlp(self.attn(x))

    @torch.no_grad()
    def init_weights(self, seed: int = 0, std: float = 0.02) -> None:
        """Seeded N(0, std) weights generated on the CPU in fp32 (norm weights stay 1)."""
        for i, p in enumerate([self.embed, self.attn.wq, self.attn.wk, self.attn.wv, self.attn.wo,
                               self.mlp.w_gate, self.mlp.w_up, self.mlp.w_down]):
            g = torch.Generator(device="cpu").manual_seed(seed + 10 + i)
            scale = 1.0 if p is self.embed else std
            chunk = 1 << 24
            flat = p.view(-1)
            for off in range(0, flat.numel(), chunk):
                n = min(chunk, flat.numel() - off)
                flat[off:off + n].copy_((torch.randn(n, generator=g, dtype=torch.float32) * scale).to(p.dtype))
