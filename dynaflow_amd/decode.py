"""Decode step (one new token per sequence) over stacked Llama-shaped layers with static KV caches.

What reaches DynaFlow in the reference is the host framework's decode graph: per layer a norm, the
QKV projection, an opaque attention custom op working on the framework's KV cache, the output
projection and the MLP (``examples/ae/scheduler/vllm/nanoflow.py:58-95`` splits and tags exactly
these pieces).  This module is that graph for the build's own measurements:

* the caches are module buffers (static device memory, one slot per sequence), so the whole
  two-stream schedule can be captured once and replayed;
* every token carries its cache slot and its attention length (``slots``, ``lengths``: token-shaped
  inputs, cut per nano-batch by the engine like the activations);
* ``attend_and_append`` is an operator of its own (``dynaflow_model::attend_and_append``, declared
  to mutate the two caches), so it is ONE graph node; on the GPU the HIP lowering replaces it with
  ``dynaflow_hip.decode_attention``; its body below is the definition in plain tensor operations,
  used on the host.

Cache layout (head_dim 128): ``k_cache [slots, kv_heads, capacity, 128]``,
``v_cache [slots, kv_heads, capacity / 8, 128, 8]`` (8 consecutive positions of one dim contiguous).
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from dynaflow_amd.decoder import MLPBlock, rope_tables

HEAD_DIM = 128


def pack_v_cache(v: torch.Tensor) -> torch.Tensor:
    """[slots, kv_heads, capacity, 128] -> the blocked layout [slots, kv_heads, capacity/8, 128, 8]."""
    s, h, c, d = v.shape
    return v.view(s, h, c // 8, 8, d).permute(0, 1, 2, 4, 3).contiguous()


def unpack_v_cache(v_cache: torch.Tensor) -> torch.Tensor:
    """Inverse of :func:`pack_v_cache`."""
    s, h, blocks, d, _ = v_cache.shape
    return v_cache.permute(0, 1, 2, 4, 3).reshape(s, h, blocks * 8, d)


@torch.library.custom_op("dynaflow_model::attend_and_append", mutates_args=("k_cache", "v_cache"))
def attend_and_append(qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, slots: torch.Tensor,
                      lengths: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, q_heads: int,
                      kv_heads: int) -> torch.Tensor:
    """Rotate q and k of the new tokens, append k and v to the caches, attend over the cache.

    Token t belongs to cache slot ``slots[t]``, sits at position ``lengths[t] - 1`` and attends to
    positions ``0 .. lengths[t] - 1``.  qkv is ``[T, (q_heads + 2 kv_heads) * 128]``.

    Declared as an operator that mutates the two caches: a function that writes to its inputs must not
    be handed to dynamo as a plain in-graph function.
    """
    T, d = qkv.shape[0], HEAD_DIM
    capacity = k_cache.shape[2]
    q, k, v = qkv.split([q_heads * d, kv_heads * d, kv_heads * d], dim=-1)
    pos = (lengths - 1).long()
    sl = slots.long()
    c, s = cos[pos][:, None, :], sin[pos][:, None, :]

    def rotate(t: torch.Tensor) -> torch.Tensor:
        t = t.reshape(T, -1, d).float()
        lo, hi = t[..., : d // 2], t[..., d // 2:]
        return torch.cat([lo * c - hi * s, hi * c + lo * s], dim=-1).to(qkv.dtype)

    q, k = rotate(q), rotate(k)
    k_cache[sl, :, pos] = k
    v_cache[sl, :, pos // 8, :, pos % 8] = v.reshape(T, kv_heads, d)
    keys = k_cache[sl].float()                                   # [T, kv, capacity, d]
    values = unpack_v_cache(v_cache[sl]).float()
    group = q_heads // kv_heads
    scores = torch.einsum("tkgd,tkpd->tkgp", q.float().view(T, kv_heads, group, d), keys) / math.sqrt(d)
    masked = torch.arange(capacity, device=qkv.device)[None, :] >= lengths[:, None]
    scores = scores.masked_fill(masked[:, None, None, :], float("-inf"))
    out = torch.einsum("tkgp,tkpd->tkgd", torch.softmax(scores, dim=-1), values)
    return out.reshape(T, q_heads * d).to(qkv.dtype)


@attend_and_append.register_fake
def _(qkv, k_cache, v_cache, slots, lengths, cos, sin, q_heads, kv_heads):
    return qkv.new_empty((qkv.shape[0], q_heads * HEAD_DIM))


class DecodeAttentionBlock(nn.Module):
    def __init__(self, hidden: int, heads: int, kv_heads: int, slots: int, capacity: int, eps: float, dtype,
                 device=None) -> None:
        super().__init__()
        assert capacity % 32 == 0 and heads % kv_heads == 0
        self.heads, self.kv_heads, self.eps = heads, kv_heads, eps
        kw = dict(dtype=dtype, device=device)
        self.norm_weight = nn.Parameter(torch.ones(hidden, **kw))
        self.wqkv = nn.Parameter(torch.empty((heads + 2 * kv_heads) * HEAD_DIM, hidden, **kw))
        self.wo = nn.Parameter(torch.empty(hidden, heads * HEAD_DIM, **kw))
        self.register_buffer("k_cache", torch.zeros(slots, kv_heads, capacity, HEAD_DIM, **kw), persistent=False)
        self.register_buffer("v_cache", torch.zeros(slots, kv_heads, capacity // 8, HEAD_DIM, 8, **kw),
                             persistent=False)

    def forward(self, x, slots, lengths, cos, sin):
        h = F.rms_norm(x, (x.shape[-1],), self.norm_weight, self.eps)
        qkv = F.linear(h, self.wqkv)
        attn = attend_and_append(qkv, self.k_cache, self.v_cache, slots, lengths, cos, sin, self.heads,
                                 self.kv_heads)
        return x + F.linear(attn, self.wo)


class DecodeModel(nn.Module):
    """Token embedding + ``layers`` decoder layers; one new token per sequence."""

    def __init__(self, layers: int = 32, vocab: int = 128256, hidden: int = 4096, heads: int = 32,
                 kv_heads: int = 8, inter: int = 14336, slots: int = 256, capacity: int = 2048,
                 theta: float = 500000.0, eps: float = 1e-5, dtype=torch.bfloat16, device=None) -> None:
        super().__init__()
        self.embed = nn.Parameter(torch.empty(vocab, hidden, dtype=dtype, device=device))
        self.attn = nn.ModuleList(
            DecodeAttentionBlock(hidden, heads, kv_heads, slots, capacity, eps, dtype, device) for _ in range(layers)
        )
        self.mlp = nn.ModuleList(MLPBlock(hidden, inter, eps, dtype, device) for _ in range(layers))
        cos, sin = rope_tables(capacity, HEAD_DIM, theta, torch.float32, device)
        self.register_buffer("cos", cos, persistent=False)
        self.register_buffer("sin", sin, persistent=False)

    def forward(self, token_ids: torch.Tensor, slots: torch.Tensor, lengths: torch.Tensor) -> torch.Tensor:
        x = F.embedding(token_ids, self.embed)
        for attn, mlp in zip(self.attn, self.mlp):
            x = mlp(attn(x, slots, lengths, self.cos, self.sin))
        return x

    @torch.no_grad()
    def init_weights(self, seed: int = 0, std: float = 0.02) -> None:
        """Seeded N(0, std) weights (embedding N(0, 1)); generated on the parameter's device."""
        gen = torch.Generator(device=self.embed.device).manual_seed(seed)
        for p in self.parameters():
            if p.dim() == 1:
                continue
            scale = 1.0 if p is self.embed else std
            chunk = 1 << 26
            flat = p.view(-1)
            for off in range(0, flat.numel(), chunk):
                n = min(chunk, flat.numel() - off)
                flat[off:off + n].copy_(
                    (torch.randn(n, generator=gen, dtype=torch.float32, device=p.device) * scale).to(p.dtype))

    @torch.no_grad()
    def fill_caches(self, seed: int = 5) -> None:
        """Standard-normal cache contents (the synthetic history of every sequence)."""
        gen = torch.Generator(device=self.embed.device).manual_seed(seed)
        for block in self.attn:
            for cache in (block.k_cache, block.v_cache):
                flat = cache.view(-1)
                chunk = 1 << 26
                for off in range(0, flat.numel(), chunk):
                    n = min(chunk, flat.numel() - off)
                    flat[off:off + n].copy_(
                        torch.randn(n, generator=gen, dtype=torch.float32, device=cache.device).to(cache.dtype))
