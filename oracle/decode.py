"""Float64 restatement of one decode step over stacked decoder layers with KV caches.

Test infrastructure (see the package header).  Written independently of the product module:
caches in the natural layout ``[slots, capacity, kv_heads, d]``, RoPE as a complex multiplication
by ``exp(i * pos * theta^(-2j/d))``, attention as an explicit loop over tokens and heads with a
plain softmax over the first ``length`` positions.  What the reference computes at this point is
the host framework's attention custom op on its own paged cache (an opaque FX node for DynaFlow,
``examples/ae/scheduler/vllm/nanoflow.py:89-95``); the definition restated here is the textbook one.

PARITY UNPINNED against reference outputs: the reference ships none for this path.  Pinned by
special cases instead (tests/test_decode_cpu.py): length 1 returns v of the new token, uniform V
returns that V, appending then attending equals attention over the concatenated history, and the
prefill oracle (``oracle.decoder``) run on the full sequence gives the same last-token output.
"""
from __future__ import annotations

import torch

from oracle.decoder import rms_norm


def rope_at(t: torch.Tensor, pos: torch.Tensor, theta: float) -> torch.Tensor:
    """t [T, heads, d] rotated by the angles of positions pos [T] (half-split pairing)."""
    d = t.shape[-1]
    inv = theta ** (-torch.arange(0, d, 2, dtype=torch.float64) / d)
    phase = torch.polar(torch.ones(pos.shape[0], d // 2, dtype=torch.float64), pos.double()[:, None] * inv[None, :])
    z = torch.complex(t[..., : d // 2].double(), t[..., d // 2:].double()) * phase[:, None, :]
    return torch.cat([z.real, z.imag], dim=-1)


def attend(q: torch.Tensor, keys: torch.Tensor, values: torch.Tensor) -> torch.Tensor:
    """q [heads, d]; keys / values [L, kv_heads, d] -> [heads, d]; query head h reads kv head h // group."""
    heads, d = q.shape
    group = heads // keys.shape[1]
    out = torch.empty(heads, d, dtype=torch.float64)
    for h in range(heads):
        s = keys[:, h // group, :] @ q[h] / d ** 0.5
        p = torch.exp(s - s.max())
        out[h] = (p / p.sum()) @ values[:, h // group, :]
    return out


def decode_layer(x, slots, lengths, params, i, k_cache, v_cache, heads, kv_heads, theta=500000.0, eps=1e-5):
    """Layer ``i`` of the step on hidden states ``x [T, hidden]`` (float64): attention block, then MLP block.
    ``k_cache`` / ``v_cache``: that layer's caches, float64 ``[slots, capacity, kv_heads, d]``, updated in place
    (token t's key and value go to position ``lengths[t] - 1`` of slot ``slots[t]``).  Returns ``[T, hidden]``."""
    d = k_cache.shape[-1]
    T = x.shape[0]
    pos = lengths.long() - 1
    h = rms_norm(x, params[f"attn_norm.{i}"], eps)
    qkv = h @ params[f"wqkv.{i}"].t()
    q = rope_at(qkv[:, : heads * d].reshape(T, heads, d), pos, theta)
    k = rope_at(qkv[:, heads * d: (heads + kv_heads) * d].reshape(T, kv_heads, d), pos, theta)
    v = qkv[:, (heads + kv_heads) * d:].reshape(T, kv_heads, d)
    attn = torch.empty(T, heads * d, dtype=torch.float64)
    for t in range(T):
        s, L = int(slots[t]), int(lengths[t])
        k_cache[s, L - 1] = k[t]
        v_cache[s, L - 1] = v[t]
        attn[t] = attend(q[t], k_cache[s, :L], v_cache[s, :L]).reshape(-1)
    x = x + attn @ params[f"wo.{i}"].t()
    h = rms_norm(x, params[f"mlp_norm.{i}"], eps)
    g = h @ params[f"w_gate.{i}"].t()
    return x + ((g / (1 + torch.exp(-g))) * (h @ params[f"w_up.{i}"].t())) @ params[f"w_down.{i}"].t()


def decode_step(token_ids, slots, lengths, params, k_caches, v_caches, heads, kv_heads, theta=500000.0, eps=1e-5):
    """One new token per sequence.  ``params``: dict with ``embed`` and per layer i ``attn_norm.i``, ``wqkv.i``,
    ``wo.i``, ``mlp_norm.i``, ``w_gate.i``, ``w_up.i``, ``w_down.i`` (float64).  ``k_caches[i]`` /
    ``v_caches[i]``: float64 ``[slots, capacity, kv_heads, d]``, updated in place.  Returns ``[T, hidden]``."""
    x = params["embed"][token_ids.long()]
    for i in range(len(k_caches)):
        x = decode_layer(x, slots, lengths, params, i, k_caches[i], v_caches[i], heads, kv_heads, theta, eps)
    return x


def params_of(model) -> dict:
    """Float64 copies of a ``dynaflow_amd.decode.DecodeModel``'s parameters under the names used above."""
    p = {"embed": model.embed.detach().double().cpu()}
    for i, (a, m) in enumerate(zip(model.attn, model.mlp)):
        p[f"attn_norm.{i}"] = a.norm_weight.detach().double().cpu()
        p[f"wqkv.{i}"] = a.wqkv.detach().double().cpu()
        p[f"wo.{i}"] = a.wo.detach().double().cpu()
        p[f"mlp_norm.{i}"] = m.norm_weight.detach().double().cpu()
        p[f"w_gate.{i}"] = m.w_gate.detach().double().cpu()
        p[f"w_up.{i}"] = m.w_up.detach().double().cpu()
        p[f"w_down.{i}"] = m.w_down.detach().double().cpu()
    return p


def caches_of(model):
    """Natural-layout float64 copies ``[slots, capacity, kv_heads, d]`` of the model's caches."""
    ks, vs = [], []
    for a in model.attn:
        ks.append(a.k_cache.detach().double().cpu().permute(0, 2, 1, 3).contiguous())
        s, h, blocks, d, _ = a.v_cache.shape
        v = a.v_cache.detach().double().cpu().permute(0, 2, 4, 1, 3).reshape(s, blocks * 8, h, d)
        vs.append(v.contiguous())
    return ks, vs
