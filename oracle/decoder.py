"""Independent CPU restatement of the decoder layer of the attention-beside-MLP configuration.

TEST INFRASTRUCTURE.  The reference has no model code of its own (models come from the host
framework, e.g. HF Llama through examples/ae/scripts/bench_hf_transformers.py:202-210), so this
restates the textbook definitions the north star names: RMSNorm (eps 1e-5), rotary embedding with
theta 500000 in the half-split convention, causal grouped-query attention with 1/sqrt(d) scaling,
SwiGLU MLP, residual connections.  Written with explicit loops over heads and an explicit mask so
that it shares nothing with the product module (no fused attention call, complex-number rotation).
Pinned by: softmax rows sum to 1, causality (changing a later token leaves earlier outputs
unchanged), rotation preserves norms and relative-position dot products, agreement with the product
module on the CPU in float64.  PARITY UNPINNED against reference outputs (there are none).
"""
import math

import torch


def rms_norm(x, w, eps):
    xf = x.double()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)) * w.double()


def rope(t, theta):
    """t: [B, S, heads, d] -> rotated, using complex multiplication on (t[i], t[i + d/2]) pairs."""
    B, S, Hn, d = t.shape
    half = d // 2
    freqs = 1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float64) / d))
    ang = torch.arange(S, dtype=torch.float64)[:, None] * freqs[None, :]
    rot = torch.polar(torch.ones_like(ang), ang)                       # e^{i pos freq}
    z = torch.complex(t.double()[..., :half], t.double()[..., half:]) * rot[None, :, None, :]
    return torch.cat((z.real, z.imag), dim=-1)


def attention(q, k, v):
    """q [B,S,Hq,d], k/v [B,S,Hkv,d] (float64) -> [B,S,Hq,d]; causal, grouped queries."""
    B, S, Hq, d = q.shape
    group = Hq // k.shape[2]
    out = torch.empty_like(q)
    mask = torch.ones(S, S, dtype=torch.bool).tril()
    for b in range(B):
        for h in range(Hq):
            kv = h // group
            scores = (q[b, :, h, :] @ k[b, :, kv, :].t()) / math.sqrt(d)
            scores = scores.masked_fill(~mask, float("-inf"))
            p = torch.softmax(scores, dim=-1)
            out[b, :, h, :] = p @ v[b, :, kv, :]
    return out


def decoder_layer(token_ids, params, seq_len, heads, kv_heads, head_dim, theta=500000.0, eps=1e-5):
    """params: dict of float tensors (embed, attn_norm, wq, wk, wv, wo, mlp_norm, w_gate, w_up, w_down)."""
    P = {k: v.double() for k, v in params.items()}
    x = P["embed"][token_ids]
    h = rms_norm(x, P["attn_norm"], eps)
    B = x.shape[0] // seq_len
    q = (h @ P["wq"].t()).view(B, seq_len, heads, head_dim)
    k = (h @ P["wk"].t()).view(B, seq_len, kv_heads, head_dim)
    v = (h @ P["wv"].t()).view(B, seq_len, kv_heads, head_dim)
    a = attention(rope(q, theta), rope(k, theta), v).reshape(x.shape[0], heads * head_dim)
    x = x + a @ P["wo"].t()
    h = rms_norm(x, P["mlp_norm"], eps)
    g = h @ P["w_gate"].t()
    return x + ((g / (1 + torch.exp(-g))) * (h @ P["w_up"].t())) @ P["w_down"].t()


def decoder_layer_rows(token_ids, params, rows, seq_len, heads, kv_heads, head_dim, theta=500000.0, eps=1e-5):
    """decoder_layer(...)[rows] computed without the other rows' share of the work, for sizes where the
    whole layer takes too long on the CPU: keys and values are needed for every token of a sampled row's
    sequence (up to the row), queries, the output projection and the MLP only for the sampled rows.
    Written as one loop over the sampled rows; pinned by equality with decoder_layer on small layers."""
    P = {k: v.double() for k, v in params.items() if k != "embed"}   # the embedding is gathered first: it is large
    group = heads // kv_heads
    half = head_dim // 2
    freqs = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))
    out = []
    for r in [int(r) for r in rows]:
        start, pos = (r // seq_len) * seq_len, r % seq_len
        x = params["embed"][token_ids[start:start + pos + 1]].double()   # the sequence up to and including the row
        h = rms_norm(x, P["attn_norm"], eps)
        ang = torch.arange(pos + 1, dtype=torch.float64)[:, None] * freqs[None, :]
        rot = torch.polar(torch.ones_like(ang), ang)

        def rotated(t, n):
            t = t.view(-1, n, head_dim)
            z = torch.complex(t[..., :half], t[..., half:]) * rot[-t.shape[0]:, None, :]
            return torch.cat((z.real, z.imag), dim=-1)

        q = rotated(h[-1:] @ P["wq"].t(), heads)[0]                  # [heads, d], position pos
        k = rotated(h @ P["wk"].t(), kv_heads)                       # [pos+1, kv_heads, d]
        v = (h @ P["wv"].t()).view(-1, kv_heads, head_dim)
        a = torch.empty(heads, head_dim, dtype=torch.float64)
        for hd in range(heads):
            kv = hd // group
            p = torch.softmax((k[:, kv, :] @ q[hd]) / math.sqrt(head_dim), dim=0)
            a[hd] = p @ v[:, kv, :]
        y = x[-1] + a.reshape(-1) @ P["wo"].t()
        hm = rms_norm(y, P["mlp_norm"], eps)
        g = hm @ P["w_gate"].t()
        out.append(y + ((g / (1 + torch.exp(-g))) * (hm @ P["w_up"].t())) @ P["w_down"].t())
    return torch.stack(out)


def params_of(layer):
    """Collect the parameters of a dynaflow_amd.decoder.DecoderLayer under the names used above."""
    return {
        "embed": layer.embed.detach().cpu(), "attn_norm": layer.attn.norm_weight.detach().cpu(),
        "wq": layer.attn.wq.detach().cpu(), "wk": layer.attn.wk.detach().cpu(), "wv": layer.attn.wv.detach().cpu(),
        "wo": layer.attn.wo.detach().cpu(), "mlp_norm": layer.mlp.norm_weight.detach().cpu(),
        "w_gate": layer.mlp.w_gate.detach().cpu(), "w_up": layer.mlp.w_up.detach().cpu(),
        "w_down": layer.mlp.w_down.detach().cpu(),
    }
