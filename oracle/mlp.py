"""The arithmetic of the path, restated with CPU PyTorch (and numpy for fp8).

The reference has no kernels of its own: its sub-graphs are executed by
PyTorch (dynaflow/runtime/engine.py:381), so "the reference DynaFlow schedule
run eagerly in PyTorch" is, per nano-batch b,

    x_b = x[split_indices[b] : split_indices[b+1]]           engine.py:466-470
    out_b = linear(silu(linear(x_b, Wg)) * linear(x_b, Wu), Wd)
    out   = cat(out_b, dim=0)                                manager.py:241-245

with weights in ``nn.Linear`` layout ([out, in]).  Functions:

  mlp_unsplit / mlp_schedule   the layer, whole and per nano-batch
  silu_mul_exact               one rounding, fp32 inside: the op written out in
                               examples/ae/up-silu-overlap.cu:75-90
  silu_mul_eager               what two bf16 aten ops give (silu rounded first)
  rms_norm                     examples/ae/scheduler/vllm/tokenweave-kernels/
                               csrc/tokenweave.cu:85-109 minus communication
  quant_e4m3 / dequant         per-tensor dynamic e4m3fn quantisation
  mlp_fp8_dequant_reference    fp32 matmuls on dequantised operands

PARITY UNPINNED against reference outputs (the reference ships none); pinned
instead by split == unsplit, a float64 closed form and oracle/mlp_ref.c.
"""
import numpy as np
import torch
import torch.nn.functional as F

FP8_MAX = 448.0


def make_inputs(tokens, hidden, inter, dtype=torch.float32, prenorm=False):
    """Seeded synthetic inputs: x ~ N(0,1) (seed 0), W_gate/W_up/W_down ~ N(0, 0.02)
    (seeds 1, 2, 3), generated in fp32 on the CPU and cast.  Weights are returned in
    ``linear`` layout [out, in]."""
    def normal(seed, shape, std):
        g = torch.Generator(device="cpu").manual_seed(seed)
        return torch.randn(shape, generator=g, dtype=torch.float32) * std

    x = normal(0, (tokens, hidden), 1.0)
    if prenorm:
        x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5)
    w_gate = normal(1, (inter, hidden), 0.02)
    w_up = normal(2, (inter, hidden), 0.02)
    w_down = normal(3, (hidden, inter), 0.02)
    return x.to(dtype), w_gate.to(dtype), w_up.to(dtype), w_down.to(dtype)


def mlp_unsplit(x, w_gate, w_up, w_down):
    return F.linear(F.silu(F.linear(x, w_gate)) * F.linear(x, w_up), w_down)


def mlp_schedule(x, w_gate, w_up, w_down, split_indices):
    parts = []
    for b in range(len(split_indices) - 1):
        xb = x[split_indices[b]:split_indices[b + 1]]
        parts.append(mlp_unsplit(xb, w_gate, w_up, w_down))
    return torch.cat(parts, dim=0)


def mlp_fp32_from(x, w_gate, w_up, w_down):
    """fp32 evaluation on the given (possibly bf16-valued) operands."""
    return mlp_unsplit(x.float(), w_gate.float(), w_up.float(), w_down.float())


def silu_mul_exact(gate, up):
    g = gate.float()
    return ((g / (1.0 + torch.exp(-g))) * up.float()).to(gate.dtype)


def silu_mul_eager(gate, up):
    return F.silu(gate) * up


def rms_norm(x, weight, eps, residual=None):
    h = x if residual is None else (x.float() + residual.float()).to(x.dtype)
    hf = h.float()
    inv = torch.rsqrt(hf.pow(2).sum(-1, keepdim=True) / hf.shape[-1] + eps)
    normed = (hf * inv).to(x.dtype)
    out = (normed.float() * weight.float()).to(x.dtype)
    return (out, h) if residual is not None else out


# ------------------------------------------------------------------ fp8 (e4m3fn)
def _e4m3_table():
    codes = np.arange(256, dtype=np.uint8)
    sign = np.where(codes & 0x80, -1.0, 1.0)
    exp = ((codes >> 3) & 0xF).astype(np.int32)
    man = (codes & 0x7).astype(np.float64)
    val = np.where(exp == 0, man / 8.0 * 2.0 ** -6, (1.0 + man / 8.0) * 2.0 ** (exp - 7.0))
    val = sign * val
    val[(codes & 0x7F) == 0x7F] = np.nan
    return val


E4M3_VALUES = _e4m3_table()


def e4m3_decode(codes):
    """uint8 codes -> float32 values (numpy), from the format definition."""
    return E4M3_VALUES[np.asarray(codes, dtype=np.uint8)].astype(np.float32)


def e4m3_encode(values):
    """float32 -> uint8 codes: round to nearest even, saturate at +-448 (numpy)."""
    v = np.clip(np.asarray(values, dtype=np.float64), -FP8_MAX, FP8_MAX)
    mag = np.abs(v)
    finite = E4M3_VALUES[:0x7F]  # non-negative codes 0 .. 0x7E, increasing
    idx = np.searchsorted(finite, mag, side="left")
    idx = np.clip(idx, 1, len(finite) - 1)
    lo, hi = finite[idx - 1], finite[idx]
    pick_hi = (mag - lo) > (hi - mag)
    tie = (mag - lo) == (hi - mag)
    code = np.where(pick_hi, idx, idx - 1)
    code = np.where(tie, np.where((idx % 2) == 0, idx, idx - 1), code)  # even mantissa code
    code = np.where(mag == 0, 0, code).astype(np.uint8)
    return np.where(np.signbit(v), code | 0x80, code).astype(np.uint8)


def quant_e4m3(x):
    """Per-tensor dynamic quantisation: returns (uint8 codes tensor, scale float32 tensor[1])."""
    xf = x.float()
    amax = xf.abs().max()
    scale = torch.clamp(amax, min=1e-12) / FP8_MAX
    scaled = (xf / scale).clamp(-FP8_MAX, FP8_MAX)
    codes = torch.from_numpy(e4m3_encode(scaled.numpy()))
    return codes, scale.reshape(1).float()


def quant_e4m3_per_channel(w):
    """Per-output-channel (row) quantisation of a [N, K] weight."""
    wf = w.float()
    amax = wf.abs().amax(dim=1)
    scale = torch.clamp(amax, min=1e-12) / FP8_MAX
    scaled = (wf / scale[:, None]).clamp(-FP8_MAX, FP8_MAX)
    codes = torch.from_numpy(e4m3_encode(scaled.numpy()))
    return codes, scale.float()


def dequant(codes, scale):
    vals = torch.from_numpy(e4m3_decode(codes.numpy()))
    if scale.numel() == 1:
        return vals * scale
    return vals * scale[:, None]


def mlp_fp8_dequant_reference(x_bf16, wg_q, wg_s, wu_q, wu_s, wd_q, wd_s, split_indices):
    """fp32 reference of the fp8 layer: every GEMM on dequantised operands,
    activations quantised per nano-batch, gate/up outputs rounded to bf16, the
    SiLU*mul product rounded to bf16 and re-quantised."""
    wg, wu, wd = dequant(wg_q, wg_s), dequant(wu_q, wu_s), dequant(wd_q, wd_s)
    parts = []
    for b in range(len(split_indices) - 1):
        xb = x_bf16[split_indices[b]:split_indices[b + 1]]
        xq, xs = quant_e4m3(xb)
        xd = dequant(xq, xs)
        g = (xd @ wg.t()).bfloat16()
        u = (xd @ wu.t()).bfloat16()
        act = silu_mul_exact(g, u)
        aq, a_s = quant_e4m3(act)
        parts.append((dequant(aq, a_s) @ wd.t()).bfloat16())
    return torch.cat(parts, dim=0)
