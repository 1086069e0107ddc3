"""fp8 (e4m3fn) SwiGLU MLP block built on the HIP operators.

Activations are quantised per tensor with a dynamic scale (computed inside the
graph, hence per nano-batch once the graph is split), weights per output channel
once at construction.  Every GEMM multiplies e4m3 operands with fp32
accumulation and writes bf16; SiLU*mul is computed in fp32 from the bf16 gate/up
outputs, rounded to bf16 and re-quantised for the down projection.

Traced by dynamo the forward is
``quant_fp8, getitem x2, linear_fp8, linear_fp8, silu_mul_quant_fp8, getitem x2,
linear_fp8``; ``MLPOverlapScheduler`` cuts it in front of ``silu_mul_quant_fp8``.  With ``fuse_gate_up`` the two
projections and the SiLU*mul are one operator (``gate_up_silu_quant_fp8``) and the cut (knob
``fuse_silu_epilogue``) is in front of the down projection.

The reference ships no fp8 model code; this block stands for the quantised MLP of a host
framework, scheduled through the same interface (dynaflow/interface.py) as the bf16 one.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from dynaflow_amd import ops

FP8_MAX = 448.0


def quantize_weight_per_channel(w: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """[N, K] weight -> (e4m3fn codes [N, K], fp32 scale [N]); one-time set-up on the device."""
    wf = w.float()
    scale = wf.abs().amax(dim=1).clamp_min(1e-12) / FP8_MAX
    q = (wf / scale[:, None]).clamp(-FP8_MAX, FP8_MAX).to(ops.FP8_DTYPE)
    return q.contiguous(), scale.contiguous()


class Fp8SwiGLU(nn.Module):
    def __init__(self, w_gate_q, w_gate_s, w_up_q, w_up_s, w_down_q, w_down_s, fuse_gate_up: bool = False) -> None:
        super().__init__()
        #: gate and up projection with the SiLU*mul as ONE GEMM's epilogue (same bits as the separate operators)
        self.fuse_gate_up = fuse_gate_up
        for name, value in (("w_gate_q", w_gate_q), ("w_gate_s", w_gate_s), ("w_up_q", w_up_q),
                            ("w_up_s", w_up_s), ("w_down_q", w_down_q), ("w_down_s", w_down_s)):
            self.register_buffer(name, value)

    @classmethod
    def from_weights(cls, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor,
                     fuse_gate_up: bool = False) -> "Fp8SwiGLU":
        """Weights in ``linear`` layout ([out, in]), any float dtype, on the GPU."""
        return cls(*quantize_weight_per_channel(w_gate), *quantize_weight_per_channel(w_up),
                   *quantize_weight_per_channel(w_down), fuse_gate_up=fuse_gate_up)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        xq, xs = ops.quant_fp8(x)
        if self.fuse_gate_up:
            aq, a_s = ops.gate_up_silu_quant_fp8(xq, self.w_gate_q, self.w_up_q, xs, self.w_gate_s, self.w_up_s)
            return ops.linear_fp8(aq, self.w_down_q, a_s, self.w_down_s)
        g = ops.linear_fp8(xq, self.w_gate_q, xs, self.w_gate_s)
        u = ops.linear_fp8(xq, self.w_up_q, xs, self.w_up_s)
        aq, a_s = ops.silu_mul_quant_fp8(g, u)
        return ops.linear_fp8(aq, self.w_down_q, a_s, self.w_down_s)

    def forward_schedule(self, x: torch.Tensor, split_indices: list[int]) -> torch.Tensor:
        """The split schedule issued directly, one nano-batch after the other."""
        parts = [self.forward(x[split_indices[b]:split_indices[b + 1]]) for b in range(len(split_indices) - 1)]
        return torch.cat(parts, dim=0)
