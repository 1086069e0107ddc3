"""The SwiGLU MLP block of the hot path as a plain ``nn.Module``.

``y = down(silu(gate(x)) * up(x))`` with bias-free ``nn.Linear`` projections,
written so that dynamo traces both projections before the activation
(``linear, linear_1, silu, mul, linear_2``); the split rule of
``MLPOverlapScheduler`` then yields the two sub-graphs {gate, up} and
{silu, mul, down}.

In the reference this block is host-model code (the MLP of the HF Llama that
examples/ae/scripts/bench_hf_transformers.py:206-210 loads, whose projections
examples/ae/scheduler/hf/nanoflow.py:30 names); its stand-alone experiment on
the same shapes is examples/ae/up-silu-overlap.cu:266-342.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F


class SwiGLUMLP(nn.Module):
    def __init__(self, hidden_size: int, intermediate_size: int, dtype=torch.bfloat16, device=None) -> None:
        super().__init__()
        kw = dict(bias=False, dtype=dtype, device=device)
        self.gate_proj = nn.Linear(hidden_size, intermediate_size, **kw)
        self.up_proj = nn.Linear(hidden_size, intermediate_size, **kw)
        self.down_proj = nn.Linear(intermediate_size, hidden_size, **kw)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        g = self.gate_proj(x)
        u = self.up_proj(x)
        return self.down_proj(F.silu(g) * u)

    @torch.no_grad()
    def load_x_at_w(self, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> None:
        """Load weights given in the ``out = x @ W`` convention ([in, out])."""
        self.gate_proj.weight.copy_(w_gate.t())
        self.up_proj.weight.copy_(w_up.t())
        self.down_proj.weight.copy_(w_down.t())
