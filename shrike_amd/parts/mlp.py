"""Dense SwiGLU feed-forward."""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import FeedForward, ParamSpec, register_ffn


class SwiGLU(FeedForward):
    """down(silu(gate(x)) * up(x)) without biases (reference:
    shrike/models/qwen.py:131-136).  gate and up are stacked into one [2I, h]
    matrix at load time so that one product feeds the activation kernel."""

    def params(self):
        inter, h = self.spec.intermediate_size, self.width
        return [
            ParamSpec(f"{self.name}.gate_proj.weight", (inter, h)),
            ParamSpec(f"{self.name}.up_proj.weight", (inter, h)),
            ParamSpec(f"{self.name}.down_proj.weight", (h, inter)),
        ]

    def load(self, tensors, runtime):
        self.inter = int(self.spec.intermediate_size)
        self.w_gate_up = runtime.weight(torch.cat(
            [tensors[f"{self.name}.gate_proj.weight"], tensors[f"{self.name}.up_proj.weight"]], dim=0
        ))
        self.w_down = runtime.weight(tensors[f"{self.name}.down_proj.weight"])
        self.linear = runtime.linear

    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        n = x.shape[0]
        gate_up = ctx.buffer("ffn_gate_up", (n, 2 * self.inter), ctx.dtype)
        self.linear(x, self.w_gate_up, gate_up)
        act = ctx.buffer("ffn_act", (n, self.inter), ctx.dtype)
        ops.silu_mul(gate_up, act)
        out = ctx.buffer("ffn_out", (n, self.width), ctx.dtype)
        self.linear(act, self.w_down, out)
        return out


register_ffn("swiglu", SwiGLU)
