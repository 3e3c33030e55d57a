"""Dense SwiGLU feed-forward."""

from __future__ import annotations

import torch

from .base import FeedForward, ParamSpec, register_ffn


class SwiGLU(FeedForward):
    """down(silu(gate(x)) * up(x)) without biases (reference:
    shrike/models/qwen.py:131-136).  gate and up are joined into one weight at
    load time, so that one product yields the activated values."""

    def params(self):
        inter, h = self.spec.intermediate_size, self.width
        return [
            ParamSpec(f"{self.name}.gate_proj.weight", (inter, h)),
            ParamSpec(f"{self.name}.up_proj.weight", (inter, h)),
            ParamSpec(f"{self.name}.down_proj.weight", (h, inter)),
        ]

    def load(self, tensors, runtime):
        self.inter = int(self.spec.intermediate_size)
        self.w_gate_up = runtime.gated_weight(
            tensors[f"{self.name}.gate_proj.weight"], tensors[f"{self.name}.up_proj.weight"]
        )
        self.w_down = runtime.weight(tensors[f"{self.name}.down_proj.weight"])
        self.linear_deferred = runtime.linear_deferred
        self.gated_linear = runtime.gated_linear

    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        n = x.shape[0]
        act = ctx.buffer("ffn_act", (n, self.inter), ctx.dtype)
        self.gated_linear(ctx, x, self.w_gate_up, act)
        # the norm that follows adds the output to the residual stream and can add up parts
        return self.linear_deferred(ctx, "ffn_out", act, self.w_down)


register_ffn("swiglu", SwiGLU)
