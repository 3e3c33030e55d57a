"""Dense gated feed-forward (SwiGLU, or its sibling with a GELU gate)."""

from __future__ import annotations

import torch

from .base import FeedForward, ParamSpec, register_ffn


class SwiGLU(FeedForward):
    """down(act(gate(x)) * up(x)) without biases; act is the spec's activation,
    SiLU for the reference's model (shrike/models/qwen.py:131-136).  gate and up
    are joined into one weight at load time, so that one product yields the
    activated values."""

    launches_follow_shape = True

    def params(self):
        inter, h = self.spec.intermediate_size, self.width
        return [
            ParamSpec(f"{self.name}.gate_proj.weight", (inter, h)),
            ParamSpec(f"{self.name}.up_proj.weight", (inter, h)),
            ParamSpec(f"{self.name}.down_proj.weight", (h, inter)),
        ]

    def check(self, runtime):
        from ..kernels import ops

        ops.activation_code(self.spec.activation)  # raises for an activation the kernels lack

    def load(self, tensors, runtime):
        self.inter = int(self.spec.intermediate_size)
        self.activation = self.spec.activation
        self.w_gate_up = runtime.gated_weight(
            tensors[f"{self.name}.gate_proj.weight"], tensors[f"{self.name}.up_proj.weight"]
        )
        self.w_down = runtime.weight(tensors[f"{self.name}.down_proj.weight"])
        self.linear_deferred = runtime.linear_deferred
        self.gated_linear = runtime.gated_linear

    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        n = x.shape[0]
        act = ctx.buffer("ffn_act", (n, self.inter), ctx.dtype)
        self.gated_linear(ctx, x, self.w_gate_up, act, self.activation)
        # the norm that follows adds the output to the residual stream and can add up parts
        return self.linear_deferred(ctx, "ffn_out", act, self.w_down)


register_ffn("swiglu", SwiGLU)
