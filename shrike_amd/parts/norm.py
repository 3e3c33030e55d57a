"""RMSNorm fused with the residual add that precedes it."""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import HiddenState, Norm, ParamSpec, register_norm


class RMSNorm(Norm):
    """y = x * rsqrt(mean(x^2) + eps) * weight in float32, one cast at the end
    (reference: shrike/models/qwen.py:70-74)."""

    launches_follow_shape = True

    def params(self):
        return [ParamSpec(f"{self.name}.weight", (self.width,), init="norm", keep_float32=True)]

    def load(self, tensors, runtime):
        self.weight = tensors[f"{self.name}.weight"]
        self.eps = float(self.spec.eps)

    def forward(self, ctx, hidden: HiddenState, rows=None, write_resid=True) -> torch.Tensor:
        n = hidden.resid.shape[0] if rows is None else rows.shape[0]
        out = ctx.buffer(f"normed", (n, self.width), ctx.dtype)
        ops.add_rmsnorm(hidden.resid, hidden.pending, self.weight, self.eps, out, rows, write_resid)
        if write_resid:
            hidden.pending = None
        return out


register_norm("rmsnorm", RMSNorm)
