"""Output matrix: logits of the wanted rows."""

from __future__ import annotations

import torch

from .base import Head, ParamSpec, register_head


class LinearHead(Head):
    """logits = x @ W.T without bias, float32 out (reference:
    shrike/models/qwen.py:178,192).  When the model ties its weights and the
    file carries no output matrix, W is the embedding table itself
    (qwen.py:211-212)."""

    launches_follow_shape = True

    def __init__(self, spec, width, name):
        super().__init__(spec, width, name)
        self.tied_to = None

    def tie(self, embedding) -> None:
        self.tied_to = embedding

    def params(self):
        # With tied weights a file may still carry the output matrix; without, it must.
        return [ParamSpec(f"{self.name}.weight", (self.spec.vocab_size, self.width),
                          optional=self.tied_to is not None)]

    def load(self, tensors, runtime):
        w = tensors.get(f"{self.name}.weight")
        if w is None:
            if self.tied_to is None or self.tied_to.table is None:
                raise KeyError(f"{self.name}.weight is absent and the model does not tie its weights")
            w = self.tied_to.table
        self.weight = runtime.weight(w)
        self.linear = runtime.linear

    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        logits = ctx.buffer("logits", (x.shape[0], self.spec.vocab_size), torch.float32)
        if x.shape[0]:
            self.linear(x, self.weight, logits)
        return logits


register_head("linear", LinearHead)
