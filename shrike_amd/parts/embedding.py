"""Token embedding: the residual stream starts as the table's rows."""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Embedding, ParamSpec, register_embedding


class TokenEmbedding(Embedding):
    """x[n] = table[token_ids[n]], widened to float32, without any scaling
    (reference: shrike/models/qwen.py:156,161)."""

    launches_follow_shape = True

    def params(self):
        return [ParamSpec(f"{self.name}.weight", (self.spec.vocab_size, self.width), init="embedding")]

    def load(self, tensors, runtime):
        self.table = tensors[f"{self.name}.weight"]

    def forward(self, ctx) -> torch.Tensor:
        resid = ctx.buffer("resid", (ctx.num_tokens, self.width), torch.float32)
        ops.embed(self.table, ctx.token_ids, resid)
        return resid


register_embedding("token_lookup", TokenEmbedding)
