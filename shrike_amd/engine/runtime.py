"""The runtime a model is loaded into: device, compute dtype, and the choice
of kernel for each matrix product and attention call.

float32: every product runs in the general float32 kernel (fused multiply-add,
no matrix mode of reduced precision) and attention in the general kernel.
bfloat16: the serving kernels.
"""

from __future__ import annotations

import torch

from ..kernels import ops


class Runtime:
    def __init__(self, device="cuda:0", dtype=torch.bfloat16):
        self.device = torch.device(device)
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"compute dtype must be bfloat16 or float32, got {dtype}")
        self.dtype = dtype

    def linear(self, x, w, out, bias=None, accumulate=False) -> None:
        """out (+)= x @ w.T + bias."""
        ops.gemm(x, w, out, bias=bias, accumulate=accumulate)

    def attend(self, ctx, qkv, out, spec, tables, cache) -> None:
        """Attention of every token of the step over its sequence's cache."""
        q = qkv[:, : spec.num_heads * spec.head_dim]
        ops.attention(
            q, out, spec.num_heads, spec.num_kv_heads, spec.head_dim, ctx.positions,
            ctx.token_seq, tables, cache.k_pool, cache.v_pool, cache.page_size,
            spec.window, spec.scale,
        )
