"""Causal grouped-query attention over the paged key/value cache."""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Mixer, PagedKVSpec, ParamSpec, build_part, register_mixer


class PagedAttention(Mixer):
    """q/k/v projections (with or without bias), position encoding of q and k,
    cache write, attention over the sequence's pages, output projection
    (reference: shrike/models/qwen.py:111-125, shrike/engine/model_runner.py:63-151).

    The three projections are stacked into one [(H + 2 Hkv) D, h] matrix at
    load time; head j of q is rows j*D..(j+1)*D-1 of the q part, as in the
    reference's view (qwen.py:120-122).
    """

    def __init__(self, spec, width, name):
        super().__init__(spec, width, name)
        self.position = (
            build_part("position", spec.position, width, name) if spec.position is not None else None
        )

    def params(self):
        s, h = self.spec, self.width
        q, kv = s.num_heads * s.head_dim, s.num_kv_heads * s.head_dim
        out = [
            ParamSpec(f"{self.name}.q_proj.weight", (q, h)),
            ParamSpec(f"{self.name}.k_proj.weight", (kv, h)),
            ParamSpec(f"{self.name}.v_proj.weight", (kv, h)),
            ParamSpec(f"{self.name}.o_proj.weight", (h, q)),
        ]
        if s.qkv_bias:
            out += [
                ParamSpec(f"{self.name}.q_proj.bias", (q,), init="bias", keep_float32=True),
                ParamSpec(f"{self.name}.k_proj.bias", (kv,), init="bias", keep_float32=True),
                ParamSpec(f"{self.name}.v_proj.bias", (kv,), init="bias", keep_float32=True),
            ]
        if s.out_bias:
            out.append(ParamSpec(f"{self.name}.o_proj.bias", (h,), init="bias", keep_float32=True))
        return out

    def cache_spec(self):
        s = self.spec
        return PagedKVSpec(s.num_kv_heads, s.head_dim, s.window)

    def check(self, runtime):
        s = self.spec
        if s.num_heads % s.num_kv_heads:
            raise ValueError(
                f"{self.name}: {s.num_heads} query heads are not a multiple of "
                f"{s.num_kv_heads} key/value heads"
            )
        if not 1 <= s.head_dim <= 256:
            raise ValueError(f"{self.name}: head_dim {s.head_dim} is outside 1..256")
        if s.window is not None and s.window < 1:
            raise ValueError(f"{self.name}: window must be positive, got {s.window}")

    def load(self, tensors, runtime):
        s, n = self.spec, self.name
        self.w_qkv = runtime.weight(torch.cat(
            [tensors[f"{n}.q_proj.weight"], tensors[f"{n}.k_proj.weight"], tensors[f"{n}.v_proj.weight"]],
            dim=0,
        ))
        self.b_qkv = (
            torch.cat([tensors[f"{n}.q_proj.bias"], tensors[f"{n}.k_proj.bias"], tensors[f"{n}.v_proj.bias"]])
            .contiguous()
            if s.qkv_bias
            else None
        )
        self.w_o = runtime.weight(tensors[f"{n}.o_proj.weight"])
        self.b_o = tensors[f"{n}.o_proj.bias"] if s.out_bias else None
        if self.position is not None:
            self.position.load(tensors, runtime)
        self.linear = runtime.linear
        self.linear_deferred = runtime.linear_deferred
        self.attend = runtime.attend

    def forward(self, ctx, x: torch.Tensor, cache) -> torch.Tensor:
        s = self.spec
        n = x.shape[0]
        qkv_width = (s.num_heads + 2 * s.num_kv_heads) * s.head_dim
        table = self.position.rotary_table() if self.position is not None else None
        fused_position = self.position is None or table is not None
        split_sum = None
        if fused_position:
            # the cache-write kernel can take the projections as partial sums
            qkv = self.linear_deferred(ctx, "attn_qkv_sum", x, self.w_qkv, bias=self.b_qkv,
                                       reader="position")
            if isinstance(qkv, ops.SplitSum):
                split_sum, qkv = qkv, ctx.buffer("attn_qkv", (n, qkv_width), ctx.dtype)
        else:
            qkv = ctx.buffer("attn_qkv", (n, qkv_width), ctx.dtype)
            self.linear(x, self.w_qkv, qkv, bias=self.b_qkv)
            self.position.apply(ctx, qkv, s.num_heads, s.num_kv_heads, s.head_dim)
        inv_freq, rot_dim = table if table is not None else (None, 0)
        tables = ctx.block_tables[cache.group]
        ops.rope_kv_store(
            qkv, s.num_heads, s.num_kv_heads, s.head_dim, rot_dim, inv_freq, ctx.positions,
            ctx.token_seq, tables, cache.k_pool, cache.v_pool, cache.page_size,
            write_kv=cache.owned, split_sum=split_sum,
        )
        attn = ctx.buffer("attn_out", (n, s.num_heads * s.head_dim), ctx.dtype)
        self.attend(ctx, qkv, attn, s, tables, cache)
        # the norm that follows adds the output to the residual stream and can add up parts
        return self.linear_deferred(ctx, "attn_proj", attn, self.w_o, bias=self.b_o)


register_mixer("paged_attention", PagedAttention)
