"""The runtime a model is loaded into: device, compute dtype, how matrices are
held, and the choice of kernel for each matrix product and attention call.

float32: every product runs in the general float32 kernel (fused multiply-add,
no matrix mode of reduced precision) and attention in the general kernel.
bfloat16: weights are held in the MFMA operand layout; products with at most
64 rows stream them once through the skinny MFMA kernel, larger ones run the
LDS-staged MFMA kernel; attention runs on the MFMA kernels where the shapes
allow, else in the general kernel.
"""

from __future__ import annotations

import torch

from ..kernels import ops


class LinearWeight:
    """A weight matrix [rows, cols] as the kernels want it."""

    __slots__ = ("rows", "cols", "dense", "tiled")

    def __init__(self, shape, dense: torch.Tensor | None, tiled: torch.Tensor | None):
        self.rows, self.cols = shape
        self.dense = dense  # row-major (float32 path)
        self.tiled = tiled  # MFMA operand layout (bfloat16 path)


class Runtime:
    def __init__(self, device="cuda:0", dtype=torch.bfloat16):
        self.device = torch.device(device)
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"compute dtype must be bfloat16 or float32, got {dtype}")
        self.dtype = dtype

    def weight(self, w: torch.Tensor) -> LinearWeight:
        """Takes a row-major [out, in] matrix in the compute dtype."""
        w = w.contiguous()
        if self.dtype == torch.bfloat16:
            return LinearWeight(w.shape, None, ops.retile_weight(w))
        return LinearWeight(w.shape, w, None)

    def gated_weight(self, gate: torch.Tensor, up: torch.Tensor):
        """The two matrices of a gated feed-forward, as `gated_linear` wants them."""
        if self.dtype == torch.bfloat16:
            tiled = ops.interleave_gate_up(gate.contiguous(), up.contiguous())
            return LinearWeight(gate.shape, None, tiled)
        return self.weight(torch.cat([gate, up], dim=0))

    def gated_linear(self, ctx, x, w: LinearWeight, out) -> None:
        """out = silu(x @ gate.T) * (x @ up.T).  bfloat16: one product whose
        epilogue applies the activation; float32: product, then activation."""
        if w.tiled is not None:
            ops.gemm_tiled_weight(x, w.tiled, w.rows, w.cols, out, gated=True)
            return
        gate_up = ctx.buffer("ffn_gate_up", (x.shape[0], w.rows), self.dtype)
        ops.gemm(x, w.dense, gate_up)
        ops.silu_mul(gate_up, out)

    def linear(self, x, w: LinearWeight, out, bias=None, accumulate=False) -> None:
        """out (+)= x @ w.T + bias."""
        if w.tiled is not None:
            ops.gemm_tiled_weight(x, w.tiled, w.rows, w.cols, out, bias=bias, accumulate=accumulate)
        else:
            ops.gemm(x, w.dense, out, bias=bias, accumulate=accumulate)

    def linear_deferred(self, ctx, name: str, x, w: LinearWeight, bias=None, reader="norm"):
        """x @ w.T + bias for a reader that can add up partial sums: a tensor
        [n, rows] in the compute dtype, or, where a matrix with few rows is split
        along k to fill the chip, the SplitSum of its parts.  reader "norm": the
        residual add of the next norm (no bias, width a multiple of 4 up to
        8192); reader "position": the position-encoding and cache-write kernel."""
        n = x.shape[0]
        splits = ops.gemm_splits(n, w.rows, w.cols) if w.tiled is not None else 1
        if reader == "norm" and (bias is not None or w.rows % 4 or w.rows > 8192):
            splits = 1
        if splits > 1:
            parts = ctx.buffer(name + "_parts", (splits, n, w.rows), torch.float32)
            ops.gemm_tiled_weight(x, w.tiled, w.rows, w.cols, parts, splits=splits)
            return ops.SplitSum(parts, bias)
        out = ctx.buffer(name, (n, w.rows), self.dtype)
        self.linear(x, w, out, bias=bias)
        return out

    def attend(self, ctx, qkv, out, spec, tables, cache) -> None:
        """Attention of every token of the step over its sequence's cache."""
        h, hkv, d = spec.num_heads, spec.num_kv_heads, spec.head_dim
        q = qkv[:, : h * d]
        if self.dtype == torch.bfloat16 and ops.attention_supports_mfma(
            h, hkv, d, cache.page_size, qkv.stride(0)
        ):
            if ctx.num_decode:
                nsplit = decode_splits(ctx.num_decode, hkv, ctx.max_decode_ctx)
                partial = ctx.buffer("attn_partial", (ctx.num_decode * h * nsplit * (d + 2),),
                                     torch.float32)
                ops.attention_decode(q, out, ctx.num_decode, h, hkv, d, ctx.positions, tables,
                                     cache.k_pool, cache.v_pool, cache.page_size, spec.window,
                                     spec.scale, partial, nsplit)
            tiles = ops.attention_prefill_shared_tiles(h, hkv, d) if ctx.num_prefill_tiles else 0
            if tiles:
                # few queries: smaller workgroups, so that there are enough for the chip
                small = -(-ctx.num_prefill_tiles // tiles) * hkv < PREFILL_MIN_WORKGROUPS
                if small and ops.attention_prefill_shared_tiles(h, hkv, d, small=True):
                    tiles = ops.attention_prefill_shared_tiles(h, hkv, d, small=True)
                else:
                    small = False
                wg_seq, wg_q0, count = ctx.prefill_workgroups(tiles)
                ops.attention_prefill_shared(q, out, count, h, hkv, d, ctx.cu_q, ctx.ctx_lens, wg_seq,
                                             wg_q0, tables, cache.k_pool, cache.v_pool,
                                             cache.page_size, spec.window, spec.scale, small=small)
            elif ctx.num_prefill_tiles:
                ops.attention_prefill(q, out, ctx.num_prefill_tiles, h, hkv, d, ctx.cu_q,
                                      ctx.ctx_lens, ctx.tile_seq, ctx.tile_q0, tables, cache.k_pool,
                                      cache.v_pool, cache.page_size, spec.window, spec.scale)
            return
        ops.attention(q, out, h, hkv, d, ctx.positions, ctx.token_seq, tables, cache.k_pool,
                      cache.v_pool, cache.page_size, spec.window, spec.scale)


# portions whose 16-wavefront workgroups would number fewer than this take 8-wavefront ones
PREFILL_MIN_WORKGROUPS = 192


def bucket(n: int, floor: int = 1) -> int:
    """The power of two (at least `floor`) that n rounds up to."""
    b = floor
    while b < n:
        b *= 2
    return b


def decode_splits(num_seqs: int, kv_heads: int, max_ctx: int) -> int:
    """Workgroups per (sequence, key/value head) of decode attention: enough to
    put one on every compute unit (256), each with at least 256 keys for its
    four wavefronts.  Both inputs are rounded up to powers of two first, so a
    step gives the same result whether it runs kernel by kernel or as a graph
    captured for its bucket."""
    want = -(-256 // (bucket(num_seqs) * kv_heads))
    most = max(1, bucket(max_ctx, 256) // 256)
    return max(1, min(want, most, 64))
