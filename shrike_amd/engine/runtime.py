"""The runtime a model is loaded into: device, compute dtype, how matrices are
held, and the choice of kernel for each matrix product.

float32: every product runs in the general float32 kernel (fused multiply-add,
no matrix mode of reduced precision).  bfloat16: weights are held in the MFMA
operand layout; products with at most 64 rows stream them once through the
skinny MFMA kernel, larger ones run the LDS-staged MFMA kernel.  What a mixer
does between its products is the mixer's own business.
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

    def gated_linear(self, ctx, x, w: LinearWeight, out, activation: str = "silu") -> None:
        """out = act(x @ gate.T) * (x @ up.T), act "silu" or "gelu_tanh".  bfloat16: one
        product whose epilogue applies the activation; float32: product, then activation."""
        if w.tiled is not None:
            ops.gemm_tiled_weight(x, w.tiled, w.rows, w.cols, out, gated=activation)
            return
        gate_up = ctx.buffer("ffn_gate_up", (x.shape[0], w.rows), self.dtype)
        ops.gemm(x, w.dense, gate_up)
        ops.act_mul(gate_up, out, activation)

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
