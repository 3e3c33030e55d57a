"""The model as the engine runs it: embedding, a schedule of blocks, final
norm, output matrix.  It is built from a ModelSpec alone."""

from __future__ import annotations

import torch

from ..config.specs import ModelSpec
from ..kernels import ops
from ..parts.base import HiddenState, ParamSpec, build_part


class DecoderModel:
    """Reference: shrike/models/qwen.py:153-192 (embedding, layers, final norm,
    selection of the wanted rows before the output matrix)."""

    def __init__(self, spec: ModelSpec):
        self.spec = spec
        h = spec.hidden_size
        self.blocks = [build_part("block", b, h, b.name) for b in spec.blocks]
        self.final_norm = build_part("norm", spec.final_norm, h, spec.final_norm_name)
        self.embed_name = f"{spec.embed_name}.weight"
        self.head_name = f"{spec.head_name}.weight"

    # ------------------------------------------------------------------ weights

    def params(self) -> list[ParamSpec]:
        s = self.spec
        out = [ParamSpec(self.embed_name, (s.vocab_size, s.hidden_size))]
        for block in self.blocks:
            out += block.params()
        out += self.final_norm.params()
        # With tied weights a file may still carry the output matrix; without, it must.
        out.append(
            ParamSpec(self.head_name, (s.vocab_size, s.hidden_size), optional=s.tie_word_embeddings)
        )
        return out

    def graph_safe(self) -> bool:
        """Whether a decode step of this model may be recorded into a HIP graph."""
        return all(block.graph_safe for block in self.blocks)

    def cache_specs(self) -> list:
        """Cache need of every schedule position (None for a position that
        reads another position's cache or whose mixer keeps nothing)."""
        out = []
        for entry in self.spec.schedule:
            mixer = self.blocks[entry.block].mixer
            out.append(None if entry.cache_of is not None else mixer.cache_spec())
        return out

    def load(self, tensors: dict[str, torch.Tensor], runtime) -> None:
        for block in self.blocks:
            block.check(runtime)
            block.load(tensors, runtime)
        self.final_norm.load(tensors, runtime)
        self.embed = tensors[self.embed_name]
        head = tensors.get(self.head_name)
        # shrike/models/qwen.py:211-212: tied and absent -> the embedding table itself
        self.head = runtime.weight(self.embed if head is None else head)
        self.linear = runtime.linear

    # ------------------------------------------------------------------ forward

    def forward(self, ctx, caches) -> torch.Tensor:
        """Logits float32 [R, vocab] at ctx.out_rows.  `caches[i]` is the
        LayerCache of schedule position i."""
        s = self.spec
        resid = ctx.buffer("resid", (ctx.num_tokens, s.hidden_size), torch.float32)
        ops.embed(self.embed, ctx.token_ids, resid)
        hidden = HiddenState(resid)
        for pos, entry in enumerate(s.schedule):
            self.blocks[entry.block].forward(ctx, hidden, caches[pos])
        rows = ctx.out_rows
        logits = ctx.buffer("logits", (rows.shape[0], s.vocab_size), torch.float32)
        if rows.shape[0]:
            x = self.final_norm.forward(ctx, hidden, rows=rows, write_resid=False)
            self.linear(x, self.head, logits)
        return logits
