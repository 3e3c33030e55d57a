"""The model as the engine runs it: embedding, a schedule of blocks, final
norm, head.  It is built from a ModelSpec alone; every stage is a part chosen
by the spec."""

from __future__ import annotations

import torch

from ..config.specs import ModelSpec
from ..parts.base import HiddenState, ParamSpec, Part, StateSpec, build_part


class DecoderModel:
    """Reference: shrike/models/qwen.py:153-192 (embedding, layers, final norm,
    selection of the wanted rows before the output matrix)."""

    def __init__(self, spec: ModelSpec):
        self.spec = spec
        h = spec.hidden_size
        self.embedding = build_part("embedding", spec.embedding, h, spec.embed_name)
        self.blocks = [build_part("block", b, h, b.name) for b in spec.blocks]
        self.final_norm = build_part("norm", spec.final_norm, h, spec.final_norm_name)
        self.head = build_part("head", spec.head, h, spec.head_name)
        if spec.tie_word_embeddings:
            self.head.tie(self.embedding)
        # the parts whose prepare() does something, in the order they run
        self._preparers = [p for p in self.parts() if type(p).prepare is not Part.prepare]

    def parts(self) -> list[Part]:
        """Every part of the model, blocks' own parts included, in running order."""
        out: list[Part] = [self.embedding]
        for block in self.blocks:
            out.append(block)
            out += list(getattr(block, "parts", ()))
        return out + [self.final_norm, self.head]

    # ------------------------------------------------------------------ weights

    def params(self) -> list[ParamSpec]:
        out = list(self.embedding.params())
        for block in self.blocks:
            out += block.params()
        return out + self.final_norm.params() + self.head.params()

    def graph_safe(self) -> bool:
        """Whether a decode step of this model may be recorded into a HIP graph:
        every part says so, and a mixer with state of its own says that it
        reaches that state through the device-side slot indices."""
        for part in self.parts():
            if not part.graph_safe:
                return False
        for block in self.blocks:
            mixer = block.mixer
            if isinstance(mixer.cache_spec(), StateSpec) and not mixer.state_graph_safe:
                return False
        return True

    def launches_follow_shape(self) -> bool:
        """Whether every part says that its launches follow from a step's shape and
        launch key alone: the forward of such a model can be run again from a recorded
        list of launches for any later step of the same shape."""
        return all(part.launches_follow_shape for part in self.parts())

    def cache_specs(self) -> list:
        """Cache need of every schedule position (None for a position that
        reads another position's cache or whose mixer keeps nothing)."""
        out = []
        for entry in self.spec.schedule:
            mixer = self.blocks[entry.block].mixer
            out.append(None if entry.cache_of is not None else mixer.cache_spec())
        return out

    def load(self, tensors: dict[str, torch.Tensor], runtime) -> None:
        self.embedding.check(runtime)
        self.embedding.load(tensors, runtime)
        for block in self.blocks:
            block.check(runtime)
            block.load(tensors, runtime)
        self.final_norm.load(tensors, runtime)
        self.head.check(runtime)
        self.head.load(tensors, runtime)

    # ------------------------------------------------------------------ forward

    def prepare(self, shape) -> None:
        """Lets every part that wants to decide its launches for the step and add
        its index arrays to the step's metadata."""
        for part in self._preparers:
            part.prepare(shape)

    def forward(self, ctx, caches) -> torch.Tensor:
        """Logits float32 [R, vocab] at ctx.out_rows.  `caches[i]` is the
        LayerCache of schedule position i."""
        hidden = HiddenState(self.embedding.forward(ctx))
        for pos, entry in enumerate(self.spec.schedule):
            self.blocks[entry.block].forward(ctx, hidden, caches[pos])
        rows = ctx.out_rows
        if rows.shape[0] == 0:
            return ctx.buffer("logits", (0, self.spec.vocab_size), torch.float32)
        x = self.final_norm.forward(ctx, hidden, rows=rows, write_resid=False)
        return self.head.forward(ctx, x)
