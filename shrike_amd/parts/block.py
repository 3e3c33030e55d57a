"""Pre-norm residual block: x += mixer(norm(x)); x += ffn(norm(x))."""

from __future__ import annotations

from .base import Block, HiddenState, build_part, register_block


class PreNormResidualBlock(Block):
    """Reference: shrike/models/qwen.py:147-150.  The additions are not done
    here: each part's output is left pending and the next norm adds it."""

    def __init__(self, spec, width, name):
        super().__init__(spec, width, name)
        self.mixer_norm = build_part("norm", spec.mixer_norm, width, f"{name}.{spec.mixer_norm_name}")
        self.mixer = build_part("mixer", spec.mixer, width, f"{name}.{spec.mixer_name}")
        self.ffn_norm = build_part("norm", spec.ffn_norm, width, f"{name}.{spec.ffn_norm_name}")
        self.ffn = build_part("ffn", spec.ffn, width, f"{name}.{spec.ffn_name}")
        self.parts = (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)

    def params(self):
        return [p for part in self.parts for p in part.params()]

    def check(self, runtime):
        for part in self.parts:
            part.check(runtime)

    @property
    def graph_safe(self):
        return all(part.graph_safe for part in self.parts)

    @property
    def launches_follow_shape(self):
        return all(part.launches_follow_shape for part in self.parts)

    def load(self, tensors, runtime):
        for part in self.parts:
            part.load(tensors, runtime)

    def forward(self, ctx, hidden: HiddenState, cache) -> None:
        x = self.mixer_norm.forward(ctx, hidden)
        hidden.pending = self.mixer.forward(ctx, x, cache)
        x = self.ffn_norm.forward(ctx, hidden)
        hidden.pending = self.ffn.forward(ctx, x)


register_block("prenorm_residual", PreNormResidualBlock)
