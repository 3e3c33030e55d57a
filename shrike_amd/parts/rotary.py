"""Rotary position encoding with the half-split pairing (i, i + rot_dim/2)."""

from __future__ import annotations

import torch

from .base import PositionEncoding, register_position


class RotaryHalf(PositionEncoding):
    """inv_freq[i] = theta ** (-2i / rot_dim), formed in float32 exactly as the
    reference does (shrike/models/qwen.py:80); the angle of position p is
    float32(p) * inv_freq[i] (:86).  The rotation itself runs inside the
    cache-write kernel."""

    launches_follow_shape = True

    def load(self, tensors, runtime):
        d = int(self.spec.rotary_dim)
        inv_freq = 1.0 / (float(self.spec.theta) ** (torch.arange(0, d, 2).float() / d))
        self.inv_freq = inv_freq.to(runtime.device)
        self.rot_dim = d

    def rotary_table(self):
        return self.inv_freq, self.rot_dim


register_position("rotary_half", RotaryHalf)
