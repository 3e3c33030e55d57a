"""What the parts see of one step: the flat token batch and its metadata on
the device, and a workspace of reusable buffers.

Layout of a step with N tokens of S sequences (sequences with one token
first, then prompt portions, each sequence's tokens contiguous):

  token_ids[N]  positions[N]  token_seq[N]     per token: id, position in its
                                               sequence, index of its sequence
  cu_q[S+1]                                    token range of each sequence
  ctx_lens[S]                                  tokens in the cache after the step
  state_slots[S]  fresh[S]                     state slot; 1 if this is the
                                               sequence's first portion
  block_tables[g][S, blocks_g]                 page ids per page group
  out_rows[R]                                  rows whose logits are wanted
  tile_seq[T]  tile_q0[T]                      prompt portions cut into tiles of 16
                                               queries: sequence and first query

The reference builds the same information per step as Python lists and one
tensor per sequence (shrike/engine/model_runner.py:205-248).
"""

from __future__ import annotations

from dataclasses import dataclass, field

import torch


class Workspace:
    """Named device buffers that persist across steps and grow on demand."""

    def __init__(self, device):
        self.device = device
        self._flat: dict[tuple[str, torch.dtype], torch.Tensor] = {}

    def get(self, name: str, shape: tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
        numel = 1
        for s in shape:
            numel *= s
        key = (name, dtype)
        flat = self._flat.get(key)
        if flat is None or flat.numel() < numel:
            flat = torch.empty(max(numel, 1), dtype=dtype, device=self.device)
            self._flat[key] = flat
        return flat[:numel].view(shape)


@dataclass
class StepContext:
    dtype: torch.dtype
    device: torch.device
    workspace: Workspace
    num_tokens: int
    num_seqs: int
    num_decode: int  # the first num_decode sequences have exactly one token
    token_ids: torch.Tensor
    positions: torch.Tensor
    token_seq: torch.Tensor
    cu_q: torch.Tensor
    ctx_lens: torch.Tensor
    state_slots: torch.Tensor
    fresh: torch.Tensor
    out_rows: torch.Tensor
    block_tables: list[torch.Tensor]
    # host copies for launch decisions (grids, kernel choice)
    q_lens: list[int] = field(default_factory=list)
    ctx_lens_host: list[int] = field(default_factory=list)
    max_q_len: int = 0
    max_ctx_len: int = 0
    max_decode_ctx: int = 0  # longest context among the single-token sequences
    tile_seq: torch.Tensor | None = None
    tile_q0: torch.Tensor | None = None
    num_prefill_tiles: int = 0

    _wg_cache: dict = field(default_factory=dict)

    def buffer(self, name: str, shape: tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
        return self.workspace.get(name, shape, dtype)

    def prefill_workgroups(self, tiles: int):
        """Prompt portions cut into runs of `tiles` 16-query tiles: (sequence of
        each run, its first query, number of runs), on the device."""
        hit = self._wg_cache.get(tiles)
        if hit is None:
            seqs, q0s = [], []
            for s in range(self.num_decode, self.num_seqs):
                for q0 in range(0, self.q_lens[s], 16 * tiles):
                    seqs.append(s)
                    q0s.append(q0)
            both = torch.tensor([seqs, q0s], dtype=torch.int32).to(self.device)
            hit = (both[0], both[1], len(seqs))
            self._wg_cache[tiles] = hit
        return hit
