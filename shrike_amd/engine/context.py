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
  extras[name]                                 int32 arrays that parts added in
                                               their prepare() (launch lists of
                                               their kernels and the like)

The reference builds the same information per step as Python lists and one
tensor per sequence (shrike/engine/model_runner.py:205-248).

A step is described twice.  `StepShape` is the host's view before anything is
on the device: the lengths, and what each part wants to add.  `StepContext` is
what `forward` gets: the same numbers plus the device arrays.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch


class Workspace:
    """Named device buffers that persist across steps and grow on demand.

    `keep_outgrown`: a buffer that is replaced by a larger one stays allocated.
    HIP graphs hold the addresses of the buffers they were recorded with; a
    workspace that graphs share must never free one of them."""

    def __init__(self, device, keep_outgrown: bool = False):
        self.device = device
        self.keep_outgrown = keep_outgrown
        self._flat: dict[tuple[str, torch.dtype], torch.Tensor] = {}
        self._outgrown: list[torch.Tensor] = []
        # (name, dtype, shape) -> the view that was handed out last time: a step asks for
        # the same few dozen buffers layer after layer, and making a view costs a microsecond
        self._views: dict[tuple, torch.Tensor] = {}
        self.generation = 0  # counts allocations: recorded launches name the buffers of one generation

    def get(self, name: str, shape: tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
        shape = tuple(shape)
        view = self._views.get((name, dtype, shape))
        if view is not None:
            return view
        numel = 1
        for s in shape:
            numel *= s
        key = (name, dtype)
        flat = self._flat.get(key)
        if flat is None or flat.numel() < numel:
            if flat is not None and self.keep_outgrown:
                self._outgrown.append(flat)
            flat = torch.empty(max(numel, 1), dtype=dtype, device=self.device)
            self._flat[key] = flat
            self.generation += 1
            # views of the buffer that was replaced must not be handed out again
            self._views = {k: v for k, v in self._views.items() if k[0] != name or k[1] != dtype}
        view = flat[:numel].view(shape)
        if len(self._views) < 4096:
            self._views[(name, dtype, shape)] = view
        return view

    def nbytes(self) -> int:
        held = list(self._flat.values()) + self._outgrown
        return sum(t.numel() * t.element_size() for t in held)


def bucket(n: int, floor: int = 1) -> int:
    """The power of two (at least `floor`) that n rounds up to."""
    b = floor
    while b < n:
        b *= 2
    return b


class StepShape:
    """The host's description of a step before its metadata goes to the device.

    The runner fills in the lengths; then every part's `prepare(shape)` may
      * `add(name, array)`: an int32 array that travels with the step's one
        metadata copy and comes back as `ctx.extras[name]` on the device;
      * `notes[key] = value`: a decision taken on the host (a grid size, a
        kernel variant) for its own `forward` to read from `ctx.notes`;
      * `launch_key.append(x)`: anything hashable that its launches depend on
        beyond the number of rows.  Steps are replayed from one HIP graph only
        if their launch keys are equal.
    Parts that share a key share the work: the first to prepare sets it, the
    others find it there.  In a step of single tokens that is replayed from a
    graph, what a part adds may depend on the step's shape only (row count and
    launch key), never on its contents: the graph's later steps reuse it.
    """

    def __init__(self, q_lens: np.ndarray, starts: np.ndarray, page_size: int,
                 padded_rows: int = 0):
        self.q_lens = q_lens
        self.starts = starts
        self.ctx_lens = starts + q_lens
        self.page_size = page_size
        self.num_seqs = int(q_lens.size)
        self.num_tokens = int(q_lens.sum())
        self.num_decode = int((q_lens == 1).sum())  # sequences with one token come first
        self.padded_rows = padded_rows  # trailing rows that stand for no request
        self.max_decode_ctx = int(self.ctx_lens[: self.num_decode].max()) if self.num_decode else 0
        self.extras: dict[str, np.ndarray] = {}
        self.notes: dict = {}
        self.launch_key: list = []

    def add(self, name: str, array) -> None:
        if name in self.extras:
            raise KeyError(f"a part already added {name!r} to this step")
        self.extras[name] = np.asarray(array, dtype=np.int64).reshape(-1)


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
    # what the parts' prepare() added: device arrays, and host-side decisions
    extras: dict = field(default_factory=dict)
    notes: dict = field(default_factory=dict)
    # everything a step's launches may depend on, for parts that say launches_follow_shape
    shape_key: tuple = ()

    def buffer(self, name: str, shape: tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
        return self.workspace.get(name, shape, dtype)
