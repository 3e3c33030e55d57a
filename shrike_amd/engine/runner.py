"""The step function: one flat batch of (sequence, its next tokens), portions
of prompts beside single decoded tokens, run from the cache; logits come back
for the wanted places only.

Reference: shrike/engine/model_runner.py:183-250.  Differences by design: the
entries carry their tokens and wanted rows explicitly (so replay can ask for
any row), all metadata goes to the device in one copy, and nothing is computed
on the host per token.
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from ..cache.manager import CacheManager, SequenceCache
from .context import StepContext, Workspace


@dataclass
class StepEntry:
    """`tokens` are the sequence's next tokens, the first at position `start`
    (= tokens already in its cache); `want` are offsets into `tokens`."""

    cache: SequenceCache
    tokens: list
    start: int
    want: list


class StepError(ValueError):
    """A step was refused before anything ran."""


class ModelRunner:
    def __init__(self, model, cache: CacheManager, runtime):
        self.model = model
        self.cache = cache
        self.runtime = runtime
        self.workspace = Workspace(runtime.device)
        self.vocab_size = model.spec.vocab_size
        self.layer_caches = []
        for pos, entry in enumerate(model.spec.schedule):
            owner = pos if entry.cache_of is None else entry.cache_of
            if cache.owns_cache(owner):
                self.layer_caches.append(cache.layer_cache(owner, reader=entry.cache_of is not None))
            else:
                self.layer_caches.append(None)
        self._pinned = None
        self._pinned_free = None  # event: the last copy out of the pinned buffer is done

    # ---------------------------------------------------------------- metadata

    def _check(self, entries: list[StepEntry]) -> None:
        ps = self.cache.page_size
        seen = set()
        for e in entries:
            if id(e.cache) in seen:
                raise StepError("a sequence appears twice in one step")
            seen.add(id(e.cache))
            n = len(e.tokens)
            if n < 1:
                raise StepError("an entry of a step needs at least one token")
            if e.start < 0:
                raise StepError(f"negative start {e.start}")
            if any(not 0 <= w < n for w in e.want):
                raise StepError(f"wanted offsets {list(e.want)} lie outside the entry's {n} tokens")
            last_page = (e.start + n - 1) // ps
            for g, table in zip(self.cache.groups, e.cache.tables):
                if len(table) <= last_page:
                    raise StepError(
                        f"block table has {len(table)} pages but the step reaches page {last_page}"
                    )
                w = g.spec.window
                first = 0 if w is None else max(0, e.start - w + 1) // ps
                if any(p < 0 or p >= self.cache.num_pages for p in table[first : last_page + 1]):
                    raise StepError("block table names a page outside the pool")

    def build_context(self, entries: list[StepEntry]) -> StepContext:
        self._check(entries)
        order = sorted(range(len(entries)), key=lambda i: 0 if len(entries[i].tokens) == 1 else 1)
        q_lens = np.array([len(entries[i].tokens) for i in order], dtype=np.int64)
        starts = np.array([entries[i].start for i in order], dtype=np.int64)
        num_seqs = len(order)
        num_tokens = int(q_lens.sum())
        num_decode = int((q_lens == 1).sum())
        cu_q = np.zeros(num_seqs + 1, dtype=np.int64)
        np.cumsum(q_lens, out=cu_q[1:])
        token_seq = np.repeat(np.arange(num_seqs), q_lens)
        positions = np.arange(num_tokens) - cu_q[token_seq] + starts[token_seq]
        token_ids = np.concatenate([np.asarray(entries[i].tokens, dtype=np.int64) for i in order])
        if token_ids.min() < 0 or token_ids.max() >= self.vocab_size:
            raise StepError(f"token ids must lie in [0, {self.vocab_size})")
        ctx_lens = starts + q_lens
        slot_of = {i: k for k, i in enumerate(order)}
        out_rows = [cu_q[slot_of[i]] + w for i, e in enumerate(entries) for w in e.want]
        state_slots = np.array([entries[i].cache.state_slot for i in order], dtype=np.int64)
        fresh = np.array([int(entries[i].cache.fresh_state) for i in order], dtype=np.int64)
        tables = []
        for gi in range(len(self.cache.groups)):
            width = max(1, max(len(entries[i].cache.tables[gi]) for i in order))
            t = np.zeros((num_seqs, width), dtype=np.int64)
            for k, i in enumerate(order):
                row = entries[i].cache.tables[gi]
                t[k, : len(row)] = row
            tables.append(t)

        # prompt portions in tiles of 16 queries for the MFMA attention kernel
        tile_counts = -(-q_lens[num_decode:] // 16)
        tile_seq = np.repeat(np.arange(num_decode, num_seqs), tile_counts)
        tile_first = np.zeros(num_seqs - num_decode + 1, dtype=np.int64)
        np.cumsum(tile_counts, out=tile_first[1:])
        tile_q0 = (np.arange(int(tile_counts.sum())) - tile_first[tile_seq - num_decode]) * 16

        parts = [token_ids, positions, token_seq, cu_q, ctx_lens, state_slots, fresh,
                 np.asarray(out_rows, dtype=np.int64), tile_seq, tile_q0]
        parts += [t.reshape(-1) for t in tables]
        sizes = [p.size for p in parts]
        total = int(sum(sizes))
        if self._pinned_free is not None:
            self._pinned_free.synchronize()
        if self._pinned is None or self._pinned.numel() < total:
            self._pinned = torch.empty(max(2 * total, 4096), dtype=torch.int32, pin_memory=True)
            self._pinned_free = torch.cuda.Event()
        host = self._pinned[:total]
        host.numpy()[:] = np.concatenate(parts).astype(np.int32)
        dev = self.workspace.get("step_meta", (total,), torch.int32)
        dev.copy_(host, non_blocking=True)
        self._pinned_free.record()
        views, off = [], 0
        for s in sizes:
            views.append(dev[off : off + s])
            off += s
        return StepContext(
            dtype=self.runtime.dtype, device=self.runtime.device, workspace=self.workspace,
            num_tokens=num_tokens, num_seqs=num_seqs, num_decode=num_decode,
            token_ids=views[0], positions=views[1], token_seq=views[2], cu_q=views[3],
            ctx_lens=views[4], state_slots=views[5], fresh=views[6], out_rows=views[7],
            tile_seq=views[8], tile_q0=views[9], num_prefill_tiles=int(tile_seq.size),
            block_tables=[v.view(num_seqs, t.shape[1]) for v, t in zip(views[10:], tables)],
            q_lens=q_lens.tolist(), ctx_lens_host=ctx_lens.tolist(),
            max_q_len=int(q_lens.max()), max_ctx_len=int(ctx_lens.max()),
            max_decode_ctx=int(ctx_lens[:num_decode].max()) if num_decode else 0,
        )

    # -------------------------------------------------------------------- step

    def step(self, entries: list[StepEntry]) -> torch.Tensor:
        """Runs the entries' tokens as one batch; returns float32 logits
        [wanted, vocab] in the order of the entries and of their `want`.
        The tensor is a view of a buffer that the next step overwrites."""
        if not entries:
            return torch.empty(0, self.vocab_size, dtype=torch.float32, device=self.runtime.device)
        ctx = self.build_context(entries)
        logits = self.model.forward(ctx, self.layer_caches)
        for e in entries:
            e.cache.fresh_state = False
        return logits
