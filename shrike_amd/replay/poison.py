"""Poisoning of cache pages that no request holds.

A page that is free, or was never used, is filled with NaN in every layer of
its group, in every floating-point tensor that the group's mixers keep per page.  Whatever reads it (a stale block table, a key beyond a request's
length, a page that a window has already given back) then shows up as NaN in
the logits, instead of as the plausible numbers a finished request left there.
The fills are ordinary tensor fills on the pool's slices, outside any HIP graph.
"""

from __future__ import annotations

from ..cache.manager import CacheManager, SequenceCache


class PagePoisoner:
    def __init__(self, cache: CacheManager):
        self.cache = cache

    def poison_everything(self) -> None:
        """Before the first step: every page of every group, the spare page included."""
        for g in self.cache.groups:
            for t in g.tensors.values():
                if t.is_floating_point():
                    t.fill_(float("nan"))

    def poison_pages(self, group: int, pages) -> None:
        pages = sorted(set(int(p) for p in pages))
        if not pages:
            return
        for t in self.cache.groups[group].tensors.values():
            if t.is_floating_point():
                t[:, pages] = float("nan")

    def held(self, seq: SequenceCache) -> list[list[int]]:
        """The pages a request holds now, per group."""
        return [[p for p in table if p >= 0] for table in seq.tables]

    def poison_released(self, before: list[list[int]], seq: SequenceCache | None = None) -> list[list[int]]:
        """Poisons those of `before` that the request no longer holds (all of them
        when `seq` is None: the request has ended) and that nobody else holds
        either.  Returns what was poisoned, per group."""
        done = []
        for gi, pages in enumerate(before):
            still = set() if seq is None else {p for p in seq.tables[gi] if p >= 0}
            pool = self.cache.groups[gi].pool
            gone = [p for p in pages if p not in still and pool.ref_count[p] == 0]
            self.poison_pages(gi, gone)
            done.append(gone)
        return done
