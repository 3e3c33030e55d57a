"""The cache manager: pages of keys and values with a block table per request,
one pool per group of layers with the same need, and slots for per-request
state of fixed size.

Layers whose mixers ask for the same PagedSpec form a group; a group has its
own pool of pages, its own device tensors (whatever the spec lists per page,
each as ``[layers, pages + 1, *its shape for one page]``: what a page holds and
how it is laid out is the mixer's business, not the manager's) and, per request,
its own block table.  A group with a window gives pages back as soon as no later
query can reach them (table entry -1); all pages come back when the request ends.
Layers whose mixers ask for a StateSpec form state groups: a tensor
``[layers, slots, *shape]`` indexed by the request's state slot.  Every request
holds one slot, whether or not any layer has state.

Reference: shrike/engine/block_manager.py (allocation by delta :60-77, prefix
matching :89-105, registration :107-119, release :121-130) and the pool of
shrike/engine/model_runner.py:52-60, which is one group without a window.
"""

from __future__ import annotations

from dataclasses import dataclass, field

from ..parts.base import PagedSpec, StateSpec
from .pages import PageError, PagePool, SlotPool


@dataclass
class SequenceCache:
    """What one request holds: a block table per page group and a state slot."""

    tables: list[list[int]]
    state_slot: int
    fresh_state: bool = True  # no portion has run since the slot was taken
    _trimmed: list[int] = field(default_factory=list)  # pages given back per group (count)


@dataclass
class LayerCache:
    """What a mixer gets for one run of its layer."""

    group: int  # index into ctx.block_tables / ctx.state tensors
    owned: bool  # False: reads the cache another schedule position writes
    page_size: int = 0
    # name -> this layer's slice [pages + 1, *shape of one page] of each tensor the
    # mixer's PagedSpec lists (empty where no device memory was allocated)
    pools: dict = field(default_factory=dict)
    window: int | None = None
    state: object = None  # [slots, *shape] for a StateSpec layer
    # the same memory with one slot more, [slots + 1, *shape]: the padding rows of
    # a fixed-size (graph) batch carry the slot index `slots`, which only this
    # view holds, so whatever they write disturbs no request
    state_padded: object = None


class PageGroup:
    def __init__(self, spec: PagedSpec, num_pages: int):
        self.spec = spec
        self.layers: list[int] = []  # schedule positions that own a cache of this group
        self.pool = PagePool(num_pages)
        self.tensors: dict = {}  # name -> [layers, pages + 1, *shape of one page]


class StateGroup:
    def __init__(self, spec: StateSpec):
        self.spec = spec
        self.layers: list[int] = []
        self.tensor = None  # [layers, slots, *shape]
        self.padded = None  # [layers, slots + 1, *shape], the same memory plus the spare slot


class CacheManager:
    """`layer_specs[i]` is the cache need of schedule position i (None when it
    owns no cache).  `allocate=False` keeps the bookkeeping only (CPU tests)."""

    def __init__(
        self,
        layer_specs: list,
        page_size: int,
        num_pages: int,
        max_slots: int = 256,
        enable_prefix_caching: bool = True,
    ):
        self.page_size = page_size
        self.num_pages = num_pages
        self.groups: list[PageGroup] = []
        self.state_groups: list[StateGroup] = []
        self._where: dict[int, tuple[str, int, int]] = {}  # position -> (family, group, index)
        for pos, spec in enumerate(layer_specs):
            if spec is None:
                continue
            if isinstance(spec, PagedSpec):
                family, groups, make = "pages", self.groups, lambda s: PageGroup(s, num_pages)
            elif isinstance(spec, StateSpec):
                family, groups, make = "state", self.state_groups, StateGroup
            else:
                raise TypeError(f"schedule position {pos}: unknown cache need {spec!r}")
            for gi, g in enumerate(groups):
                if g.spec == spec:
                    break
            else:
                groups.append(make(spec))
                gi = len(groups) - 1
            self._where[pos] = (family, gi, len(groups[gi].layers))
            groups[gi].layers.append(pos)
        self.slots = SlotPool(max_slots)
        # A prefix can only be shared where every layer's cache is a pure
        # function of the prefix, page by page: no window, no state.
        self.enable_prefix_caching = bool(
            enable_prefix_caching
            and not self.state_groups
            and all(g.spec.window is None for g in self.groups)
        )
        self.cache_hit_blocks = 0
        self.cache_query_blocks = 0

    # ----------------------------------------------------------- device memory

    def bytes_per_page(self, elem_size: int) -> int:
        """Bytes that one page id costs over all groups and layers; `elem_size` is
        that of the compute dtype, which tensors without a dtype of their own have."""
        import torch

        total = 0
        for g in self.groups:
            for t in g.spec.tensors:
                size = elem_size if t.dtype is None else torch.empty(0, dtype=getattr(torch, t.dtype)).element_size()
                total += len(g.layers) * t.numel(self.page_size) * size
        return total

    def allocate(self, dtype, device) -> None:
        import torch

        for g in self.groups:
            # one page more than the pool hands out: page `num_pages` is where the
            # padding rows of a fixed-size (graph) batch put what they write
            for t in g.spec.tensors:
                g.tensors[t.name] = torch.zeros(
                    len(g.layers), self.num_pages + 1, *t.shape(self.page_size),
                    dtype=dtype if t.dtype is None else getattr(torch, t.dtype), device=device,
                )
        for g in self.state_groups:
            g.padded = torch.zeros(
                len(g.layers), self.slots.num_slots + 1, *g.spec.shape,
                dtype=getattr(torch, g.spec.dtype), device=device,
            )
            g.tensor = g.padded[:, : self.slots.num_slots]

    def layer_cache(self, position: int, reader: bool = False) -> LayerCache:
        """The cache of schedule position `position`; `reader` marks a layer that
        only reads it."""
        family, gi, li = self._where[position]
        if family == "pages":
            g = self.groups[gi]
            return LayerCache(
                group=gi, owned=not reader, page_size=self.page_size,
                pools={name: t[li] for name, t in g.tensors.items()},
                window=g.spec.window,
            )
        g = self.state_groups[gi]
        return LayerCache(group=gi, owned=not reader, state=None if g.tensor is None else g.tensor[li],
                          state_padded=None if g.padded is None else g.padded[li])

    def owns_cache(self, position: int) -> bool:
        return position in self._where

    # ------------------------------------------------------------- per request

    @property
    def num_free(self) -> int:
        """Free pages of the scarcest group (every group has `num_pages` pages)."""
        return min((g.pool.num_free for g in self.groups), default=self.num_pages)

    def new_sequence(self) -> SequenceCache:
        slot = self.slots.take()
        for g in self.state_groups:
            if g.tensor is not None:
                from ..kernels import ops

                for layer in range(g.tensor.shape[0]):
                    ops.zero_(g.tensor[layer, slot])
        return SequenceCache(
            tables=[[] for _ in self.groups], state_slot=slot, _trimmed=[0] * len(self.groups)
        )

    def pages_needed(self, seq: SequenceCache, num_computed: int, n_new: int) -> list[int]:
        """Additional pages each group needs to hold num_computed + n_new tokens."""
        total = -(-(num_computed + n_new) // self.page_size)
        return [max(0, total - len(table)) for table in seq.tables]

    def can_append(self, seq: SequenceCache, num_computed: int, n_new: int) -> bool:
        need = self.pages_needed(seq, num_computed, n_new)
        return all(n <= g.pool.num_free for n, g in zip(need, self.groups))

    def append(self, seq: SequenceCache, num_computed: int, n_new: int) -> None:
        need = self.pages_needed(seq, num_computed, n_new)
        if not all(n <= g.pool.num_free for n, g in zip(need, self.groups)):
            raise PageError("append without room: call can_append first")
        for n, g, table in zip(need, self.groups, seq.tables):
            for _ in range(n):
                table.append(g.pool.take())

    def trim(self, seq: SequenceCache, num_computed: int) -> int:
        """Give back the pages of windowed groups that no later query can reach.

        After `num_computed` tokens the next query sits at position >=
        num_computed and reads keys > num_computed - window; pages that end at
        or before num_computed - window + 1 are done.  Returns pages released.
        """
        released = 0
        for gi, (g, table) in enumerate(zip(self.groups, seq.tables)):
            w = g.spec.window
            if w is None:
                continue
            first_needed = max(0, num_computed - w + 1)
            done = min(first_needed // self.page_size, len(table))
            for i in range(seq._trimmed[gi], done):
                if table[i] >= 0:
                    g.pool.release(table[i])
                    table[i] = -1
                    released += 1
            seq._trimmed[gi] = max(seq._trimmed[gi], done)
        return released

    def free(self, seq: SequenceCache) -> None:
        """Everything the request holds goes back; the object must not be used again."""
        for g, table in zip(self.groups, seq.tables):
            for page in table:
                if page >= 0:
                    g.pool.release(page)
            table.clear()
        if seq.state_slot >= 0:
            self.slots.release(seq.state_slot)
            seq.state_slot = -1

    def release_pages(self, seq: SequenceCache) -> None:
        """Give the pages back but keep the state slot (a failed admission)."""
        for gi, (g, table) in enumerate(zip(self.groups, seq.tables)):
            for page in table:
                if page >= 0:
                    g.pool.release(page)
            table.clear()
            seq._trimmed[gi] = 0

    # ---------------------------------------------------------- prefix caching

    @staticmethod
    def chain_hash(prev_hash: int | None, tokens) -> int:
        return hash((prev_hash, tuple(tokens)))

    def match_prefix(self, seq: SequenceCache, token_ids: list[int]) -> int:
        """Put the pages of the longest cached prefix of `token_ids` into the
        (empty) tables of `seq`; returns the number of tokens they hold.  At
        least one token is always left to compute (block_manager.py:96-98)."""
        if not self.enable_prefix_caching or not self.groups:
            return 0
        prev = None
        matched = 0
        for i in range((len(token_ids) - 1) // self.page_size):
            prev = self.chain_hash(prev, token_ids[i * self.page_size : (i + 1) * self.page_size])
            self.cache_query_blocks += 1
            pages = [g.pool.lookup(prev) for g in self.groups]
            if any(p is None for p in pages):
                break
            for g, table, page in zip(self.groups, seq.tables, pages):
                g.pool.share(page)
                table.append(page)
            self.cache_hit_blocks += 1
            matched += 1
        return matched * self.page_size

    def register_full_pages(self, seq: SequenceCache, token_ids: list[int], num_computed: int,
                            start_page: int = 0, prev_hash: int | None = None):
        """Hash the full pages of `seq` so that later requests can share them.
        Returns (number of full pages, hash of the last) to continue from."""
        if not self.enable_prefix_caching or not self.groups:
            return start_page, prev_hash
        num_full = num_computed // self.page_size
        for i in range(start_page, num_full):
            prev_hash = self.chain_hash(
                prev_hash, token_ids[i * self.page_size : (i + 1) * self.page_size]
            )
            for g, table in zip(self.groups, seq.tables):
                g.pool.set_hash(table[i], prev_hash)
        return max(start_page, num_full), prev_hash

    # --------------------------------------------------------------- invariants

    def check(self, live: list[SequenceCache]) -> None:
        """No page lost, none held by more holders than its count says."""
        for gi, g in enumerate(self.groups):
            g.pool.check()
            holders: dict[int, int] = {}
            for seq in live:
                for page in seq.tables[gi]:
                    if page >= 0:
                        holders[page] = holders.get(page, 0) + 1
            for page in range(g.pool.num_pages):
                if g.pool.ref_count[page] != holders.get(page, 0):
                    raise PageError(
                        f"group {gi} page {page}: count {g.pool.ref_count[page]} but "
                        f"{holders.get(page, 0)} holders"
                    )
        slots = [seq.state_slot for seq in live]
        if len(set(slots)) != len(slots) or set(slots) != self.slots.held:
            raise PageError("state slots and live requests disagree")
