"""A pool of cache pages: free list, reference counts and the hashes that let
a later request reuse the pages of an equal prompt prefix.

Reference: shrike/engine/block_manager.py:21-58, 121-126.  Pages are handed
out oldest-freed first; a freed page keeps its hash until it is handed out
again, so it can still be revived by a prefix match.
"""

from __future__ import annotations

from collections import deque


class PageError(RuntimeError):
    """A page was released more often than it was taken, or the pool ran dry."""


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages < 1:
            raise ValueError(f"a page pool needs at least one page, got {num_pages}")
        self.num_pages = num_pages
        self.ref_count = [0] * num_pages
        self.hash_of: list[int | None] = [None] * num_pages
        self.page_of_hash: dict[int, int] = {}
        self.free: deque[int] = deque(range(num_pages))

    @property
    def num_free(self) -> int:
        return len(self.free)

    def take(self) -> int:
        """Oldest free page, with its stale hash dropped; reference count 1."""
        if not self.free:
            raise PageError("page pool is empty")
        page = self.free.popleft()
        h = self.hash_of[page]
        if h is not None:
            if self.page_of_hash.get(h) == page:
                del self.page_of_hash[h]
            self.hash_of[page] = None
        self.ref_count[page] = 1
        return page

    def share(self, page: int) -> None:
        """One more holder of `page`; a free page is taken off the free list."""
        if self.ref_count[page] == 0:
            self.free.remove(page)
        self.ref_count[page] += 1

    def release(self, page: int) -> None:
        if not 0 <= page < self.num_pages:
            raise PageError(f"page {page} is not in the pool")
        if self.ref_count[page] <= 0:
            raise PageError(f"page {page} released while nobody holds it")
        self.ref_count[page] -= 1
        if self.ref_count[page] == 0:
            self.free.append(page)

    def set_hash(self, page: int, h: int) -> None:
        """Remember that `page` holds the prefix with hash `h` (first owner wins)."""
        if self.hash_of[page] is None:
            self.hash_of[page] = h
            self.page_of_hash.setdefault(h, page)

    def lookup(self, h: int) -> int | None:
        return self.page_of_hash.get(h)

    def check(self) -> None:
        """Invariant: every page is either free (count 0, once in the list) or held."""
        free = list(self.free)
        if len(set(free)) != len(free):
            raise PageError("a page is in the free list twice")
        for page in range(self.num_pages):
            held = self.ref_count[page] > 0
            if held == (page in set(free)):
                raise PageError(f"page {page}: count {self.ref_count[page]} but free={not held}")


class SlotPool:
    """Slots for per-request state of fixed size."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self.free: deque[int] = deque(range(num_slots))
        self.held: set[int] = set()

    @property
    def num_free(self) -> int:
        return len(self.free)

    def take(self) -> int:
        if not self.free:
            raise PageError("no state slot is free")
        slot = self.free.popleft()
        self.held.add(slot)
        return slot

    def release(self, slot: int) -> None:
        if slot not in self.held:
            raise PageError(f"state slot {slot} released while nobody holds it")
        self.held.remove(slot)
        self.free.append(slot)
