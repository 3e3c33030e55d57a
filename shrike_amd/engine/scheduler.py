"""Continuous batching under a token budget, with chunked prompts, first-come
first-served admission and preemption when pages run out.

Behaviour follows shrike/engine/scheduler.py:69-148:
  1. Running requests are served first, in admission order.  A request with
     one uncomputed token costs 1; one with more (a prompt in progress, or a
     preempted request catching up) gets a portion that fits the rest of the
     budget.
  2. What is left of the budget admits waiting requests, head of the queue
     only; a prompt is cut by the budget.  If the head's portion does not fit
     in the free pages, admission stops (nothing overtakes it, nothing is
     preempted for it).
  3. When a running request cannot get the pages for its portion, the newest
     running request is preempted: all it holds goes back, it will recompute
     from its first token, and it returns to the head of the waiting queue.
     If the request that needs pages is itself the newest, it is the victim
     and sits this step out.

One difference: a request that resumes after preemption recomputes its prompt
and the tokens it had generated in portions, where the reference re-decodes
generated tokens one per step (scheduler.py:80-86); the logits are the same.
"""

from __future__ import annotations

from collections import deque

from ..cache.manager import CacheManager
from .request import Request, Status


class _StepPlan:
    """What one schedule() call has handed out so far, and what is left of the budget."""

    def __init__(self, budget: int):
        self.budget = budget
        self.singles: list[tuple[Request, int]] = []
        self.portions: list[tuple[Request, int]] = []

    def take(self, req: Request, n: int) -> None:
        (self.singles if n == 1 else self.portions).append((req, n))
        self.budget -= n

    def batch(self) -> list[tuple[Request, int]]:
        return self.singles + self.portions


class Scheduler:
    def __init__(self, cache: CacheManager, max_tokens_per_step: int = 512, max_running: int = 256):
        self.cache = cache
        self.max_tokens_per_step = max_tokens_per_step
        self.max_running = max_running
        self.waiting: deque[Request] = deque()
        self.running: list[Request] = []
        self.num_preemptions = 0

    def add(self, req: Request) -> None:
        """A new request queues behind those that wait already."""
        self.waiting.append(req)

    @property
    def has_work(self) -> bool:
        return len(self.running) + len(self.waiting) > 0

    def _release(self, req: Request) -> None:
        if req.cache is not None:
            self.cache.free(req.cache)
            req.cache = None
        req.hashed_pages, req.last_hash = 0, None

    def _preempt_newest(self) -> Request:
        """The request admitted last loses its pages and its slot and goes to the
        head of the waiting queue, to start over from its first token."""
        newest = self.running.pop()
        self._release(newest)
        newest.status, newest.num_computed_tokens = Status.WAITING, 0
        self.waiting.appendleft(newest)
        self.num_preemptions += 1
        return newest

    def schedule(self) -> list[tuple[Request, int]]:
        """The next step's (request, number of its next tokens), requests with one
        token first (the step function's order), each group in admission order."""
        step = _StepPlan(self.max_tokens_per_step)
        self._serve_running(step)
        self._admit_waiting(step)
        return step.batch()

    def _serve_running(self, step: "_StepPlan") -> None:
        """Rule 1 and 3: every running request gets its next tokens while the budget
        lasts; the pages for them are taken from the newest running requests if
        need be."""
        for req in tuple(self.running):
            if step.budget == 0:
                return
            if req.status is not Status.RUNNING:
                continue  # preempted for an older request a moment ago
            wanted = min(req.num_tokens - req.num_computed_tokens, step.budget)
            while wanted > 0 and not self.cache.can_append(req.cache, req.num_computed_tokens, wanted):
                if self._preempt_newest() is req:
                    wanted = 0  # it was the newest itself: it sits this step out
            if wanted > 0:
                self.cache.append(req.cache, req.num_computed_tokens, wanted)
                step.take(req, wanted)

    def _admit_waiting(self, step: "_StepPlan") -> None:
        """Rule 2: the head of the waiting queue, again and again, while budget, running
        places, state slots and pages allow; nothing overtakes a head that does not fit."""
        while self.waiting and step.budget > 0 and len(self.running) < self.max_running \
                and self.cache.slots.num_free > 0:
            req = self.waiting[0]
            seq = self.cache.new_sequence()
            # a request that was preempted recomputes what it had generated as well
            cached = self.cache.match_prefix(seq, req.token_ids[: req.num_prompt_tokens])
            wanted = min(req.num_tokens - cached, step.budget)
            if not self.cache.can_append(seq, cached, wanted):
                self.cache.free(seq)  # the slot, and the references that the prefix match took
                return
            self.cache.append(seq, cached, wanted)
            self.waiting.popleft()
            req.cache, req.num_computed_tokens, req.status = seq, cached, Status.RUNNING
            req.hashed_pages, req.last_hash = 0, None
            self.running.append(req)
            step.take(req, wanted)

    def plan_decode_step(self) -> list[tuple[Request, int]] | None:
        """What the next schedule() will return if every running request goes on
        with the one token that is being sampled for it right now and nothing
        arrives meanwhile: that token for each of them, in admission order.  Called
        after postprocess() and before the sampled tokens are known, so that the
        host prepares the next step while the device still computes this one.
        None when the next step is not of this kind (somebody waits, a prompt is
        in progress, a request reaches its length, the budget or the pages do not
        suffice): schedule() then decides as ever.  Pages taken here are those
        schedule() would take; a request that ends after all gives them back with
        the rest."""
        if self.waiting or not self.running or len(self.running) > self.max_tokens_per_step:
            return None
        for req in self.running:
            if req.status is not Status.RUNNING or req.num_computed_tokens != req.num_tokens:
                return None
            if req.num_generated + 1 >= req.sampling.max_new_tokens:
                return None
        for req in self.running:
            if not self.cache.can_append(req.cache, req.num_computed_tokens, 1):
                return None  # schedule() finds the same shortage, and preempts
            self.cache.append(req.cache, req.num_computed_tokens, 1)
        return [(req, 1) for req in self.running]

    def postprocess(self, batch: list[tuple[Request, int]]) -> None:
        """Count the step's tokens as computed, publish full pages for prefix
        sharing, and give back pages that a window has passed."""
        for req, n_new in batch:
            req.num_computed_tokens += n_new
            req.hashed_pages, req.last_hash = self.cache.register_full_pages(
                req.cache, req.token_ids, req.num_computed_tokens, req.hashed_pages, req.last_hash
            )
            self.cache.trim(req.cache, req.num_computed_tokens)

    def finish(self, req: Request, reason: str) -> None:
        """A running request is done: it leaves the running list and everything
        it holds goes back to the cache manager."""
        self.running.remove(req)
        self._release(req)
        req.status, req.finish_reason = Status.FINISHED, reason

    def abort(self, req: Request) -> None:
        """Drop a request wherever it is (command line interrupt)."""
        if req in self.running:
            self.finish(req, "aborted")
            return
        if req in self.waiting:
            self.waiting.remove(req)
        self._release(req)
        req.status, req.finish_reason = Status.FINISHED, "aborted"
