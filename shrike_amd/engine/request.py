"""A request's life in the engine, and its sampling parameters.

Reference: shrike/engine/request.py (same names and meanings; `seed` is added
so that a sampled generation can be repeated).
"""

from __future__ import annotations

import enum
import itertools
from dataclasses import dataclass, field

from ..cache.manager import SequenceCache


class Status(enum.Enum):
    WAITING = enum.auto()
    RUNNING = enum.auto()
    FINISHED = enum.auto()


@dataclass
class SamplingParams:
    """max_new_tokens: cap on generated tokens (>= 1); the request ends with
        reason "length" when it is reached.
    temperature: 0 selects the argmax; must be >= 0.
    top_p: nucleus threshold in (0, 1]; ignored when greedy.  The largest
        entry is always kept.
    ignore_eos: generate past the end-of-sequence token (fixed-length runs).
    seed: seed of this request's draws; None derives one from the engine's
        seed and the request's id.
    """

    max_new_tokens: int = 128
    temperature: float = 0.0
    top_p: float = 1.0
    ignore_eos: bool = False
    seed: int | None = None

    def __post_init__(self) -> None:
        problems = []
        if self.max_new_tokens < 1:
            problems.append(f"max_new_tokens={self.max_new_tokens} (at least one token must be generated)")
        if self.temperature < 0.0:
            problems.append(f"temperature={self.temperature} (negative; 0 means greedy)")
        if not 0.0 < self.top_p <= 1.0:
            problems.append(f"top_p={self.top_p} (the nucleus mass lies in (0, 1])")
        if problems:
            raise ValueError("bad sampling parameters: " + "; ".join(problems))


# ids of requests made outside an engine (an engine numbers its own from 0, so
# that its default sampling seeds do not depend on what else the process ran)
_loose_ids = itertools.count()


@dataclass
class Request:
    token_ids: list[int]  # prompt; generated tokens are appended in place
    sampling: SamplingParams
    req_id: int = field(default_factory=_loose_ids.__next__)
    status: Status = Status.WAITING
    num_prompt_tokens: int = 0
    num_computed_tokens: int = 0  # tokens whose keys/values are in the cache
    cache: SequenceCache | None = None  # pages and state slot while admitted
    finish_reason: str | None = None
    # prefix-cache registration continues from here
    hashed_pages: int = 0
    last_hash: int | None = None

    def __post_init__(self):
        self.num_prompt_tokens = len(self.token_ids)

    @property
    def num_tokens(self) -> int:
        return len(self.token_ids)

    @property
    def prefill_done(self) -> bool:
        return self.num_computed_tokens >= self.num_prompt_tokens

    @property
    def num_generated(self) -> int:
        return len(self.token_ids) - self.num_prompt_tokens

    @property
    def block_table(self) -> list[int]:
        """Pages of the first page group (the only one without windows or state)."""
        if self.cache is None or not self.cache.tables:
            return []
        return self.cache.tables[0]
