"""Interfaces of the parts a layer is put together from, and their registries.

A part is built from its spec (``shrike_amd.config.specs``) and the model's
width; it never sees which model it is in.  It declares the tensors it needs
(`params`), takes them (`load`), and runs on a step's flat token batch
(`forward`).  Kinds of parts:

* Norm:              forward(ctx, hidden) -> normed [N, width] in the compute dtype;
                     folds hidden.pending into hidden.resid first.
* PositionEncoding:  tells a mixer how queries and keys depend on position.
* Mixer:             forward(ctx, x, cache) -> [N, width]; mixes information
                     between the tokens of a sequence, through `cache`
                     (pages of keys/values, or a state slot per request).
* FeedForward:       forward(ctx, x) -> [N, width]; token by token.
* Block:             forward(ctx, hidden, cache) ; arranges norms, mixer and
                     feed-forward around the residual stream.
* Embedding:         forward(ctx) -> float32 [N, width], the residual stream's
                     first value, from ctx.token_ids (and ctx.positions).
* Head:              forward(ctx, x) -> float32 [R, vocab] from the normed rows.

Any part may implement prepare(shape): it is called once per step, before the
step's metadata goes to the device, with the host-side StepShape; there a part
decides how its kernels will be launched and adds the index arrays they need.

To add a part: write its spec dataclass with a unique ``kind``, write the
class, and register it with the matching ``register_*`` function.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

import torch


@dataclass(frozen=True)
class ParamSpec:
    """One tensor a part needs from the weight file.

    init: how the random-weights mode draws it: "matrix", "embedding" and
        "bias" are N(0, 0.02), "norm" is 1 + N(0, 0.1); the "unit" mode scales
        a "matrix" by its fan-in and leaves an "embedding" at N(0, 1).
    keep_float32: held in float32 whatever the compute dtype (vectors that
        enter float32 arithmetic); others are held in the compute dtype.
    """

    name: str
    shape: tuple[int, ...]
    init: str = "matrix"
    keep_float32: bool = False
    optional: bool = False


PAGE = "page"  # in a PageTensor's dims: the place of the page size


@dataclass(frozen=True)
class PageTensor:
    """One tensor that a mixer keeps for every page of a sequence.  `dims` is the
    shape of one page's part of it, ints and PAGE (the page size, which only the
    engine's options fix); the layout within a page is the mixer's own business
    and that of its kernels.  `dtype` None: the compute dtype."""

    name: str
    dims: tuple
    dtype: str | None = None

    def shape(self, page_size: int) -> tuple[int, ...]:
        return tuple(page_size if d == PAGE else int(d) for d in self.dims)

    def numel(self, page_size: int) -> int:
        n = 1
        for d in self.shape(page_size):
            n *= d
        return n


@dataclass(frozen=True)
class PagedSpec:
    """Cache need of a mixer: something per token, kept in pages, for all earlier
    tokens (window None) or for the last `window` of them.  The cache manager
    allocates every listed tensor as [layers, pages + 1, *dims] and hands a
    layer its slice under the tensor's name; it knows nothing else about them."""

    tensors: tuple[PageTensor, ...]
    window: int | None = None

    def __post_init__(self):
        names = [t.name for t in self.tensors]
        if not names or len(set(names)) != len(names):
            raise ValueError(f"a paged cache needs tensors with distinct names, got {names}")


@dataclass(frozen=True)
class StateSpec:
    """Cache need of a mixer: one tensor of fixed shape per request."""

    shape: tuple[int, ...]
    dtype: str = "float32"


class HiddenState:
    """The residual stream of a step: `resid` float32 [N, width], plus a part's
    output `pending` (compute dtype) that has not been added yet.  The next
    norm adds it while it reads the row anyway."""

    __slots__ = ("resid", "pending")

    def __init__(self, resid: torch.Tensor, pending: torch.Tensor | None = None):
        self.resid = resid
        self.pending = pending


class Part:
    """Common face of every part."""

    # False for a part whose forward cannot be recorded into a HIP graph (it reads
    # device data on the host, or launches work whose shape depends on the data);
    # a model with such a part runs every step kernel by kernel.
    graph_safe = True
    # True for a part whose launches (kernels, their scalar arguments, the buffers
    # they name) follow from the step's shape alone: the numbers of tokens, sequences,
    # single tokens and wanted rows, the widths of the block tables, the sizes of the
    # arrays that parts added, and the step's launch key.  Steps of equal shape then
    # run such a model's forward from a recorded list of launches.  A part that
    # decides anything else on the host per step must put it into the launch key.
    launches_follow_shape = False

    def __init__(self, spec, width: int, name: str):
        self.spec = spec
        self.width = width
        self.name = name

    def params(self) -> list[ParamSpec]:
        return []

    def load(self, tensors: dict[str, torch.Tensor], runtime) -> None:
        """`tensors` maps each declared name to a device tensor."""

    def check(self, runtime) -> None:
        """Raise if the kernels cannot take this part's sizes."""

    def prepare(self, shape) -> None:
        """Called once per step with the host-side StepShape, before anything is
        copied to the device: decide launches, `shape.add` index arrays,
        leave `shape.notes` for forward, extend `shape.launch_key`."""


class Norm(Part):
    def forward(self, ctx, hidden: HiddenState, rows=None, write_resid=True) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    def rotary_table(self):
        """(inv_freq float32 [rot_dim/2], rot_dim) when the encoding is a
        half-split rotation that the cache-write kernel applies; else None."""
        return None

    def apply(self, ctx, qkv: torch.Tensor, heads: int, kv_heads: int, head_dim: int) -> None:
        """Encode queries and keys of qkv in place (for encodings without a fused kernel)."""
        raise NotImplementedError


class Mixer(Part):
    # A mixer whose cache is a StateSpec is recorded into HIP graphs only if it
    # says that its forward finds its state through ctx.state_slots and
    # ctx.fresh on the device (nothing read on the host, no launch that depends
    # on which slots the step uses).
    state_graph_safe = False

    def cache_spec(self):
        """PagedSpec, StateSpec or None."""
        return None

    def forward(self, ctx, x: torch.Tensor, cache) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    mixer: Mixer

    def forward(self, ctx, hidden: HiddenState, cache) -> None:
        raise NotImplementedError


class Embedding(Part):
    """Built from a spec with `vocab_size`; `table` is what a tied head may share."""

    table: torch.Tensor | None = None

    def forward(self, ctx) -> torch.Tensor:
        raise NotImplementedError


class Head(Part):
    """Logits from the normed rows.  `tie(embedding)` is called before load when
    the model ties its output matrix to the embedding."""

    def tie(self, embedding: Embedding) -> None:
        raise NotImplementedError

    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


_REGISTRIES: dict[str, dict[str, Callable]] = {
    "norm": {},
    "position": {},
    "mixer": {},
    "ffn": {},
    "block": {},
    "embedding": {},
    "head": {},
}


def _register(family: str, kind: str, cls) -> None:
    _REGISTRIES[family][kind] = cls


def register_norm(kind: str, cls) -> None:
    _register("norm", kind, cls)


def register_position(kind: str, cls) -> None:
    _register("position", kind, cls)


def register_mixer(kind: str, cls) -> None:
    _register("mixer", kind, cls)


def register_ffn(kind: str, cls) -> None:
    _register("ffn", kind, cls)


def register_block(kind: str, cls) -> None:
    _register("block", kind, cls)


def register_embedding(kind: str, cls) -> None:
    _register("embedding", kind, cls)


def register_head(kind: str, cls) -> None:
    _register("head", kind, cls)


def build_part(family: str, spec, width: int, name: str):
    """The part registered for ``spec.kind`` in `family`, built for `width`."""
    kind = getattr(spec, "kind", None)
    try:
        cls = _REGISTRIES[family][kind]
    except KeyError:
        known = ", ".join(sorted(_REGISTRIES[family])) or "none"
        raise ValueError(f"no {family} part of kind {kind!r} is registered (known: {known})") from None
    return cls(spec, width, name)
