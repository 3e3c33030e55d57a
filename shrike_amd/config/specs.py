"""Descriptions of a model as data: which parts each layer is made of, with
every size and constant as a field, and the order in which layers run.

A spec is a frozen dataclass with a class attribute ``kind``; the part class
registered under that kind (``shrike_amd.parts.registry``) is built from it.
An architecture turns its config.json into a :class:`ModelSpec`; nothing below
this level knows which architecture it came from.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import ClassVar


@dataclass(frozen=True)
class RMSNormSpec:
    """y = x * rsqrt(mean(x^2) + eps) * weight."""

    kind: ClassVar[str] = "rmsnorm"
    eps: float


@dataclass(frozen=True)
class RotarySpec:
    """Rotation of element pairs (i, i + rotary_dim/2) by position * theta**(-2i/rotary_dim)."""

    kind: ClassVar[str] = "rotary_half"
    theta: float
    rotary_dim: int


@dataclass(frozen=True)
class AttentionSpec:
    """Causal grouped-query attention over a paged key/value cache.

    ``window``: a query at position p reads keys j with p - window < j <= p;
    None reads every key.  ``position`` is applied to queries and keys after
    the projections; None leaves them as they are.
    """

    kind: ClassVar[str] = "paged_attention"
    num_heads: int
    num_kv_heads: int
    head_dim: int
    qkv_bias: bool
    out_bias: bool
    scale: float
    window: int | None = None
    position: RotarySpec | None = None


@dataclass(frozen=True)
class SwiGLUSpec:
    """down(act(gate(x)) * up(x)) without biases; act is "silu" (SwiGLU proper) or
    "gelu_tanh" (the tanh form of GELU)."""

    kind: ClassVar[str] = "swiglu"
    intermediate_size: int
    activation: str = "silu"


@dataclass(frozen=True)
class BlockSpec:
    """x += mixer(mixer_norm(x)); x += ffn(ffn_norm(x)).

    ``name`` is the prefix of the block's tensors in the weight file; the
    ``*_name`` fields are the sub-names of its parts below that prefix.
    """

    kind: ClassVar[str] = "prenorm_residual"
    name: str
    mixer: object
    ffn: object
    mixer_norm: object
    ffn_norm: object
    mixer_name: str = "self_attn"
    ffn_name: str = "mlp"
    mixer_norm_name: str = "input_layernorm"
    ffn_norm_name: str = "post_attention_layernorm"


@dataclass(frozen=True)
class TokenEmbeddingSpec:
    """x = table[token id], no scaling."""

    kind: ClassVar[str] = "token_lookup"
    vocab_size: int


@dataclass(frozen=True)
class LinearHeadSpec:
    """logits = x @ W.T, no bias."""

    kind: ClassVar[str] = "linear"
    vocab_size: int


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a block.  ``cache_of`` names an earlier schedule position whose
    cache this run reads instead of owning one; None means it owns its cache."""

    block: int
    cache_of: int | None = None


@dataclass(frozen=True)
class ModelSpec:
    """Token ids -> embedding -> schedule of blocks -> final norm -> head.

    ``embedding`` and ``head`` are part specs like the others; left as None they
    are the plain table lookup and the plain output matrix over ``vocab_size``.
    """

    architecture: str
    hidden_size: int
    vocab_size: int
    blocks: tuple[BlockSpec, ...]
    final_norm: object
    tie_word_embeddings: bool
    schedule: tuple[ScheduleEntry, ...] = ()
    embed_name: str = "model.embed_tokens"
    final_norm_name: str = "model.norm"
    head_name: str = "lm_head"
    eos_token_ids: tuple[int, ...] = ()
    max_position_embeddings: int | None = None
    stored_dtype: str = "bfloat16"
    extra: dict = field(default_factory=dict, compare=False)
    embedding: object = None
    head: object = None

    def __post_init__(self):
        if self.embedding is None:
            object.__setattr__(self, "embedding", TokenEmbeddingSpec(self.vocab_size))
        if self.head is None:
            object.__setattr__(self, "head", LinearHeadSpec(self.vocab_size))
        if not self.schedule:
            object.__setattr__(
                self, "schedule", tuple(ScheduleEntry(i) for i in range(len(self.blocks)))
            )
        for pos, entry in enumerate(self.schedule):
            if not 0 <= entry.block < len(self.blocks):
                raise ValueError(f"schedule[{pos}] names block {entry.block}, which does not exist")
            if entry.cache_of is not None:
                if not 0 <= entry.cache_of < pos:
                    raise ValueError(
                        f"schedule[{pos}] reads the cache of position {entry.cache_of}, "
                        "which is not an earlier position"
                    )
                if self.schedule[entry.cache_of].cache_of is not None:
                    raise ValueError(
                        f"schedule[{pos}] reads the cache of position {entry.cache_of}, "
                        "which does not own one"
                    )
