"""Qwen2.5 dense decoder (``Qwen2ForCausalLM``): its typed configuration and
the function that lays its layers out as parts.

The formulas are those of the reference's shrike/models/qwen.py: RMSNorm
(:70-74), q/k/v projections with bias and an output projection without
(:111-114), half-split rotary position encoding on q and k (:80-101), causal
grouped-query attention scaled by head_dim**-0.5, a SwiGLU feed-forward
without biases (:131-136), pre-norm residual blocks (:147-150), a final norm
and an output matrix that is the embedding table when the weights are tied
(:164, :190-192, :211-212).
"""

from __future__ import annotations

from dataclasses import dataclass

from ..config.engine_config import canonical_dtype
from ..config.registry import ConfigError, register_architecture
from ..config.specs import (
    AttentionSpec,
    BlockSpec,
    ModelSpec,
    RMSNormSpec,
    RotarySpec,
    SwiGLUSpec,
)

ARCHITECTURE = "Qwen2ForCausalLM"


def _need(raw: dict, key: str, kind):
    if key not in raw or raw[key] is None:
        raise ConfigError(f"config.json lacks the key {key!r}, which {ARCHITECTURE} needs")
    value = raw[key]
    if kind is int:
        if isinstance(value, bool) or not isinstance(value, int):
            raise ConfigError(f"config.json: {key} must be an integer, got {value!r}")
    elif kind is float:
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise ConfigError(f"config.json: {key} must be a number, got {value!r}")
        value = float(value)
    return value


@dataclass(frozen=True)
class Qwen2Config:
    """The keys of a Qwen2.5 config.json.

    Required, as in the reference (shrike/models/qwen.py:33-43): hidden_size,
    intermediate_size, num_hidden_layers, num_attention_heads,
    num_key_value_heads, vocab_size, rms_norm_eps, rope_theta.  head_dim falls
    back to hidden_size // num_attention_heads when absent or zero (:38),
    tie_word_embeddings to False (:42), torch_dtype to bfloat16 (:49).
    eos_token_id may be an int or a list (:44-48); it and
    max_position_embeddings may be absent here because replay needs neither.
    The reference does not read use_sliding_window, sliding_window and
    max_window_layers; here a window that is switched on is honoured: layers
    max_window_layers.. read only the last sliding_window keys.
    """

    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool = False
    attention_bias: bool = True
    max_position_embeddings: int | None = None
    eos_token_ids: tuple[int, ...] = ()
    torch_dtype: str = "bfloat16"
    use_sliding_window: bool = False
    sliding_window: int | None = None
    max_window_layers: int = 0

    def __post_init__(self):
        for name in (
            "hidden_size",
            "intermediate_size",
            "num_hidden_layers",
            "num_attention_heads",
            "num_key_value_heads",
            "head_dim",
            "vocab_size",
        ):
            if getattr(self, name) < 1:
                raise ConfigError(f"config.json: {name} must be positive, got {getattr(self, name)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"config.json: num_attention_heads ({self.num_attention_heads}) must be a "
                f"multiple of num_key_value_heads ({self.num_key_value_heads})"
            )
        if self.head_dim % 2:
            raise ConfigError(f"config.json: head_dim must be even for rotation, got {self.head_dim}")
        if not self.rms_norm_eps > 0:
            raise ConfigError(f"config.json: rms_norm_eps must be > 0, got {self.rms_norm_eps}")
        if not self.rope_theta > 0:
            raise ConfigError(f"config.json: rope_theta must be > 0, got {self.rope_theta}")
        if self.use_sliding_window and (self.sliding_window is None or self.sliding_window < 1):
            raise ConfigError("config.json: use_sliding_window needs a positive sliding_window")

    @classmethod
    def from_dict(cls, raw: dict) -> "Qwen2Config":
        hidden = _need(raw, "hidden_size", int)
        heads = _need(raw, "num_attention_heads", int)
        if heads < 1:
            raise ConfigError(f"config.json: num_attention_heads must be positive, got {heads}")
        head_dim = raw.get("head_dim") or hidden // heads
        eos = raw.get("eos_token_id")
        eos_ids = tuple(eos) if isinstance(eos, (list, tuple)) else (() if eos is None else (eos,))
        if raw.get("rope_scaling") not in (None, {}):
            raise ConfigError("config.json: rope_scaling is not supported for Qwen2ForCausalLM")
        act = raw.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"config.json: hidden_act must be 'silu', got {act!r}")
        dtype = raw.get("torch_dtype", raw.get("dtype")) or "bfloat16"
        try:
            dtype = canonical_dtype(dtype)
        except ValueError as e:
            raise ConfigError(f"config.json: {e}") from None
        use_window = bool(raw.get("use_sliding_window", False))
        return cls(
            hidden_size=hidden,
            intermediate_size=_need(raw, "intermediate_size", int),
            num_hidden_layers=_need(raw, "num_hidden_layers", int),
            num_attention_heads=heads,
            num_key_value_heads=_need(raw, "num_key_value_heads", int),
            head_dim=int(head_dim),
            vocab_size=_need(raw, "vocab_size", int),
            rms_norm_eps=_need(raw, "rms_norm_eps", float),
            rope_theta=_need(raw, "rope_theta", float),
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            attention_bias=bool(raw.get("attention_bias", True)),
            max_position_embeddings=raw.get("max_position_embeddings"),
            eos_token_ids=tuple(int(t) for t in eos_ids),
            torch_dtype=dtype,
            use_sliding_window=use_window,
            sliding_window=raw.get("sliding_window") if use_window else None,
            max_window_layers=int(raw.get("max_window_layers") or 0) if use_window else 0,
        )

    def to_dict(self) -> dict:
        """A config.json that `from_dict` reads back to the same configuration."""
        out = {
            "architectures": [ARCHITECTURE],
            "model_type": "qwen2",
            "hidden_act": "silu",
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "vocab_size": self.vocab_size,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "attention_bias": self.attention_bias,
            "torch_dtype": self.torch_dtype,
            "use_sliding_window": self.use_sliding_window,
        }
        if self.max_position_embeddings is not None:
            out["max_position_embeddings"] = self.max_position_embeddings
        if self.eos_token_ids:
            out["eos_token_id"] = (
                self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
            )
        if self.use_sliding_window:
            out["sliding_window"] = self.sliding_window
            out["max_window_layers"] = self.max_window_layers
        return out


def build_spec(cfg: Qwen2Config) -> ModelSpec:
    norm = RMSNormSpec(eps=cfg.rms_norm_eps)
    rotary = RotarySpec(theta=cfg.rope_theta, rotary_dim=cfg.head_dim)
    ffn = SwiGLUSpec(intermediate_size=cfg.intermediate_size)
    blocks = []
    for i in range(cfg.num_hidden_layers):
        windowed = cfg.use_sliding_window and i >= cfg.max_window_layers
        mixer = AttentionSpec(
            num_heads=cfg.num_attention_heads,
            num_kv_heads=cfg.num_key_value_heads,
            head_dim=cfg.head_dim,
            qkv_bias=cfg.attention_bias,
            out_bias=False,
            scale=cfg.head_dim**-0.5,
            window=cfg.sliding_window if windowed else None,
            position=rotary,
        )
        blocks.append(
            BlockSpec(
                name=f"model.layers.{i}", mixer=mixer, ffn=ffn, mixer_norm=norm, ffn_norm=norm
            )
        )
    return ModelSpec(
        architecture=ARCHITECTURE,
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        blocks=tuple(blocks),
        final_norm=norm,
        tie_word_embeddings=cfg.tie_word_embeddings,
        eos_token_ids=cfg.eos_token_ids,
        max_position_embeddings=cfg.max_position_embeddings,
        stored_dtype=cfg.torch_dtype,
    )


register_architecture(ARCHITECTURE, Qwen2Config, build_spec, model_types=("qwen2",))
