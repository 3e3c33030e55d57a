"""Plain, slow implementation of the Qwen2.5 dense decoder on the CPU.

Whole sequences, no cache, one function for each part, written from the
formulas of the reference (cited as ``path:line`` of Azimml/shrike's tree).
It shares no code with the product path: it parses config.json and reads
model.safetensors by itself and uses only torch tensor arithmetic.

Everything is computed in float64 by default so that it can judge the float32
engine; ``dtype=torch.float32`` gives the reference's own float32 arithmetic.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path

import torch
from safetensors import safe_open


@dataclass
class PlainConfig:
    """The keys the reference reads from config.json (shrike/models/qwen.py:32-49)."""

    hidden_size: int
    intermediate_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    vocab_size: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    # Not in the reference: layers from `first_window_layer` on see only the
    # last `window` keys (query included). None = every key, as the reference.
    window: int | None = None
    first_window_layer: int = 0

    @classmethod
    def from_dir(cls, model_dir: str | Path) -> "PlainConfig":
        raw = json.loads((Path(model_dir) / "config.json").read_text())
        hidden, heads = raw["hidden_size"], raw["num_attention_heads"]
        window = None
        if raw.get("use_sliding_window") and raw.get("sliding_window"):
            window = int(raw["sliding_window"])
        return cls(
            hidden_size=hidden,
            intermediate_size=raw["intermediate_size"],
            num_layers=raw["num_hidden_layers"],
            num_heads=heads,
            num_kv_heads=raw["num_key_value_heads"],
            # qwen.py:38 - absent or falsy head_dim falls back to hidden // heads
            head_dim=raw.get("head_dim") or hidden // heads,
            vocab_size=raw["vocab_size"],
            rms_norm_eps=raw["rms_norm_eps"],
            rope_theta=raw["rope_theta"],
            tie_word_embeddings=raw.get("tie_word_embeddings", False),
            window=window,
            first_window_layer=int(raw.get("max_window_layers", 0)) if window else 0,
        )


def read_weights(model_dir: str | Path, dtype=torch.float64) -> dict[str, torch.Tensor]:
    """All tensors of every *.safetensors file, by name (qwen.py:202-212)."""
    out: dict[str, torch.Tensor] = {}
    for shard in sorted(Path(model_dir).glob("*.safetensors")):
        with safe_open(str(shard), framework="pt") as f:
            for name in f.keys():
                out[name] = f.get_tensor(name).to(dtype)
    return out


# --------------------------------------------------------------------------- parts


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x * rsqrt(mean(x^2) + eps) * weight, eps inside the root (qwen.py:70-74)."""
    inv = torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return (x * inv) * weight


def rope_tables(positions: torch.Tensor, head_dim: int, theta: float, dtype=torch.float64):
    """cos, sin of shape [N, head_dim] (qwen.py:80, 84-88).

    inv_freq[i] = 1 / theta**(2i/D); the table is the half table repeated twice
    so that element i and element i + D/2 share one angle.
    The reference forms inv_freq and the angle in float32; the float32 values
    are reproduced here and only then widened, so that both sides take the
    sine of the same number.
    """
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2).float() / head_dim))
    freqs = torch.outer(positions.float(), inv_freq)  # float32 product, as qwen.py:86
    emb = torch.cat((freqs, freqs), dim=-1).to(dtype)
    return emb.cos(), emb.sin()


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """(-x2, x1) for x = (x1, x2) split in halves (qwen.py:91-93)."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x: [N, heads, D]; cos/sin: [N, D] broadcast over heads (qwen.py:96-101)."""
    return x * cos[:, None, :] + rotate_half(x) * sin[:, None, :]


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None):
    """y = x @ weight.T + bias with weight stored [out, in] (torch.nn.Linear)."""
    y = x @ weight.t()
    return y if bias is None else y + bias


def causal_attention(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: int | None = None, first: int = 0
) -> torch.Tensor:
    """q: [N - first, H, D], the queries at positions first .. N-1; k, v:
    [N, Hkv, D] of one whole sequence -> [N - first, H, D].

    Query head h reads KV head h // (H // Hkv) (model_runner.py:129,
    triton_attention.py:43); scores are (q.k) * D**-0.5 (model_runner.py:131);
    a query at position p sees keys j <= p (qwen.py:243-244); softmax over the
    kept keys; output sum_j a_j v_j.  With `window` a query also needs
    p - j < window (not in the reference).
    """
    n, (m, h, d) = k.shape[0], q.shape
    assert m == n - first
    groups = h // k.shape[1]
    out = torch.empty_like(q)
    pos_q, pos_k = torch.arange(first, n), torch.arange(n)
    keep = pos_k[None, :] <= pos_q[:, None]
    if window is not None:
        keep &= (pos_q[:, None] - pos_k[None, :]) < window
    for head in range(h):
        kv = head // groups
        scores = (q[:, head, :] @ k[:, kv, :].t()) * d**-0.5
        scores = scores.masked_fill(~keep, float("-inf"))
        out[:, head, :] = torch.softmax(scores, dim=-1) @ v[:, kv, :]
    return out


def swiglu(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor):
    """down(silu(gate(x)) * up(x)), silu(z) = z * sigmoid(z), no biases (qwen.py:131-136)."""
    g = linear(x, w_gate)
    u = linear(x, w_up)
    return linear(g * torch.sigmoid(g) * u, w_down)


# --------------------------------------------------------------------------- model


def attention_block(cfg: PlainConfig, w: dict, prefix: str, x, cos, sin, window):
    """Projections with bias, rotation of q and k, attention, output projection
    without bias (qwen.py:111-125)."""
    n = x.shape[0]
    q = linear(x, w[f"{prefix}.q_proj.weight"], w[f"{prefix}.q_proj.bias"])
    k = linear(x, w[f"{prefix}.k_proj.weight"], w[f"{prefix}.k_proj.bias"])
    v = linear(x, w[f"{prefix}.v_proj.weight"], w[f"{prefix}.v_proj.bias"])
    q = apply_rope(q.view(n, cfg.num_heads, cfg.head_dim), cos, sin)
    k = apply_rope(k.view(n, cfg.num_kv_heads, cfg.head_dim), cos, sin)
    v = v.view(n, cfg.num_kv_heads, cfg.head_dim)
    o = causal_attention(q, k, v, window)
    return linear(o.reshape(n, -1), w[f"{prefix}.o_proj.weight"])


def decoder_layer(cfg: PlainConfig, w: dict, i: int, x, cos, sin):
    """x + attn(norm(x)); then x + mlp(norm(x)) (qwen.py:147-150)."""
    p = f"model.layers.{i}"
    window = cfg.window if (cfg.window and i >= cfg.first_window_layer) else None
    h = rms_norm(x, w[f"{p}.input_layernorm.weight"], cfg.rms_norm_eps)
    x = x + attention_block(cfg, w, f"{p}.self_attn", h, cos, sin, window)
    h = rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], cfg.rms_norm_eps)
    return x + swiglu(
        h,
        w[f"{p}.mlp.gate_proj.weight"],
        w[f"{p}.mlp.up_proj.weight"],
        w[f"{p}.mlp.down_proj.weight"],
    )


def forward(cfg: PlainConfig, w: dict, token_ids: list[int], first_position: int = 0, rows=None):
    """Logits [N, V] of one whole sequence (qwen.py:160-164, 188-192); with
    `rows`, of those positions only, selected after the final norm as the
    reference does (qwen.py:190-191).

    Embedding lookup without scaling, the layers, the final norm, then the
    output matrix, which is the embedding table when the weights are tied and
    the file has no lm_head.weight (qwen.py:211-212).  `first_position` shifts
    every position; the model only depends on distances.
    """
    dtype = w["model.embed_tokens.weight"].dtype
    ids = torch.tensor(token_ids, dtype=torch.long)
    positions = torch.arange(first_position, first_position + len(token_ids))
    cos, sin = rope_tables(positions, cfg.head_dim, cfg.rope_theta, dtype)
    x = w["model.embed_tokens.weight"][ids]
    for i in range(cfg.num_layers):
        x = decoder_layer(cfg, w, i, x, cos, sin)
    x = rms_norm(x, w["model.norm.weight"], cfg.rms_norm_eps)
    if rows is not None:
        x = x[torch.tensor(list(rows), dtype=torch.long)]
    head = w.get("lm_head.weight")
    if head is None:
        if not cfg.tie_word_embeddings:
            raise KeyError("lm_head.weight is absent and the embeddings are not tied")
        head = w["model.embed_tokens.weight"]
    return linear(x, head)


class PlainModel:
    """A model folder read once; `logits(ids)` and greedy generation over it."""

    def __init__(self, model_dir: str | Path, dtype=torch.float64):
        self.cfg = PlainConfig.from_dir(model_dir)
        self.weights = read_weights(model_dir, dtype)

    def logits(self, token_ids: list[int], rows=None) -> torch.Tensor:
        return forward(self.cfg, self.weights, list(token_ids), rows=rows)

    def greedy(self, prompt: list[int], max_new_tokens: int) -> list[int]:
        """Recompute the whole sequence for every new token; argmax takes the
        lowest index among equal maxima."""
        seq, out = list(prompt), []
        for _ in range(max_new_tokens):
            row = self.logits(seq)[-1]
            tok = int(torch.argmax(row))
            out.append(tok)
            seq.append(tok)
        return out


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """max |got - want| / max |want|: the scale of the logits is the yardstick."""
    want = want.double()
    return float((got.double() - want).abs().max() / want.abs().max().clamp_min(1e-30))


def softmax_sample_reference(logits: torch.Tensor, temperature: float, top_p: float):
    """The weights the reference draws from (sampler.py:20-29): softmax of
    logits/T, sorted descending, kept where the mass before an entry is below
    top_p (the largest is always kept).  Returns (kept token ids, weights)."""
    probs = torch.softmax(logits.double() / temperature, dim=-1)
    sorted_probs, sorted_idx = probs.sort(dim=-1, descending=True, stable=True)
    before = sorted_probs.cumsum(-1) - sorted_probs
    keep = before < top_p
    return sorted_idx[keep], sorted_probs[keep]


__all__ = [
    "PlainConfig",
    "PlainModel",
    "apply_rope",
    "causal_attention",
    "forward",
    "linear",
    "read_weights",
    "rel_err",
    "rms_norm",
    "rope_tables",
    "rotate_half",
    "softmax_sample_reference",
    "swiglu",
]
