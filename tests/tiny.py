"""Tiny configurations of the architecture for tests.  A and B differ in every
size and option; C has an explicit head_dim (heads * head_dim != hidden) and a
window on its later layers; D has a head size that the matrix-instruction
attention kernels take (64) and a window on all layers but the first."""

from __future__ import annotations

import json
import tempfile
from pathlib import Path

TINY_A = {
    "architectures": ["Qwen2ForCausalLM"],
    "model_type": "qwen2",
    "hidden_size": 64,
    "intermediate_size": 172,
    "num_hidden_layers": 2,
    "num_attention_heads": 4,
    "num_key_value_heads": 2,
    "vocab_size": 256,
    "rope_theta": 10000.0,
    "rms_norm_eps": 1e-6,
    "tie_word_embeddings": True,
    "max_position_embeddings": 128,
    "eos_token_id": 255,
    "torch_dtype": "float32",
    "use_sliding_window": False,
    "sliding_window": 32,
}

TINY_B = {
    "architectures": ["Qwen2ForCausalLM"],
    "model_type": "qwen2",
    "hidden_size": 128,
    "intermediate_size": 352,
    "num_hidden_layers": 3,
    "num_attention_heads": 4,
    "num_key_value_heads": 1,
    "head_dim": 32,
    "vocab_size": 503,
    "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False,
    "max_position_embeddings": 256,
    "eos_token_id": [501, 502],
    "torch_dtype": "float32",
}

TINY_C = {
    "architectures": ["Qwen2ForCausalLM"],
    "hidden_size": 96,
    "intermediate_size": 200,
    "num_hidden_layers": 4,
    "num_attention_heads": 6,
    "num_key_value_heads": 3,
    "head_dim": 48,
    "vocab_size": 311,
    "rope_theta": 50000.0,
    "rms_norm_eps": 3e-6,
    "tie_word_embeddings": False,
    "torch_dtype": "float32",
    "use_sliding_window": True,
    "sliding_window": 24,
    "max_window_layers": 2,
}

TINY_D = {
    "architectures": ["Qwen2ForCausalLM"],
    "hidden_size": 160,
    "intermediate_size": 296,
    "num_hidden_layers": 3,
    "num_attention_heads": 4,
    "num_key_value_heads": 2,
    "head_dim": 64,
    "vocab_size": 389,
    "rope_theta": 200000.0,
    "rms_norm_eps": 2e-5,
    "tie_word_embeddings": False,
    "torch_dtype": "float32",
    "use_sliding_window": True,
    "sliding_window": 40,
    "max_window_layers": 1,
}

# A with an output matrix of its own.  With "unit" weights the tied table is N(0, 1), and
# a token's logit for itself (its embedding's squared length) towers over all others:
# greedy generation of tied A says little about the layers in between, so tests of
# generated tokens take this variant; logits are compared on A itself.
TINY_A_UNTIED = dict(TINY_A, tie_word_embeddings=False)

CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "A_untied": TINY_A_UNTIED}
SEEDS = {"A": 11, "B": 23, "C": 37, "D": 41, "A_untied": 11}
PAGE_SIZES = {"A": 4, "B": 8, "C": 16, "D": 16, "A_untied": 4}


def make_model_dir(name: str, root=None, dtype: str = "float32", mode: str = "reference") -> Path:
    """Writes the tiny model `name` with seeded random weights into a fresh
    temporary folder (or `root`/name) and returns the folder."""
    from shrike_amd.weights import write_model_folder

    if root is None:
        root = tempfile.mkdtemp(prefix="shrike_tiny_")
    path = Path(root) / f"tiny_{name}_{dtype}_{mode}"
    if not (path / "model.safetensors").is_file():
        write_model_folder(dict(CONFIGS[name]), path, seed=SEEDS[name], dtype=dtype, mode=mode)
    return path


def read_config(path) -> dict:
    return json.loads((Path(path) / "config.json").read_text())
