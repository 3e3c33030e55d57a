"""The numbers bench.py prices its measurements against, checked against the
sizes of the Qwen2.5-7B shape worked out by hand (CPU)."""

import importlib.util
from pathlib import Path

import shrike_amd.models  # noqa: F401  (registers the architecture)
from shrike_amd.models.qwen2 import Qwen2Config

spec = importlib.util.spec_from_file_location("bench", Path(__file__).resolve().parent.parent / "bench.py")
bench = importlib.util.module_from_spec(spec)
spec.loader.exec_module(bench)


def test_bytes_and_flops_of_the_7b_shape():
    cfg = Qwen2Config.from_dict(bench._shape("7b"))
    per_layer_total, head = bench.matmul_params(cfg)
    # q,k,v: 4608 x 3584; o: 3584 x 3584; gate, up, down: 3 x 18944 x 3584
    assert per_layer_total == 28 * (4608 * 3584 + 3584 * 3584 + 3 * 18944 * 3584) == 28 * 233_046_016
    assert head == 152064 * 3584
    # weights a decode step reads: 14.141 GB in bfloat16
    assert abs(2 * (per_layer_total + head) / 1e9 - 14.141) < 0.001
    # keys and values of one token over 28 layers, 4 kv heads of 128, bfloat16
    assert bench.kv_bytes_per_token(cfg) == 28 * 2 * 4 * 128 * 2 == 57_344
    # a 2,048-token prompt: 26.73 TFLOP in the matrices (the head on one row), 0.84 in causal attention
    flops = bench.prefill_flops(cfg, 2048)
    assert abs(flops / 1e12 - 27.57) < 0.02
    attention = 4.0 * 128 * 28 * 28 * 2048 * 2049 / 2
    assert abs(attention / 1e12 - 0.84) < 0.01 and flops > attention


def test_the_other_shapes_are_the_presets_that_the_package_ships():
    from shrike_amd.config.presets import load_preset, preset_names

    assert preset_names() == ["qwen2.5-0.5b", "qwen2.5-14b", "qwen2.5-32b", "qwen2.5-7b"]
    for name, layers, hidden in (("14b", 48, 5120), ("32b", 64, 5120)):
        cfg = Qwen2Config.from_dict(bench._shape(name))
        assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads) == (layers, hidden, 40, 8)
        assert cfg.vocab_size == 152064 and cfg.head_dim == 128
    small = Qwen2Config.from_dict(load_preset("Qwen2.5-0.5B"))
    assert (small.hidden_size, small.num_attention_heads, small.num_key_value_heads, small.head_dim) == (896, 14, 2, 64)
    assert small.tie_word_embeddings and small.vocab_size == 151936
