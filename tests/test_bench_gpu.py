"""bench.py's own runs on a tiny model: the offline run hands out what it was asked
for, and a decode run counts its tokens (the numbers themselves are the bench's)."""

import importlib.util
from pathlib import Path

import pytest

from .tiny import CONFIGS

pytestmark = pytest.mark.gpu

spec_ = importlib.util.spec_from_file_location("bench", Path(__file__).resolve().parent.parent / "bench.py")
bench = importlib.util.module_from_spec(spec_)
spec_.loader.exec_module(bench)


def test_offline_run_and_decode_run_on_a_tiny_model():
    import shrike_amd.models  # noqa: F401
    from shrike_amd.models.qwen2 import Qwen2Config, build_spec

    cfg = Qwen2Config.from_dict(dict(CONFIGS["B"], torch_dtype="bfloat16"))
    spec = build_spec(cfg)
    got = bench.run_offline(cfg, spec, 12, seed=3)
    assert got["tokens"] >= 12 * 32 and got["tok_s"] > 0 and got["preemptions"] == 0
    assert got["steps"] >= 32 and got["token_budget"] == 512 and got["page_size"] == 16
    engine = bench.make_engine(cfg, spec, 4, seed=1)
    run = bench.run_decode(engine, cfg, 4, steps=10, warmup=2, seed=5, prompt_len=40)
    assert run["context_end"] - run["context_start"] == 10 and run["tok_s"] > 0
    sampled = bench.run_decode(engine, cfg, 4, steps=10, warmup=2, seed=6, prompt_len=40, temperature=0.8, top_p=0.9)
    assert sampled["context_end"] - sampled["context_start"] == 10


def test_products_mode_times_every_product_of_a_layer_both_ways():
    import shrike_amd.models  # noqa: F401
    from shrike_amd.models.qwen2 import Qwen2Config

    cfg = Qwen2Config.from_dict(dict(CONFIGS["D"], torch_dtype="bfloat16"))
    got = bench.run_products(cfg, [8, 200])
    assert set(got) == {f"{name}_n{n}" for n in (8, 200) for name in ("qkv", "o", "gate_up", "down")} | {"lm_head_n8"}
    for entry in got.values():
        assert entry["own_us"] > 0 and entry["library_us"] > 0 and entry["k_shares"] >= 1
