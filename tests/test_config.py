"""Configuration and registry (CPU)."""

import importlib
import json

import pytest

import shrike_amd.models  # noqa: F401  registers the architecture
from shrike_amd.config import (
    ConfigError,
    EngineConfig,
    architectures,
    get_architecture,
    load_model_config,
)
from shrike_amd.models.qwen2 import Qwen2Config, build_spec

from .tiny import CONFIGS, TINY_A, TINY_B, TINY_C


def write(tmp_path, raw):
    (tmp_path / "config.json").write_text(json.dumps(raw))
    return tmp_path


def test_registry_maps_architecture_name_to_model():
    assert "Qwen2ForCausalLM" in architectures()
    arch = get_architecture("Qwen2ForCausalLM")
    assert arch.config_cls is Qwen2Config
    with pytest.raises(ConfigError, match="unknown architecture"):
        get_architecture("NoSuchModel")


def test_config_reads_the_keys_of_config_json(tmp_path):
    cfg, spec = load_model_config(write(tmp_path, TINY_B))
    assert (cfg.hidden_size, cfg.intermediate_size, cfg.num_hidden_layers) == (128, 352, 3)
    assert (cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim) == (4, 1, 32)
    assert cfg.vocab_size == 503 and cfg.rope_theta == 1e6 and cfg.rms_norm_eps == 1e-5
    assert cfg.eos_token_ids == (501, 502) and not cfg.tie_word_embeddings
    assert len(spec.blocks) == 3 and spec.vocab_size == 503
    assert spec.blocks[0].mixer.scale == 32**-0.5
    assert spec.blocks[0].mixer.position.theta == 1e6
    assert spec.blocks[0].mixer_norm.eps == 1e-5


def test_head_dim_falls_back_to_hidden_over_heads(tmp_path):
    # shrike/models/qwen.py:38
    cfg, _ = load_model_config(write(tmp_path, TINY_A))
    assert cfg.head_dim == 64 // 4
    raw = dict(TINY_A, head_dim=0)
    assert Qwen2Config.from_dict(raw).head_dim == 16
    assert Qwen2Config.from_dict(TINY_C).head_dim == 48  # heads * head_dim != hidden


def test_eos_may_be_int_list_or_absent():
    assert Qwen2Config.from_dict(TINY_A).eos_token_ids == (255,)
    raw = {k: v for k, v in TINY_A.items() if k != "eos_token_id"}
    assert Qwen2Config.from_dict(raw).eos_token_ids == ()


def test_model_type_stands_in_for_architectures(tmp_path):
    raw = {k: v for k, v in TINY_A.items() if k != "architectures"}
    cfg, _ = load_model_config(write(tmp_path, raw))
    assert cfg.hidden_size == 64


@pytest.mark.parametrize(
    "change, match",
    [
        ({"hidden_size": None}, "hidden_size"),
        ({"num_key_value_heads": 3}, "multiple"),
        ({"rms_norm_eps": 0.0}, "rms_norm_eps"),
        ({"vocab_size": 0}, "vocab_size"),
        ({"head_dim": 15}, "even"),
        ({"hidden_act": "gelu"}, "hidden_act"),
        ({"rope_scaling": {"type": "yarn"}}, "rope_scaling"),
        ({"torch_dtype": "float16"}, "dtype"),
        ({"architectures": ["Mystery"]}, "unknown architecture"),
        ({"num_hidden_layers": "2"}, "integer"),
    ],
)
def test_bad_values_are_refused(tmp_path, change, match):
    raw = dict(TINY_A)
    raw.update(change)
    raw = {k: v for k, v in raw.items() if v is not None}
    with pytest.raises(ConfigError, match=match):
        load_model_config(write(tmp_path, raw))


def test_missing_config_json(tmp_path):
    with pytest.raises(FileNotFoundError, match="config.json"):
        load_model_config(tmp_path)


def test_window_is_ignored_unless_switched_on():
    spec = build_spec(Qwen2Config.from_dict(TINY_A))  # sliding_window given, use_sliding_window false
    assert all(b.mixer.window is None for b in spec.blocks)
    spec = build_spec(Qwen2Config.from_dict(TINY_C))
    assert [b.mixer.window for b in spec.blocks] == [None, None, 24, 24]


def test_to_dict_round_trips():
    for raw in CONFIGS.values():
        cfg = Qwen2Config.from_dict(raw)
        assert Qwen2Config.from_dict(cfg.to_dict()) == cfg


def test_no_size_stands_in_code():
    """Two configurations that differ in every size give specs that differ in every size."""
    a, b = (build_spec(Qwen2Config.from_dict(c)) for c in (TINY_A, TINY_B))
    ma, mb = a.blocks[0].mixer, b.blocks[0].mixer
    for x, y in [
        (a.hidden_size, b.hidden_size), (a.vocab_size, b.vocab_size), (len(a.blocks), len(b.blocks)),
        (ma.num_kv_heads, mb.num_kv_heads), (ma.head_dim, mb.head_dim), (ma.scale, mb.scale),
        (ma.position.theta, mb.position.theta), (a.final_norm.eps, b.final_norm.eps),
        (a.blocks[0].ffn.intermediate_size, b.blocks[0].ffn.intermediate_size),
        (a.tie_word_embeddings, b.tie_word_embeddings),
    ]:
        assert x != y


def test_schedule_defaults_to_every_block_once_and_is_checked():
    from dataclasses import replace

    from shrike_amd.config import ScheduleEntry

    spec = build_spec(Qwen2Config.from_dict(TINY_A))
    assert [e.block for e in spec.schedule] == [0, 1]
    twice = replace(spec, schedule=(ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0, cache_of=0)))
    assert len(twice.schedule) == 3
    with pytest.raises(ValueError, match="earlier"):
        replace(spec, schedule=(ScheduleEntry(0, cache_of=1), ScheduleEntry(1)))
    with pytest.raises(ValueError, match="does not exist"):
        replace(spec, schedule=(ScheduleEntry(5),))


def test_engine_config_validation():
    EngineConfig(block_size=4, num_kv_blocks=3, dtype="fp32")
    for bad in ({"block_size": 0}, {"gpu_mem_util": 0.0}, {"max_tokens_per_step": 0},
                {"max_running": 0}, {"num_kv_blocks": 0}, {"dtype": "int8"}):
        with pytest.raises(ValueError):
            EngineConfig(**bad)


def test_default_model_dir_env_override(monkeypatch):
    # shrike/config.py:29
    import shrike_amd.config.registry as reg

    monkeypatch.setenv("SHRIKE_MODEL_DIR", "/somewhere/else")
    importlib.reload(reg)
    assert reg.DEFAULT_MODEL_DIR == "/somewhere/else"
    monkeypatch.delenv("SHRIKE_MODEL_DIR")
    importlib.reload(reg)
    import shrike_amd.models.qwen2 as q

    importlib.reload(q)  # the reload emptied the registry; register again


def test_plugins_named_in_the_environment_are_loaded_for_an_unknown_architecture(tmp_path, monkeypatch):
    """SHRIKE_AMD_PLUGINS: how a program started from the command line learns an
    architecture that is defined outside the package."""
    import sys

    from shrike_amd.config import registry

    (tmp_path / "my_plugin.py").write_text(
        "from shrike_amd.config.registry import register_architecture\n"
        "from shrike_amd.models.qwen2 import Qwen2Config, build_spec\n"
        "def install():\n"
        "    register_architecture('PluggedInForCausalLM', Qwen2Config, build_spec)\n")
    monkeypatch.syspath_prepend(str(tmp_path))
    monkeypatch.setattr(registry, "_plugins_loaded", False)
    monkeypatch.setenv("SHRIKE_AMD_PLUGINS", "my_plugin:install")
    with pytest.raises(registry.ConfigError, match="unknown architecture"):
        registry.get_architecture("NobodyForCausalLM")  # loads the plugins, still unknown
    assert registry.get_architecture("PluggedInForCausalLM").config_cls.__name__ == "Qwen2Config"
    registry._ARCHITECTURES.pop("PluggedInForCausalLM")
    sys.modules.pop("my_plugin", None)
    monkeypatch.setattr(registry, "_plugins_loaded", False)
    monkeypatch.setenv("SHRIKE_AMD_PLUGINS", "no_such_module_anywhere")
    with pytest.raises(registry.ConfigError, match="cannot load 'no_such_module_anywhere'"):
        registry.get_architecture("NobodyForCausalLM")
