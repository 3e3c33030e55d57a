"""Weight files: binding by name, the one error that lists everything, random weights (CPU)."""

import json

import pytest
import torch
from safetensors.torch import load_file, save_file

import shrike_amd.models  # noqa: F401
from shrike_amd.config import load_model_config
from shrike_amd.models import DecoderModel
from shrike_amd.weights import WeightError, load_weights, random_tensors, write_model_folder

from .tiny import TINY_A, TINY_B, make_model_dir


def model_for(path):
    _, spec = load_model_config(path)
    return DecoderModel(spec)


def test_folder_has_config_and_safetensors_and_loads(tmp_path):
    path = make_model_dir("B", tmp_path)
    assert sorted(p.name for p in path.iterdir()) == ["config.json", "model.safetensors"]
    model = model_for(path)
    tensors = load_weights(path, model.params(), torch.bfloat16, "cpu")
    assert tensors["model.layers.0.self_attn.q_proj.weight"].dtype == torch.bfloat16
    assert tensors["model.layers.0.self_attn.q_proj.weight"].shape == (4 * 32, 128)
    # vectors that enter float32 arithmetic stay float32
    assert tensors["model.norm.weight"].dtype == torch.float32
    assert tensors["model.layers.2.self_attn.k_proj.bias"].dtype == torch.float32
    assert tensors["lm_head.weight"].shape == (503, 128)


def test_tied_folder_has_no_output_matrix(tmp_path):
    path = make_model_dir("A", tmp_path)
    names = set(load_file(str(path / "model.safetensors")))
    assert "lm_head.weight" not in names and "model.embed_tokens.weight" in names
    tensors = load_weights(path, model_for(path).params(), torch.float32, "cpu")
    assert "lm_head.weight" not in tensors


def test_same_seed_same_weights_other_seed_other_weights(tmp_path):
    a = write_model_folder(dict(TINY_A), tmp_path / "a", seed=5)
    b = write_model_folder(dict(TINY_A), tmp_path / "b", seed=5)
    c = write_model_folder(dict(TINY_A), tmp_path / "c", seed=6)
    ta, tb, tc = (load_file(str(p / "model.safetensors")) for p in (a, b, c))
    assert all(torch.equal(ta[k], tb[k]) for k in ta)
    assert not torch.equal(ta["model.norm.weight"], tc["model.norm.weight"])


def test_distributions(tmp_path):
    path = write_model_folder(dict(TINY_B), tmp_path / "m", seed=1)
    t = load_file(str(path / "model.safetensors"))
    w = t["model.layers.1.mlp.gate_proj.weight"].float()
    assert abs(w.std().item() - 0.02) < 0.002 and abs(w.mean().item()) < 0.002
    n = t["model.layers.1.input_layernorm.weight"].float()
    assert abs(n.mean().item() - 1.0) < 0.05 and 0.05 < n.std().item() < 0.15


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    path = make_model_dir("A", tmp_path)
    tensors = load_file(str(path / "model.safetensors"))
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.extra.weight"] = torch.zeros(3)
    tensors["model.layers.0.self_attn.k_proj.bias"] = torch.zeros(7)
    save_file(tensors, str(path / "model.safetensors"))
    with pytest.raises(WeightError) as info:
        load_weights(path, model_for(path).params(), torch.float32, "cpu")
    err = info.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.extra.weight"]
    assert [w[0] for w in err.wrong_shape] == ["model.layers.0.self_attn.k_proj.bias"]
    text = str(err)
    for needle in ("missing (2)", "unexpected (1)", "wrong shape (1)", "is [7], expected [32]"):
        assert needle in text


def test_untied_model_needs_its_output_matrix(tmp_path):
    path = make_model_dir("B", tmp_path)
    tensors = load_file(str(path / "model.safetensors"))
    del tensors["lm_head.weight"]
    save_file(tensors, str(path / "model.safetensors"))
    with pytest.raises(WeightError, match="lm_head.weight"):
        load_weights(path, model_for(path).params(), torch.float32, "cpu")


def test_no_weight_files(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    with pytest.raises(FileNotFoundError, match="safetensors"):
        load_weights(tmp_path, model_for(tmp_path).params(), torch.float32, "cpu")


def test_stored_dtype_and_held_dtype(tmp_path):
    path = make_model_dir("A", tmp_path, dtype="bfloat16")
    stored = load_file(str(path / "model.safetensors"))
    assert all(t.dtype == torch.bfloat16 for t in stored.values())
    held = load_weights(path, model_for(path).params(), torch.float32, "cpu")
    assert held["model.embed_tokens.weight"].dtype == torch.float32
    # widening bfloat16 is exact
    assert torch.equal(held["model.embed_tokens.weight"], stored["model.embed_tokens.weight"].float())


def test_integer_tables_are_held_as_int32():
    from shrike_amd.parts.base import ParamSpec
    from shrike_amd.weights.loader import convert

    t = convert(torch.arange(5, dtype=torch.int64), ParamSpec("t", (5,)), torch.bfloat16)
    assert t.dtype == torch.int32


def test_random_tensors_do_not_depend_on_their_neighbours(tmp_path):
    path = make_model_dir("A", tmp_path)
    params = model_for(path).params()
    full = random_tensors(params, 3, torch.float32)
    part = random_tensors(params[5:9], 3, torch.float32)
    assert all(torch.equal(full[k], part[k]) for k in part)
