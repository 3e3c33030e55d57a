"""A whole toy architecture that exists only in this file: a config.json with
keys of its own, a block of its own (feed-forward first, then the mixer), other
tensor names, attention with an output bias, a rotation of part of each head
and a scale that is not head_size**-0.5, and a schedule that runs the last
layer twice (the second run with a cache of its own).  It is registered by
name; the framework's writer makes its model folder, the Python entry point
generates with it, bin/trace_run replays it (told of this module by
SHRIKE_AMD_PLUGINS), and a computation written out here with the plain
functions checks both.  It is no model of anyone's: it
shows that an architecture is added without a change to the framework's files."""

import json
import os
import subprocess
from dataclasses import dataclass
from pathlib import Path
from typing import ClassVar

import numpy as np
import pytest
import torch

from .plain import model as plain

pytestmark = pytest.mark.gpu

ARCH = "ToyFfnFirstForCausalLM"
CONFIG = {
    "architectures": [ARCH],
    "width": 80,
    "depth": 3,
    "heads": 5,
    "groups": 1,
    "head_size": 32,
    "rotated": 16,
    "inner": 136,
    "tokens": 211,
    "eps": 2e-5,
    "theta": 3000.0,
    "score_scale": 0.2,
    "end_token": 210,
    "stored_as": "float32",
}


@dataclass(frozen=True)
class FfnFirstBlockSpec:
    """x += ffn(ffn_norm(x)); x += mixer(mixer_norm(x))."""

    kind: ClassVar[str] = "toy_ffn_first"
    name: str
    mixer: object
    ffn: object
    mixer_norm: object
    ffn_norm: object


@dataclass(frozen=True)
class ToyConfig:
    raw: dict

    @classmethod
    def from_dict(cls, raw: dict) -> "ToyConfig":
        missing = [k for k in CONFIG if k not in raw]
        if missing:
            from shrike_amd.config.registry import ConfigError

            raise ConfigError(f"config.json lacks {missing}")
        return cls(dict(raw))


def define():
    """Registers the block and the architecture (once per process)."""
    from shrike_amd.config.registry import architectures, register_architecture
    from shrike_amd.config.specs import (AttentionSpec, ModelSpec, RMSNormSpec, RotarySpec, ScheduleEntry,
                                         SwiGLUSpec)
    from shrike_amd.parts.base import Block, build_part, register_block

    if ARCH in architectures():
        return

    class FfnFirstBlock(Block):
        def __init__(self, spec, width, name):
            super().__init__(spec, width, name)
            self.ffn_norm = build_part("norm", spec.ffn_norm, width, f"{name}.pre_ff")
            self.ffn = build_part("ffn", spec.ffn, width, f"{name}.ff")
            self.mixer_norm = build_part("norm", spec.mixer_norm, width, f"{name}.pre_mix")
            self.mixer = build_part("mixer", spec.mixer, width, f"{name}.mix")
            self.parts = (self.ffn_norm, self.ffn, self.mixer_norm, self.mixer)

        def params(self):
            return [p for part in self.parts for p in part.params()]

        def check(self, runtime):
            for part in self.parts:
                part.check(runtime)

        def load(self, tensors, runtime):
            for part in self.parts:
                part.load(tensors, runtime)

        def forward(self, ctx, hidden, cache):
            hidden.pending = self.ffn.forward(ctx, self.ffn_norm.forward(ctx, hidden))
            hidden.pending = self.mixer.forward(ctx, self.mixer_norm.forward(ctx, hidden), cache)

    register_block(FfnFirstBlockSpec.kind, FfnFirstBlock)

    def build_spec(cfg: ToyConfig) -> ModelSpec:
        c = cfg.raw
        norm = RMSNormSpec(eps=c["eps"])
        mixer = AttentionSpec(num_heads=c["heads"], num_kv_heads=c["groups"], head_dim=c["head_size"],
                              qkv_bias=False, out_bias=True, scale=c["score_scale"],
                              position=RotarySpec(theta=c["theta"], rotary_dim=c["rotated"]))
        blocks = tuple(FfnFirstBlockSpec(f"body.{i}", mixer, SwiGLUSpec(c["inner"]), norm, norm)
                       for i in range(c["depth"]))
        # every layer once, the last one a second time
        schedule = tuple(ScheduleEntry(i) for i in range(c["depth"])) + (ScheduleEntry(c["depth"] - 1),)
        return ModelSpec(architecture=ARCH, hidden_size=c["width"], vocab_size=c["tokens"], blocks=blocks,
                         final_norm=norm, tie_word_embeddings=True, schedule=schedule, embed_name="table",
                         final_norm_name="last_norm", eos_token_ids=(c["end_token"],),
                         stored_dtype=c["stored_as"])

    register_architecture(ARCH, ToyConfig, build_spec)


def plain_logits(weights: dict, ids: list[int]) -> torch.Tensor:
    """The toy model written out with the plain functions, whole sequence, float64."""
    c = CONFIG
    w = {k: v.double() for k, v in weights.items()}
    n, h, g, d, r = len(ids), c["heads"], c["groups"], c["head_size"], c["rotated"]
    cos, sin = plain.rope_tables(torch.arange(n), r, c["theta"])
    x = w["table.weight"][torch.tensor(ids)]

    def rotate(t):  # the first `rotated` elements of every head, pairs (i, i + rotated/2)
        return torch.cat([plain.apply_rope(t[..., :r], cos, sin), t[..., r:]], dim=-1)

    def layer(x, i):
        p = f"body.{i}"
        x = x + plain.swiglu(plain.rms_norm(x, w[f"{p}.pre_ff.weight"], c["eps"]), w[f"{p}.ff.gate_proj.weight"],
                             w[f"{p}.ff.up_proj.weight"], w[f"{p}.ff.down_proj.weight"])
        y = plain.rms_norm(x, w[f"{p}.pre_mix.weight"], c["eps"])
        q = plain.linear(y, w[f"{p}.mix.q_proj.weight"]).view(n, h, d)
        k = plain.linear(y, w[f"{p}.mix.k_proj.weight"]).view(n, g, d)
        v = plain.linear(y, w[f"{p}.mix.v_proj.weight"]).view(n, g, d)
        # causal_attention scales by d**-0.5: fold the toy's own scale into the queries
        a = plain.causal_attention(rotate(q) * (c["score_scale"] / d**-0.5), rotate(k), v)
        return x + plain.linear(a.reshape(n, h * d), w[f"{p}.mix.o_proj.weight"], w[f"{p}.mix.o_proj.bias"])

    for i in list(range(c["depth"])) + [c["depth"] - 1]:
        x = layer(x, i)
    return plain.linear(plain.rms_norm(x, w["last_norm.weight"], c["eps"]), w["table.weight"])


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    from safetensors.torch import load_file

    from shrike_amd.weights import write_model_folder

    define()
    folder = write_model_folder(dict(CONFIG), tmp_path_factory.mktemp("toy") / "m", seed=4, mode="unit")
    return folder, load_file(str(folder / "model.safetensors"))


def test_the_writer_and_the_loader_know_the_toy_by_its_config_alone(toy):
    folder, weights = toy
    assert json.loads((folder / "config.json").read_text())["architectures"] == [ARCH]
    assert "body.2.mix.o_proj.bias" in weights and "body.0.ff.down_proj.weight" in weights
    assert "lm_head.weight" not in weights and weights["table.weight"].shape == (211, 80)
    from shrike_amd.engine.loading import load_model

    model, _, _ = load_model(folder, "float32")
    assert len(model.cache_specs()) == 4 and all(s is not None for s in model.cache_specs())


@pytest.mark.parametrize("dtype, tol", [("float32", 1e-4), ("bfloat16", 1.5e-2)])
def test_the_toy_steps_and_generates_like_its_plain_form(toy, dtype, tol):
    from shrike_amd import LLM, SamplingParams

    folder, weights = toy
    g = torch.Generator().manual_seed(2)
    prompts = [torch.randint(0, 210, (n,), generator=g).tolist() for n in (3, 41, 18)]
    llm = LLM(str(folder), dtype=dtype, block_size=16, num_kv_blocks=24, max_tokens_per_step=16)
    outs = llm.generate(prompts, SamplingParams(max_new_tokens=9, ignore_eos=True), chat=False)
    for prompt, new in zip(prompts, outs):
        assert len(new) == 9
        seq = list(prompt)
        for tok in new:  # each token is the plain form's choice, unless that was a near-tie in bfloat16
            row = plain_logits(weights, seq)[-1]
            if int(row.argmax()) != tok:
                top2 = row.topk(2).values
                assert dtype == "bfloat16" and float(top2[0] - top2[1]) < 0.03 * float(row.abs().max())
            seq.append(tok)
    # and the logits themselves, through the step function, portions beside a single token
    from shrike_amd.cache import CacheManager
    from shrike_amd.engine.loading import load_model
    from shrike_amd.engine.runner import ModelRunner, StepEntry

    model, rt, _ = load_model(folder, dtype)
    cache = CacheManager(model.cache_specs(), 16, 12, enable_prefix_caching=False)
    cache.allocate(rt.dtype, rt.device)
    runner = ModelRunner(model, cache, rt)
    ids = prompts[1]
    want = plain_logits(weights, ids)
    seq, rows, p = cache.new_sequence(), [], 0
    for n in (17, 2, 21, 1):
        cache.append(seq, p, n)
        rows.append(runner.step([StepEntry(seq, ids[p : p + n], p, list(range(n)))]).cpu().double())
        p += n
    assert plain.rel_err(torch.cat(rows), want) <= tol
    cache.free(seq)
    cache.check([])


def test_the_toy_through_trace_run(toy, tmp_path):
    """bin/trace_run is another process: SHRIKE_AMD_PLUGINS names this module's
    define(), which the registry calls when config.json names an architecture it
    does not know."""
    folder, weights = toy
    repo = Path(__file__).resolve().parent.parent
    ids = torch.randint(0, 210, (30,), generator=torch.Generator().manual_seed(6)).tolist()
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": ids[:19], "want": [0, 18]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": ids[19:29], "want": [9]}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": ids[29:], "want": [0]}], "end": ["a"]},
    ]
    out = tmp_path / "out"
    env = dict(os.environ, SHRIKE_AMD_PLUGINS="tests.test_toy_architecture_gpu:define",
               PYTHONPATH=os.pathsep.join(filter(None, [str(repo), os.environ.get("PYTHONPATH")])))
    proc = subprocess.run(
        [str(repo / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32", "--out", str(out),
         "--max-tokens", "64"],
        input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300, env=env)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    want = plain_logits(weights, ids)
    got = np.concatenate([np.fromfile(out / f"{s}.f32", dtype="<f4").reshape(-1, 211) for s in range(3)])
    assert plain.rel_err(torch.from_numpy(got).double(), want[[0, 18, 28, 29]]) <= 1e-4
