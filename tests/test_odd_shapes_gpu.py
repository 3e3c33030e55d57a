"""Configurations at the edges of what the kernels take: a width that is no
multiple of 8, heads * head_dim != hidden, 32 query heads on one key/value
head, 16 and 17 on one, head sizes 16, 80, 96, 160 and 256, a window, vocabularies
that are no power of two, tied weights; each in float32 and bfloat16, with pages of 16 (MFMA attention where
the shape allows) and of 4 (general kernel)."""

import tempfile

import pytest
import torch

from .plain.model import PlainModel, rel_err

pytestmark = pytest.mark.gpu

BASE = {"architectures": ["Qwen2ForCausalLM"], "rope_theta": 1e4, "rms_norm_eps": 1e-5,
        "tie_word_embeddings": False, "torch_dtype": "bfloat16"}
CASES = {
    "width100_heads5x16": dict(hidden_size=100, intermediate_size=54, num_hidden_layers=2,
                               num_attention_heads=5, num_key_value_heads=5, head_dim=16, vocab_size=77),
    "group32": dict(hidden_size=96, intermediate_size=130, num_hidden_layers=2, num_attention_heads=32,
                    num_key_value_heads=1, head_dim=32, vocab_size=1001),
    "head80": dict(hidden_size=72, intermediate_size=99, num_hidden_layers=1, num_attention_heads=3,
                   num_key_value_heads=1, head_dim=80, vocab_size=300),
    "head256_tied": dict(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=2,
                         num_key_value_heads=2, head_dim=256, vocab_size=999, tie_word_embeddings=True),
    "width130_group3": dict(hidden_size=130, intermediate_size=70, num_hidden_layers=1,
                            num_attention_heads=9, num_key_value_heads=3, head_dim=64, vocab_size=513),
    # 16 query heads on a key/value head is the most the matrix-instruction kernels take; a
    # head size above 128 leaves prompt portions to the kernel that works tile by tile
    "head160_group16": dict(hidden_size=88, intermediate_size=120, num_hidden_layers=2,
                            num_attention_heads=16, num_key_value_heads=1, head_dim=160, vocab_size=4099),
    # one head more than that: the general kernel serves it
    "group17": dict(hidden_size=68, intermediate_size=80, num_hidden_layers=1, num_attention_heads=17,
                    num_key_value_heads=1, head_dim=32, vocab_size=211),
    # seven heads per group of 96 with a window from the second layer on
    "head96_group7_window": dict(hidden_size=120, intermediate_size=200, num_hidden_layers=3,
                                 num_attention_heads=14, num_key_value_heads=2, head_dim=96, vocab_size=8200,
                                 use_sliding_window=True, sliding_window=33, max_window_layers=1),
}


@pytest.mark.parametrize("name", list(CASES))
def test_odd_shapes(name):
    from shrike_amd.cache import CacheManager
    from shrike_amd.engine.loading import load_model
    from shrike_amd.engine.runner import ModelRunner, StepEntry
    from shrike_amd.weights import write_model_folder

    case = CASES[name]
    with tempfile.TemporaryDirectory() as root:
        model_dir = write_model_folder(dict(BASE, **case), root + "/m", seed=len(name), mode="unit")
        plain = PlainModel(model_dir)
        ids = torch.randint(0, case["vocab_size"], (90,), generator=torch.Generator().manual_seed(1)).tolist()
        want = plain.logits(ids)
        for dtype, tol in (("float32", 1e-4), ("bfloat16", 1.5e-2)):
            model, rt, _ = load_model(model_dir, dtype)
            for page_size in (16, 4):
                cache = CacheManager(model.cache_specs(), page_size, 64, enable_prefix_caching=False)
                cache.allocate(rt.dtype, rt.device)
                runner = ModelRunner(model, cache, rt)
                seq, outs, p = cache.new_sequence(), [], 0
                for n in (70, 3, 1, 1, 1, 14):
                    cache.append(seq, p, n)
                    outs.append(runner.step([StepEntry(seq, ids[p : p + n], p, list(range(n)))]).cpu().clone())
                    p += n
                    cache.trim(seq, p)
                err = rel_err(torch.cat(outs), want)
                assert err <= tol, f"{name} {dtype} page {page_size}: rel err {err:.2e}"
                cache.free(seq)


def test_head_sizes_beyond_256_are_refused():
    from shrike_amd.config import AttentionSpec, RotarySpec
    from shrike_amd.engine.runtime import Runtime
    from shrike_amd.parts import build_part

    spec = AttentionSpec(num_heads=2, num_kv_heads=1, head_dim=272, qkv_bias=True, out_bias=False,
                         scale=272**-0.5, position=RotarySpec(theta=1e4, rotary_dim=272))
    with pytest.raises(ValueError, match="head_dim 272"):
        build_part("mixer", spec, 64, "m").check(Runtime("cuda:0", torch.bfloat16))
