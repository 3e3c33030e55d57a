"""bin/trace_run against the plain implementation: the same requests whole,
with the last 32 tokens one by one, in portions of changing size, and mixed
with other requests over so few pages that they are used again; in float32 and
in bfloat16; for four tiny configurations (D runs the matrix-instruction
attention kernels with a window, so that pages a window has passed are given
back, poisoned and handed out again under those kernels and under the graphs
of its single-token steps)."""

import random

import numpy as np
import pytest
import torch

from .plain.model import PlainModel
from .tiny import CONFIGS, PAGE_SIZES, make_model_dir
from .traces import (TraceBuilder, changing_portions, check_pages, last_one_by_one, mixed, read_pages,
                     run_trace, whole)

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [5, 11, 17, 70, 45], "B": [1, 9, 30, 64, 100], "C": [3, 40, 97, 65, 130],
           "D": [6, 50, 130, 90, 200]}
# float32: rel err <= 1e-4 is the engine's stated bound.  bfloat16: 8 bits of
# mantissa, a handful of roundings per layer; the worst error seen over some
# thousands of seeds of these models is 8e-3 of the largest logit.
TOL = {"float32": 1e-4, "bfloat16": 1.5e-2}


def requests_for(name: str) -> dict[str, list[int]]:
    rng = random.Random(sum(map(ord, name)))
    vocab = CONFIGS[name]["vocab_size"]
    return {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(LENGTHS[name])}


@pytest.fixture(scope="module")
def model_root(tmp_path_factory):
    return tmp_path_factory.mktemp("models")


# each tiny model at its own page size (4, 8, 16) and at 16, the size that serving uses
CASES = sorted({(name, size) for name in "ABCD" for size in (PAGE_SIZES[name], 16)})


@pytest.mark.parametrize("mode", ["reference", "unit"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name, page_size", CASES)
def test_four_cuttings_agree_with_the_plain_implementation(name, page_size, dtype, mode, model_root, tmp_path):
    """Every free page is poisoned with NaN, at the start and whenever a request
    gives it back: a row that read one would not pass the comparison."""
    model_dir = make_model_dir(name, model_root, dtype=dtype, mode=mode)
    vocab = CONFIGS[name]["vocab_size"]
    seqs = requests_for(name)
    plain = PlainModel(model_dir)
    want = {rid: plain.logits(ids).numpy() for rid, ids in seqs.items()}

    tb = TraceBuilder()
    budget = max(-(-len(ids) // 64) * 64 for ids in seqs.values())
    whole(tb, "w_", seqs)
    last_one_by_one(tb, "d_", seqs)
    changing_portions(tb, "p_", seqs)
    # room for the largest request plus two small ones: the others wait for pages
    mixed_budget = budget + 128
    mixed(tb, "m_", seqs, mixed_budget, seed=3)
    outputs = run_trace(model_dir, dtype, tb.steps, mixed_budget, tmp_path / "out", vocab,
                        block_size=page_size, poison=True, pages=True)
    got = tb.collect(outputs)
    assert all(np.isfinite(rows).all() for rows in outputs.values())
    reused = check_pages(tb.steps, read_pages(tmp_path / "out", tb.steps), page_size, mixed_budget // page_size)
    assert reused > 0, "the pool was meant to be so small that pages are used again"

    scale = {rid: np.abs(w).max() for rid, w in want.items()}
    worst = {}
    for (rid, pos), row in got.items():
        cut, name_ = rid.split("_", 1)
        err = np.abs(row.astype(np.float64) - want[name_][pos]).max() / scale[name_]
        worst[cut] = max(worst.get(cut, 0.0), err)
        assert err <= TOL[dtype], f"{rid} position {pos}: rel err {err:.3e}"
    assert set(worst) == {"w", "d", "p", "m"}
    # every position of every request was asked for in the first three cuttings
    for cut in "wdp":
        assert all((f"{cut}_{rid}", p) in got for rid, ids in seqs.items() for p in range(len(ids)))
    # cuttings agree with each other far more closely than with the plain model in float32
    if dtype == "float32":
        for (rid, pos), row in got.items():
            cut, name_ = rid.split("_", 1)
            ref = got[(f"w_{name_}", pos)]
            assert np.abs(row - ref).max() / scale[name_] <= 1e-5
    print(f"{name} page {page_size} {dtype} {mode}: worst rel err per cutting {worst}")


def test_greedy_tokens_from_replayed_logits_match_plain(model_root, tmp_path):
    """Teacher-forced decode of the plain model's own greedy continuation: the
    argmax of every replayed row is the plain model's next token."""
    model_dir = make_model_dir("B", model_root, dtype="float32", mode="unit")
    plain = PlainModel(model_dir)
    prompt = [7, 300, 21, 99, 5, 410, 8]
    gen = plain.greedy(prompt, 12)
    ids = prompt + gen
    tb = TraceBuilder()
    tb.add([("g", prompt, 0, [len(prompt) - 1])])
    for i, tok in enumerate(gen[:-1]):
        tb.add([("g", [tok], len(prompt) + i, [0])])
    out = run_trace(model_dir, "float32", tb.steps, 64, tmp_path / "out", 503)
    got = [int(out[s][0].argmax()) for s in range(len(tb.steps))]
    assert got == gen
    assert torch.equal(torch.tensor(ids[len(prompt):]), torch.tensor(got))
