"""The layer sizes of the Qwen2.5-7B shape (hidden 3584, 28 query heads over 4
key/value heads of 128, intermediate 18944, vocabulary 152064) with one layer
and seeded random weights, against the plain implementation: the kernels that
serving uses at their real sizes (split products, 7 heads per group, a
vocabulary that is no power of two), in float32 and in bfloat16, cut four ways."""

import random

import pytest
import torch

from .plain.model import PlainModel, rel_err

pytestmark = pytest.mark.gpu

SHAPE = {
    "architectures": ["Qwen2ForCausalLM"],
    "hidden_size": 3584,
    "intermediate_size": 18944,
    "num_hidden_layers": 1,
    "num_attention_heads": 28,
    "num_key_value_heads": 4,
    "vocab_size": 152064,
    "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-6,
    "tie_word_embeddings": False,
    "torch_dtype": "bfloat16",
}


# One layer of the Qwen2.5-14B shape: 40 query heads over 8 key/value heads (groups
# of 5), another width, another eps; a smaller vocabulary keeps the test short.
SHAPE_14B = dict(SHAPE, hidden_size=5120, intermediate_size=13824, num_attention_heads=40,
                 num_key_value_heads=8, rms_norm_eps=1e-5, vocab_size=32003)


@pytest.fixture(scope="module")
def model_dir(tmp_path_factory):
    from shrike_amd.weights import write_model_folder

    return write_model_folder(dict(SHAPE), tmp_path_factory.mktemp("big") / "m", seed=7, mode="unit")


@pytest.fixture(scope="module")
def plain_model(model_dir):
    return PlainModel(model_dir, dtype=torch.float32)  # float64 weights would not fit comfortably


@pytest.fixture(scope="module")
def reference(plain_model):
    rng = random.Random(5)
    ids = [rng.randrange(SHAPE["vocab_size"]) for _ in range(150)]
    return ids, plain_model.logits(ids).double()


def four_cuttings(model_dir, dtype, tol, ids, want):
    from shrike_amd.cache import CacheManager
    from shrike_amd.engine.loading import load_model
    from shrike_amd.engine.runner import ModelRunner, StepEntry

    model, rt, _ = load_model(model_dir, dtype)
    cache = CacheManager(model.cache_specs(), 16, 24, enable_prefix_caching=False)
    cache.allocate(rt.dtype, rt.device)
    runner = ModelRunner(model, cache, rt)

    def run(cuts, other=None):
        seq = cache.new_sequence()
        rows, p = [], 0
        for n in cuts:
            cache.append(seq, p, n)
            entries = [StepEntry(seq, ids[p : p + n], p, list(range(n)))]
            if other is not None:  # another request's single token rides along
                o, op = other
                cache.append(o, op[0], 1)
                entries.insert(0, StepEntry(o, [ids[op[0]]], op[0], [0]))
                op[0] += 1
            out = runner.step(entries).cpu()
            rows.append(out[-n:].clone())
            p += n
        cache.free(seq)
        return torch.cat(rows).double()

    n = len(ids)
    whole = run([n])
    assert rel_err(whole, want) <= tol
    tail = run([n - 32] + [1] * 32)  # the last 32 tokens one by one (graph replays)
    assert rel_err(tail, want) <= tol
    portions = run([70, 2, 17, 33, 5, 23])
    assert rel_err(portions, want) <= tol
    rider = cache.new_sequence()
    mixed = run([64, 40, 2, 44], other=(rider, [0]))
    cache.free(rider)
    assert rel_err(mixed, want) <= tol
    if dtype == "float32":
        for other in (tail, portions, mixed):
            assert rel_err(other, whole) <= 1e-5
    cache.check([])


@pytest.mark.parametrize("dtype, tol", [("float32", 1e-4), ("bfloat16", 1.5e-2)])
def test_one_layer_of_the_7b_shape(dtype, tol, model_dir, reference):
    ids, want = reference
    four_cuttings(model_dir, dtype, tol, ids, want)


@pytest.mark.parametrize("dtype, tol", [("float32", 1e-4), ("bfloat16", 1.5e-2)])
def test_one_layer_of_the_14b_shape(dtype, tol, tmp_path_factory):
    """Five query heads per key/value head, width 5120: the four cuttings again."""
    from shrike_amd.weights import write_model_folder

    folder = tmp_path_factory.getbasetemp() / "big14"
    if not (folder / "model.safetensors").is_file():
        write_model_folder(dict(SHAPE_14B), folder, seed=9, mode="unit")
    rng = random.Random(6)
    ids = [rng.randrange(SHAPE_14B["vocab_size"]) for _ in range(150)]
    want = PlainModel(folder, dtype=torch.float32).logits(ids).double()
    four_cuttings(folder, dtype, tol, ids, want)


@pytest.fixture(scope="module")
def long_reference(plain_model):
    """4,103 tokens through the plain model; logits at the rows the tests below ask for."""
    rng = random.Random(8)
    ids = [rng.randrange(SHAPE["vocab_size"]) for _ in range(4103)]
    rows = [0, 15, 16, 1023, 2047] + list(range(4095, 4103))
    return ids, plain_model.logits(ids, rows=rows).double()


@pytest.mark.parametrize("dtype, tol", [("float32", 1e-4), ("bfloat16", 1.5e-2)])
def test_a_2048_token_prompt_and_decoding_past_context_4096(dtype, tol, model_dir, long_reference):
    """What the benchmark times, compared with the plain implementation: a
    2,048-token prompt in one step (64 chunks of keys for the last query tile),
    then the sequence grown to 4,095 tokens in portions, then 8 single tokens
    through the graph path with the key splits the engine chooses itself."""
    from shrike_amd.cache import CacheManager
    from shrike_amd.engine.loading import load_model
    from shrike_amd.engine.runner import ModelRunner, StepEntry

    ids, want = long_reference
    model, rt, _ = load_model(model_dir, dtype)
    cache = CacheManager(model.cache_specs(), 16, 300, enable_prefix_caching=False)
    cache.allocate(rt.dtype, rt.device)
    for g in cache.groups:  # a slot that is read before it is written shows up as NaN
        for t in g.tensors.values():
            t.fill_(float("nan"))
    runner = ModelRunner(model, cache, rt)
    seq = cache.new_sequence()
    cache.append(seq, 0, 2048)
    first = runner.step([StepEntry(seq, ids[:2048], 0, [0, 15, 16, 1023, 2047])]).cpu().double()
    assert rel_err(first, want[:5]) <= tol
    p = 2048
    for n in (1000, 512, 535):
        cache.append(seq, p, n)
        runner.step([StepEntry(seq, ids[p : p + n], p, [])])
        p += n
    assert p == 4095
    rows = []
    for p in range(4095, 4103):
        cache.append(seq, p, 1)
        rows.append(runner.step([StepEntry(seq, [ids[p]], p, [0])]).cpu().double()[0])
    assert runner.graph_replays == 8
    got = torch.stack(rows)
    assert torch.isfinite(got).all()
    assert rel_err(got, want[5:]) <= tol
    cache.free(seq)


@pytest.mark.parametrize("count", [100, 150])
def test_many_single_tokens_as_a_graph_and_kernel_by_kernel(model_dir, plain_model, count):
    """100 or 150 sequences decode together (graphs of 128 and 256 rows): a batch that the large product kernels
    serve (tiles of 128 and 256 tokens, operands loaded straight into LDS, shares
    of k).  Replayed from a HIP graph several times, with the program's own work
    between the replays, the logits equal those of kernel-by-kernel execution
    bit for bit."""
    from shrike_amd.cache import CacheManager
    from shrike_amd.engine.loading import load_model
    from shrike_amd.engine.runner import ModelRunner, StepEntry

    model, rt, _ = load_model(model_dir, "bfloat16")
    rng = random.Random(11)
    prompts = [[rng.randrange(SHAPE["vocab_size"]) for _ in range(rng.randint(1, 5))] for _ in range(count)]
    feed = [[rng.randrange(SHAPE["vocab_size"]) for _ in range(4)] for _ in range(count)]

    def run(graphs):
        cache = CacheManager(model.cache_specs(), 16, 160, enable_prefix_caching=False)
        cache.allocate(rt.dtype, rt.device)
        runner = ModelRunner(model, cache, rt, graphs=graphs)
        seqs = [cache.new_sequence() for _ in prompts]
        for s, p in zip(seqs, prompts):
            cache.append(s, 0, len(p))
        runner.step([StepEntry(s, p, 0, []) for s, p in zip(seqs, prompts)])
        outs = []
        for step in range(4):
            entries = []
            for s, p, f in zip(seqs, prompts, feed):
                cache.append(s, len(p) + step, 1)
                entries.append(StepEntry(s, [f[step]], len(p) + step, [0]))
            outs.append(runner.step(entries).clone())
            torch.cuda.synchronize()
        assert runner.graph_replays == (4 if graphs else 0)
        for s in seqs:
            cache.free(s)
        return outs

    eager, replayed = run(False), run(True)
    for a, b in zip(eager, replayed):
        assert torch.isfinite(a).all() and torch.equal(a, b)
    # and both are right: some rows, the first and the last among them, against the
    # plain implementation run on each sequence alone
    for row in (0, 1, 37, 63, 64, count - 2, count - 1):
        for step in (0, 3):
            want = plain_model.logits(prompts[row] + feed[row][: step + 1], rows=[-1]).double()[0]
            assert rel_err(replayed[step][row].cpu().double(), want) <= 1.5e-2, (row, step)


@pytest.mark.parametrize("dtype, tol", [("float32", 1e-4), ("bfloat16", 1.5e-2)])
def test_decoding_requests_beside_a_portion_far_into_a_prompt(dtype, tol, tmp_path_factory, monkeypatch):
    """One step of 32 single tokens beside a 480-token portion that starts at
    position 1,120 of its prompt, with the 14B layer sizes: what a long prompt
    under the 512-token budget looks like while others decode.  In bfloat16 the
    portion's keys are shared among several workgroups whose results are merged
    behind the single tokens' rows; the portion's rows and the riders' rows are
    compared with the plain implementation."""
    from shrike_amd.cache import CacheManager
    from shrike_amd.engine.loading import load_model
    from shrike_amd.engine.runner import ModelRunner, StepEntry
    from shrike_amd.kernels import ops
    from shrike_amd.weights import write_model_folder

    folder = tmp_path_factory.getbasetemp() / "big14"
    if not (folder / "model.safetensors").is_file():
        write_model_folder(dict(SHAPE_14B), folder, seed=9, mode="unit")
    rng = random.Random(12)
    vocab = SHAPE_14B["vocab_size"]
    main = [rng.randrange(vocab) for _ in range(1600)]
    riders = [[rng.randrange(vocab) for _ in range(rng.choice([1, 2, 15, 16, 17, 100, 333]) + 1)]
              for _ in range(32)]
    plain = PlainModel(folder, dtype=torch.float32)
    main_rows = [1120, 1121, 1135, 1136, 1300, 1407, 1598, 1599]
    want_main = plain.logits(main, rows=main_rows).double()
    checked_riders = [0, 7, 19, 31]
    want_riders = torch.stack([plain.logits(riders[i], rows=[-1]).double()[0] for i in checked_riders])

    seen = []
    launch = ops.attention_prefill_shared

    def spy(*args, **kwargs):
        seen.append((kwargs.get("nsplit", 1), kwargs.get("first_token", 0)))
        return launch(*args, **kwargs)

    monkeypatch.setattr(ops, "attention_prefill_shared", spy)
    model, rt, _ = load_model(folder, dtype)
    cache = CacheManager(model.cache_specs(), 16, 100 + 32 * 22, enable_prefix_caching=False)
    cache.allocate(rt.dtype, rt.device)
    for g in cache.groups:
        for t in g.tensors.values():
            t.fill_(float("nan"))
    runner = ModelRunner(model, cache, rt)
    seq = cache.new_sequence()
    cache.append(seq, 0, 1120)
    runner.step([StepEntry(seq, main[:1120], 0, [])])
    rider_seqs = [cache.new_sequence() for _ in riders]
    warm = []
    for s, ids in zip(rider_seqs, riders):
        cache.append(s, 0, len(ids) - 1)
        warm.append(StepEntry(s, ids[:-1], 0, []))
    runner.step(warm)
    seen.clear()
    entries = [StepEntry(seq, main[1120:], 1120, [r - 1120 for r in main_rows])]  # the portion first:
    cache.append(seq, 1120, 480)
    for s, ids in zip(rider_seqs, riders):  # the step function puts the single tokens in front itself
        cache.append(s, len(ids) - 1, 1)
        entries.append(StepEntry(s, [ids[-1]], len(ids) - 1, [0]))
    out = runner.step(entries).cpu().double()
    assert out.shape[0] == len(main_rows) + 32 and torch.isfinite(out).all()
    if dtype == "bfloat16":  # one launch for the layer: keys shared, 32 single tokens in front
        assert seen and all(nsplit > 1 and first == 32 for nsplit, first in seen), seen
    assert rel_err(out[: len(main_rows)], want_main) <= tol
    got_riders = torch.stack([out[len(main_rows) + i] for i in checked_riders])
    assert rel_err(got_riders, want_riders) <= tol
    for s in [seq] + rider_seqs:
        cache.free(s)
    cache.check([])


def test_two_layers_of_the_7b_shape_generate_the_plain_tokens(tmp_path_factory):
    """Greedy generation through the entry point with two layers of the 7B sizes:
    in float32 every token is the plain implementation's, prompts cut by a token
    budget of 24; in bfloat16 but for a few near-ties."""
    from shrike_amd import LLM, SamplingParams
    from shrike_amd.weights import write_model_folder

    from .compare import GreedyCheck

    folder = write_model_folder(dict(SHAPE, num_hidden_layers=2), tmp_path_factory.mktemp("big2") / "m",
                                seed=13, mode="unit")
    plain = PlainModel(folder, dtype=torch.float32)
    rng = random.Random(14)
    prompts = [[rng.randrange(SHAPE["vocab_size"]) for _ in range(n)] for n in (40, 7)]
    for dtype in ("float32", "bfloat16"):
        llm = LLM(str(folder), dtype=dtype, block_size=16, num_kv_blocks=16, max_tokens_per_step=24)
        outs = llm.generate(prompts, SamplingParams(max_new_tokens=6, ignore_eos=True))
        check = GreedyCheck(plain, dtype)
        for prompt, out in zip(prompts, outs):
            assert len(out) == 6
            check.request(prompt, out)
        if dtype == "float32":
            assert check.excused == 0
        else:
            assert check.excused <= 2
        del llm
        torch.cuda.empty_cache()
