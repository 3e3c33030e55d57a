"""The engine end to end on the GPU: generation through the Python entry point
against the plain implementation, sampling, what happens when pages run out,
prefix sharing, long decoding, and the guards of add_request."""

import random

import pytest
import torch

from .compare import TOL, GreedyCheck
from .plain.model import PlainModel, softmax_sample_reference
from .tiny import CONFIGS, PAGE_SIZES, make_model_dir

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def model_root(tmp_path_factory):
    return tmp_path_factory.mktemp("models")


def prompts_for(name, lengths, seed=0):
    rng = random.Random(seed)
    vocab = CONFIGS[name]["vocab_size"]
    eos = CONFIGS[name].get("eos_token_id", [])
    eos = set(eos if isinstance(eos, list) else [eos])
    return [[rng.choice([t for t in range(vocab) if t not in eos]) for _ in range(n)] for n in lengths]


@pytest.mark.parametrize(
    "name, lengths, new, budget",
    [("A", [5, 11, 17], 8, 512), ("A_untied", [5, 11, 17], 24, 512), ("B", [1, 9, 30, 64], 12, 16),
     ("C", [3, 50, 28], 40, 24),
     ("D", [2, 70, 33, 120], 60, 48)],
)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(name, lengths, new, budget, dtype, model_root):
    from shrike_amd import LLM, SamplingParams

    model_dir = make_model_dir(name, model_root, dtype=dtype, mode="unit")
    plain = PlainModel(model_dir)
    prompts = prompts_for(name, lengths)
    llm = LLM(str(model_dir), dtype=dtype, block_size=PAGE_SIZES[name], num_kv_blocks=64,
              max_tokens_per_step=budget)
    outs = llm.generate(prompts, SamplingParams(max_new_tokens=new, ignore_eos=True))
    assert [len(o) for o in outs] == [new] * len(prompts)
    check = GreedyCheck(plain, dtype)  # float32: identical greedy tokens
    for prompt, out in zip(prompts, outs):
        check.request(prompt, out)
    check.finish()
    assert llm.engine.cache.num_free == llm.engine.cache.num_pages  # tests/test_paged.py:102-103
    assert llm.engine.cache.slots.num_free == llm.engine.cache.slots.num_slots


def test_reference_weights_greedy_identical_in_float32(model_root):
    from shrike_amd import LLM, SamplingParams

    model_dir = make_model_dir("A", model_root)
    plain = PlainModel(model_dir)
    prompts = prompts_for("A", [5, 11, 17], seed=4)
    llm = LLM(str(model_dir), dtype="float32", block_size=4, num_kv_blocks=32, max_tokens_per_step=3)
    outs = llm.generate(prompts, SamplingParams(max_new_tokens=8, ignore_eos=True))
    assert outs == [plain.greedy(p, 8) for p in prompts]


def test_eos_stops_and_is_emitted(model_root):
    from shrike_amd import LLM, SamplingParams

    model_dir = make_model_dir("B", model_root, mode="unit")
    plain = PlainModel(model_dir)
    prompt = prompts_for("B", [12], seed=9)[0]
    free_run = plain.greedy(prompt, 30)
    llm = LLM(str(model_dir), dtype="float32", block_size=8, num_kv_blocks=32)
    llm.engine.eos_ids = {free_run[6]}  # whatever the 7th token is ends the request
    out = llm.generate([prompt], SamplingParams(max_new_tokens=30))[0]
    stop = free_run.index(free_run[6])
    assert out == free_run[: stop + 1]
    out = llm.generate([prompt], SamplingParams(max_new_tokens=10, ignore_eos=True))[0]
    assert out == free_run[:10]


def test_temperature_sampling_is_repeatable_and_stays_in_the_nucleus(model_root):
    from shrike_amd import LLM, SamplingParams

    model_dir = make_model_dir("B", model_root, mode="unit")
    plain = PlainModel(model_dir)
    prompts = prompts_for("B", [1, 9, 30, 64], seed=2)
    llm = LLM(str(model_dir), dtype="float32", block_size=8, num_kv_blocks=64, max_tokens_per_step=16)
    sp = SamplingParams(max_new_tokens=12, temperature=0.7, top_p=0.8, seed=1234, ignore_eos=True)
    a = llm.generate(prompts, sp)
    b = llm.generate(list(reversed(prompts)), sp)[::-1]  # other batch order, other request ids
    assert a == b
    c = llm.generate(prompts, SamplingParams(max_new_tokens=12, temperature=0.7, top_p=0.8, seed=99, ignore_eos=True))
    assert a != c
    greedy = llm.generate(prompts, SamplingParams(max_new_tokens=12, ignore_eos=True))
    assert a != greedy
    for prompt, out in zip(prompts, a):
        seq = list(prompt)
        for tok in out:
            kept, weights = softmax_sample_reference(plain.logits(seq)[-1], 0.7, 0.8)
            # the rule's kept set, give or take its last entry (float32 against float64 at the edge)
            kept2, _ = softmax_sample_reference(plain.logits(seq)[-1], 0.7, 0.8 + 1e-4)
            assert tok in kept.tolist() or tok in kept2.tolist()
            seq.append(tok)


def test_when_pages_run_out_the_newest_request_is_preempted_and_recomputes(model_root):
    from shrike_amd import SamplingParams
    from shrike_amd.engine.llm_engine import LLMEngine

    model_dir = make_model_dir("A", model_root, mode="unit")
    prompts = prompts_for("A", [9, 14, 6, 11], seed=5)
    sp = SamplingParams(max_new_tokens=20, ignore_eos=True)
    roomy = LLMEngine(str(model_dir), dtype="float32", block_size=4, num_kv_blocks=64)
    want = roomy.generate(prompts, sp)
    assert roomy.metrics()["preemptions"] == 0
    # 12 pages of 4: all four prompts fit, their generations do not
    tight = LLMEngine(str(model_dir), dtype="float32", block_size=4, num_kv_blocks=12,
                      enable_prefix_caching=False)
    got = tight.generate(prompts, sp)
    assert tight.metrics()["preemptions"] > 0
    assert got == want
    assert tight.cache.num_free == 12 and not tight.has_work


@pytest.mark.parametrize("dtype, page", [("float32", 8), ("bfloat16", 16)])
def test_prefix_sharing_changes_nothing_but_the_work(model_root, dtype, page):
    """bfloat16 at page size 16 runs the matrix-instruction attention kernels: a
    request that finds its prefix in the cache computes the rest as a portion
    that starts inside the sequence, over pages that another request wrote."""
    from shrike_amd import SamplingParams
    from shrike_amd.engine.llm_engine import LLMEngine

    model_dir = make_model_dir("B", model_root, dtype=dtype, mode="unit")
    common = prompts_for("B", [40], seed=6)[0]
    prompts = [common + tail for tail in ([5, 6, 7], [8], [9, 10, 11, 12, 13])]
    sp = SamplingParams(max_new_tokens=6 if dtype == "float32" else 30, ignore_eos=True)
    off = LLMEngine(str(model_dir), dtype=dtype, block_size=page, num_kv_blocks=64, enable_prefix_caching=False)
    want = [off.generate([p], sp)[0] for p in prompts]
    on = LLMEngine(str(model_dir), dtype=dtype, block_size=page, num_kv_blocks=64)
    got = [on.generate([p], sp)[0] for p in prompts]
    if dtype == "float32":
        assert got == want
    else:  # another cutting of the prompt may round another way: both are judged by the plain model
        plain = PlainModel(model_dir)
        for outs in (want, got):
            check = GreedyCheck(plain, dtype)
            for prompt, out in zip(prompts, outs):
                check.request(prompt, out)
            check.finish()
    assert on.metrics()["prefix_cache_hit_rate"] > 0.5 and off.metrics()["prefix_cache_hit_rate"] == 0


def test_long_decoding_and_first_tokens(model_root):
    """300 decoded tokens across many pages, and the logits at the first
    positions of a sequence (one key, two keys, the first page's edge)."""
    from shrike_amd.cache import CacheManager
    from shrike_amd.engine.loading import load_model
    from shrike_amd.engine.runner import ModelRunner, StepEntry

    for dtype, tol in TOL.items():
        model_dir = make_model_dir("C", model_root, dtype=dtype, mode="unit")
        plain = PlainModel(model_dir)
        model, rt, cfg = load_model(model_dir, dtype)
        cache = CacheManager(model.cache_specs(), 16, 32, enable_prefix_caching=False)
        cache.allocate(rt.dtype, rt.device)
        runner = ModelRunner(model, cache, rt)
        ids = prompts_for("C", [320], seed=7)[0]
        want = plain.logits(ids)
        seq = cache.new_sequence()
        rows = []
        for p, tok in enumerate(ids):  # every token on the single-token path, from the very first
            cache.append(seq, p, 1)
            rows.append(runner.step([StepEntry(seq, [tok], p, [0])]).cpu().clone())
            cache.trim(seq, p + 1)
        got = torch.cat(rows).double()
        err = (got - want).abs().amax(-1) / want.abs().max()
        assert float(err.max()) <= tol, f"{dtype}: worst at position {int(err.argmax())}: {float(err.max()):.3e}"
        cache.free(seq)
        cache.check([])


@pytest.mark.parametrize("dtype, tol, streamed", [("float32", TOL["float32"], False),
                                                  ("bfloat16", TOL["bfloat16"], False),
                                                  ("bfloat16", TOL["bfloat16"], True)])
def test_a_context_of_ten_thousand_tokens(model_root, dtype, tol, streamed, monkeypatch):
    """A 10,000-token prompt in portions of up to 4,096 tokens (the later ones
    read keys far back, through block tables of more than 600 pages), then six
    single tokens from a graph with the key splits the engine chooses there;
    `streamed`: with the non-temporal loads that the engine takes for large batches."""
    from shrike_amd.cache import CacheManager
    from shrike_amd.engine.loading import load_model
    from shrike_amd.engine.runner import ModelRunner, StepEntry
    from shrike_amd.kernels import ops
    from shrike_amd.parts import attention

    if streamed:
        monkeypatch.setattr(attention, "STREAMING_FROM_BYTES", 0)
    flags = []
    launch = ops.attention_decode
    monkeypatch.setattr(ops, "attention_decode", lambda *a, **kw: (flags.append(a[15]), launch(*a, **kw))[1])

    model_dir = make_model_dir("B", model_root, dtype=dtype, mode="unit")
    ids = prompts_for("B", [10006], seed=9)[0]
    wanted = {0: [0, 4095], 4096: [0, 4095], 8192: [0, 1807]}  # portion start -> rows within it
    rows = [start + r for start, rs in wanted.items() for r in rs] + list(range(10000, 10006))
    want = PlainModel(model_dir).logits(ids, rows=rows).double()
    model, rt, _ = load_model(model_dir, dtype)
    cache = CacheManager(model.cache_specs(), 16, 640, enable_prefix_caching=False)
    cache.allocate(rt.dtype, rt.device)
    for g in cache.groups:  # a slot that is read before it is written shows up as NaN
        for t in g.tensors.values():
            t.fill_(float("nan"))
    runner = ModelRunner(model, cache, rt)
    seq = cache.new_sequence()
    got = []
    for start, rs in wanted.items():
        n = min(4096, 10000 - start)
        cache.append(seq, start, n)
        got.append(runner.step([StepEntry(seq, ids[start : start + n], start, rs)]).cpu().double())
    for p in range(10000, 10006):
        cache.append(seq, p, 1)
        got.append(runner.step([StepEntry(seq, [ids[p]], p, [0])]).cpu().double())
    assert runner.graph_replays == 6
    assert flags and all(f == streamed for f in flags) if dtype == "bfloat16" else not flags
    got = torch.cat(got)
    assert torch.isfinite(got).all()
    err = (got - want).abs().amax(-1) / want.abs().max()
    assert float(err.max()) <= tol, f"worst at row {rows[int(err.argmax())]}: {float(err.max()):.3e}"
    cache.free(seq)
    cache.check([])


@pytest.mark.parametrize("dtype, page", [("float32", 8), ("bfloat16", 16)])
def test_overlapped_steps_change_no_token(model_root, tmp_path, dtype, page):
    """The next decode step is launched before the host has read this step's tokens.
    With a fifth of all token ids ending a sequence, requests end at steps that
    nobody can foresee, and some are aborted while a step that holds them is
    already running: every request still yields exactly what an engine that does
    not overlap yields for it alone, greedy or drawn.  In bfloat16 (page size 16:
    the matrix-instruction attention kernels, graphs and steps in flight together)
    a row's bits depend on the batch it runs in, so every request is greedy and is
    judged by the plain model instead: its tokens are the plain argmax but for a
    few near-ties, and it ends at its first end-of-sequence token or at its length."""
    from shrike_amd import SamplingParams
    from shrike_amd.engine.llm_engine import LLMEngine
    from shrike_amd.weights import write_model_folder

    exact = dtype == "float32"
    eos = list(range(3, CONFIGS["B"]["vocab_size"], 5))
    cfg = dict(CONFIGS["B"], eos_token_id=eos)
    model_dir = write_model_folder(cfg, tmp_path / "many_ends", seed=5, mode="unit", dtype=dtype)
    rng = random.Random(21)
    jobs = []
    for i in range(24):
        prompt = prompts_for("B", [rng.randint(1, 40)], seed=300 + i)[0]
        jobs.append((prompt, SamplingParams(max_new_tokens=rng.randint(1, 40), top_p=0.95, seed=i,
                                            temperature=0.9 if exact and i % 3 == 0 else 0.0)))
    alone = LLMEngine(str(model_dir), dtype=dtype, block_size=page, num_kv_blocks=64,
                      enable_prefix_caching=False, overlap_steps=False)
    want = [alone.generate([p], sp)[0] for p, sp in jobs]
    assert 4 < sum(len(w) < sp.max_new_tokens for w, (_, sp) in zip(want, jobs)) < 24

    engine = LLMEngine(str(model_dir), dtype=dtype, block_size=page, num_kv_blocks=80, max_running=8)
    assert engine.config.overlap_steps
    got, ids, pending, aborted, overlapped = {}, {}, list(range(len(jobs))), set(), 0
    while pending or engine.has_work:
        for _ in range(8 if len(pending) == len(jobs) else int(rng.random() < 0.3)):
            if pending:  # eight requests to begin with, then one now and then
                i = pending.pop(0)
                ids[engine.add_request(jobs[i][0], jobs[i][1])] = i
        if engine._inflight is not None:
            overlapped += 1
            if len(aborted) < 3 and rng.random() < 0.3:  # a request of the step that is running
                victim = rng.choice(engine._inflight[0])[0]
                aborted.add(ids[victim.req_id])
                engine.abort(victim.req_id)
        for o in engine.step():
            got.setdefault(ids[o.req_id], []).append(o.token_id)
        engine.cache.check([r.cache for r in engine.scheduler.running if r.cache is not None])
    assert overlapped > 10 and aborted
    if exact:
        for i, w in enumerate(want):
            mine = got.get(i, [])
            assert mine == (w[: len(mine)] if i in aborted else w), f"request {i}"
    else:
        check = GreedyCheck(PlainModel(model_dir), dtype)
        for i, (prompt, sp) in enumerate(jobs):
            mine = got.get(i, [])
            check.request(prompt, mine)
            assert not set(mine[:-1]) & set(eos), f"request {i} went on after an end-of-sequence token"
            if i not in aborted:
                assert mine and (mine[-1] in eos or len(mine) == sp.max_new_tokens), f"request {i}"
        check.finish()
    assert engine.cache.num_free == 80 and not engine.scheduler.running
    engine.cache.check([])


def test_add_request_guards(model_root):
    # tests/test_review_regressions.py:90-93
    from shrike_amd import SamplingParams
    from shrike_amd.engine.llm_engine import LLMEngine

    engine = LLMEngine(str(make_model_dir("A", model_root)), dtype="float32", block_size=4, num_kv_blocks=8)
    with pytest.raises(ValueError, match="empty"):
        engine.add_request([], SamplingParams())
    with pytest.raises(ValueError, match="never be scheduled"):
        engine.add_request([1, 2, 3], SamplingParams(max_new_tokens=10_000_000))
    with pytest.raises(ValueError, match="token ids"):
        engine.add_request([1, 2, 256], SamplingParams())
    with pytest.raises(ValueError, match="tokenizer"):
        engine.add_request("some text", SamplingParams())
    assert engine.step() == [] and not engine.has_work


def test_metrics_and_streaming_outputs(model_root):
    from shrike_amd import SamplingParams
    from shrike_amd.engine.llm_engine import LLMEngine

    engine = LLMEngine(str(make_model_dir("A", model_root)), dtype="bfloat16", block_size=4, num_kv_blocks=32)
    rid = engine.add_request([1, 2, 3, 4, 5], SamplingParams(max_new_tokens=3, ignore_eos=True))
    outs = []
    while engine.has_work:
        outs += engine.step()
    assert [o.req_id for o in outs] == [rid] * 3
    assert [o.finished for o in outs] == [False, False, True] and outs[-1].finish_reason == "length"
    m = engine.metrics()
    assert m["tokens_generated"] == 3 and m["steps"] == 3 and m["running"] == 0
    assert m["kv_blocks_total"] == 32 and m["kv_blocks_free"] == 32


def test_command_line_generates(model_root, capsys):
    from shrike_amd.__main__ import main

    model_dir = make_model_dir("A", model_root, mode="unit")
    rc = main(["--model", str(model_dir), "--prompt-ids", "5,6,7,8", "--max-tokens", "5",
               "--dtype", "fp32", "--block-size", "4", "--num-kv-blocks", "16", "--ignore-eos", "--metrics"])
    assert rc == 0
    out = capsys.readouterr()
    assert [int(t) for t in out.out.split()] == PlainModel(model_dir).greedy([5, 6, 7, 8], 5)
    assert "tokens_generated" in out.err


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replays_equal_eager_steps(dtype, model_root):
    """Decode steps replayed from HIP graphs, with eager prompt portions and
    batch-size changes between the replays, give bit for bit what the same
    steps give when every kernel is launched on its own."""
    from shrike_amd.cache import CacheManager
    from shrike_amd.engine.loading import load_model
    from shrike_amd.engine.runner import ModelRunner, StepEntry

    model_dir = make_model_dir("B", model_root, dtype=dtype, mode="unit")
    model, rt, cfg = load_model(model_dir, dtype)
    prompts = prompts_for("B", [40, 7, 90, 23, 5], seed=8)

    def run(graphs):
        cache = CacheManager(model.cache_specs(), 16, 40, enable_prefix_caching=False)
        cache.allocate(rt.dtype, rt.device)
        runner = ModelRunner(model, cache, rt, graphs=graphs)
        live, outs = [], []
        rng = random.Random(1)

        def add(ids):
            seq = cache.new_sequence()
            cache.append(seq, 0, len(ids))
            outs.append(runner.step([StepEntry(seq, ids, 0, [len(ids) - 1])]).cpu().clone())
            live.append([seq, len(ids)])

        add(prompts[0])
        for step in range(60):
            if step in (5, 11, 30, 31):  # a prompt arrives between decode steps: batch 1 -> 2 -> 3 -> 5
                add(prompts[len(live)])
            entries = []
            for item in live:
                cache.append(item[0], item[1], 1)
                entries.append(StepEntry(item[0], [rng.randrange(cfg.vocab_size)], item[1], [0]))
                item[1] += 1
            outs.append(runner.step(entries).cpu().clone())
        for item in live:
            cache.free(item[0])
        return outs, runner.graph_replays

    eager, n0 = run(False)
    graphed, n1 = run(True)
    assert n0 == 0 and n1 == 60
    assert len(eager) == len(graphed)
    for a, b in zip(eager, graphed):
        assert torch.equal(a, b)


def test_random_arrivals_under_page_pressure_with_shared_prefixes(model_root):
    """Requests arrive while others run, share prefixes, differ in length and in
    sampling, and the pool is small enough for preemptions: every greedy
    request still produces what it produces alone in a roomy engine, and every
    page and slot is back in the end."""
    from shrike_amd import SamplingParams
    from shrike_amd.engine.llm_engine import LLMEngine

    model_dir = make_model_dir("B", model_root, mode="unit")
    rng = random.Random(11)
    stems = prompts_for("B", [24, 17], seed=12)
    jobs = []
    for i in range(14):
        stem = stems[i % 2][: rng.choice([8, 16, 17, 24])] if i % 3 else []
        tail = prompts_for("B", [rng.randint(1, 30)], seed=100 + i)[0]
        greedy = i % 4 != 3
        sp = SamplingParams(max_new_tokens=rng.randint(1, 25), ignore_eos=True,
                            temperature=0.0 if greedy else 0.8, top_p=0.9, seed=i)
        jobs.append((stem + tail, sp, greedy))

    roomy = LLMEngine(str(model_dir), dtype="float32", block_size=8, num_kv_blocks=128,
                      enable_prefix_caching=False)
    want = [roomy.generate([p], sp)[0] for p, sp, _ in jobs]

    tight = LLMEngine(str(model_dir), dtype="float32", block_size=8, num_kv_blocks=22,
                      max_tokens_per_step=24, max_running=5)
    got, ids, pending = {}, {}, list(range(len(jobs)))
    while pending or tight.has_work:
        for _ in range(rng.randint(0, 2)):  # zero to two arrivals before each step
            if pending:
                i = pending.pop(0)
                ids[tight.add_request(jobs[i][0], jobs[i][1])] = i
        for o in tight.step():
            got.setdefault(ids[o.req_id], []).append(o.token_id)
        tight.cache.check([r.cache for r in tight.scheduler.running if r.cache is not None])
    assert tight.metrics()["preemptions"] > 0 and tight.metrics()["prefix_cache_hit_rate"] > 0
    for i, (_, sp, greedy) in enumerate(jobs):
        assert len(got[i]) == sp.max_new_tokens
        if greedy:
            assert got[i] == want[i], f"request {i}"
    assert tight.cache.num_free == 22 and not tight.scheduler.running
    tight.cache.check([])


def test_graph_cache_is_bounded_and_memory_stops_growing(model_root, monkeypatch):
    """Decode steps over 3 batch buckets, contexts that change the split of the
    keys three times, and two table widths, with room for 4 graphs only: graphs
    are evicted and captured again, device memory stops growing after the first
    pass, and every step's logits equal those of kernel-by-kernel execution."""
    from shrike_amd.cache import CacheManager
    from shrike_amd.engine import runner as runner_module
    from shrike_amd.engine.loading import load_model
    from shrike_amd.engine.runner import ModelRunner, StepEntry

    monkeypatch.setattr(runner_module, "MAX_GRAPHS", 4)
    model_dir = make_model_dir("B", model_root, dtype="bfloat16", mode="unit")
    model, rt, cfg = load_model(model_dir, "bfloat16")
    rng = random.Random(21)
    work = []  # (batch, prompt length): 3 single-token steps follow each
    for batch in (1, 3, 6):
        for length in (250, 500, 1022):  # 1022 + 3 tokens: 65 pages, the wider table; 8 splits of the keys
            work.append((batch, length, [[rng.randrange(cfg.vocab_size) for _ in range(length + 3)]
                                         for _ in range(batch)]))

    def one_pass(runner, cache):
        outs = []
        for batch, length, seqs_ids in work:
            seqs = [cache.new_sequence() for _ in range(batch)]
            for s, ids in zip(seqs, seqs_ids):
                cache.append(s, 0, length)
                runner.step([StepEntry(s, ids[:length], 0, [])])
            for k in range(3):
                entries = []
                for s, ids in zip(seqs, seqs_ids):
                    cache.append(s, length + k, 1)
                    entries.append(StepEntry(s, [ids[length + k]], length + k, [0]))
                outs.append(runner.step(entries).clone())
            for s in seqs:
                cache.free(s)
        torch.cuda.synchronize()
        return outs

    def make(graphs):
        cache = CacheManager(model.cache_specs(), 16, 6 * 65 + 2, enable_prefix_caching=False)
        cache.allocate(rt.dtype, rt.device)
        return ModelRunner(model, cache, rt, graphs=graphs), cache

    eager_runner, eager_cache = make(False)
    want = one_pass(eager_runner, eager_cache)
    graph_runner, graph_cache = make(True)
    first = one_pass(graph_runner, graph_cache)
    after_first = torch.cuda.memory_allocated()
    second = one_pass(graph_runner, graph_cache)
    after_second = torch.cuda.memory_allocated()
    assert graph_runner.graph_replays == 2 * 3 * len(work)
    assert len(graph_runner._graphs) <= 4 < graph_runner.graph_captures  # graphs were evicted
    assert len(graph_runner._graph_workspaces) == 3  # one set of buffers per batch bucket
    for a, b, c in zip(want, first, second):
        assert torch.equal(a, b) and torch.equal(a, c)
    # the second pass captures again what was evicted, into the buffers that exist
    assert after_second - after_first <= 1 << 20
    held = sum(w.nbytes() for w in graph_runner._graph_workspaces.values())
    assert held <= 8 * 6 * (cfg.vocab_size * 4 + 64 * 1024)  # a few buffers of [rows, vocab] at most


def test_bfloat16_generation_survives_preemption(model_root):
    """Pages run out in bfloat16 too: preempted requests recompute in portions
    and every token is the plain model's choice, or differs from it only where
    the plain model's two best logits nearly tie (tests/test_paged.py:88-99)."""
    from shrike_amd import SamplingParams
    from shrike_amd.engine.llm_engine import LLMEngine

    model_dir = make_model_dir("A_untied", model_root, dtype="bfloat16", mode="unit")
    plain = PlainModel(model_dir)
    prompts = prompts_for("A", [9, 14, 6, 11], seed=5)
    tight = LLMEngine(str(model_dir), dtype="bfloat16", block_size=4, num_kv_blocks=12,
                      max_tokens_per_step=7, enable_prefix_caching=False)
    got = tight.generate(prompts, SamplingParams(max_new_tokens=20, ignore_eos=True))
    assert tight.metrics()["preemptions"] > 0
    check = GreedyCheck(plain, "bfloat16")
    for prompt, out in zip(prompts, got):
        assert len(out) == 20
        check.request(prompt, out)
    check.finish()
    assert tight.cache.num_free == 12 and not tight.has_work
    tight.cache.check([])


def test_pool_sized_from_free_memory_leaves_room_for_the_step_buffers(model_root):
    from shrike_amd import SamplingParams
    from shrike_amd.config import EngineConfig
    from shrike_amd.engine.llm_engine import LLMEngine, workspace_reserve
    from shrike_amd.engine.loading import load_model

    model_dir = make_model_dir("B", model_root, dtype="bfloat16", mode="unit")
    model, rt, _ = load_model(model_dir, "bfloat16")
    cfg = EngineConfig(block_size=16, gpu_mem_util=0.001, max_tokens_per_step=300, max_running=40,
                       dtype="bfloat16")
    reserve = workspace_reserve(model, rt, cfg)
    # at least: two sets of [64 rows, vocab] float32 logits, and the slack
    assert reserve >= 2 * 64 * 503 * 4 + (64 << 20)
    free, _ = torch.cuda.mem_get_info()
    engine = LLMEngine(None, cfg, model=model, runtime=rt)
    per_page = engine.cache.bytes_per_page(2)
    assert engine.cache.num_pages <= int((free - reserve) * 0.001) // per_page + 1
    assert engine.cache.num_pages >= int((free - reserve - (1 << 30)) * 0.001) // per_page
    out = engine.generate([[5, 6, 7]], SamplingParams(max_new_tokens=4, ignore_eos=True))
    assert len(out[0]) == 4


def test_command_line_builds_a_random_model_from_a_config(tmp_path, capsys):
    """--random-config: no model folder, weights drawn on the device from the seed;
    the same seed gives the same tokens, another seed gives others."""
    import json

    from shrike_amd.__main__ import main

    path = tmp_path / "config.json"
    path.write_text(json.dumps(dict(CONFIGS["B"], torch_dtype="bfloat16")))
    runs = []
    for seed in ("3", "3", "4"):
        rc = main(["--random-config", str(path), "--prompt-len", "9", "--max-tokens", "6", "--seed", seed,
                   "--num-kv-blocks", "16", "--ignore-eos"])
        assert rc == 0
        runs.append([int(t) for t in capsys.readouterr().out.split()])
    assert len(runs[0]) == 6 and runs[0] == runs[1]
    assert main(["--random-config", str(tmp_path / "absent.json"), "--prompt-len", "3"]) == 2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recorded_launch_lists_equal_kernel_by_kernel_steps(dtype, model_root):
    """Steps that are no graph (prompt portions beside single tokens, rows that are not
    wanted) run from the recorded launches of an earlier step of the same shape.  With
    shapes that come back, shapes that do not, and a step in between that outgrows the
    buffers (which drops every list), the logits are bit for bit those of a runner that
    launches every kernel from Python."""
    from shrike_amd.cache import CacheManager
    from shrike_amd.engine.loading import load_model
    from shrike_amd.engine.runner import ModelRunner, StepEntry

    model_dir = make_model_dir("D", model_root, dtype=dtype, mode="unit")
    model, rt, cfg = load_model(model_dir, dtype)
    assert model.launches_follow_shape()
    rng = random.Random(3)
    ids = [[rng.randrange(cfg.vocab_size) for _ in range(400)] for _ in range(3)]
    # (portion of sequence 0, portion of sequence 1, single token of sequence 2?) per step: the same
    # shapes several times over, at other positions, then a larger step, then the first shapes again
    plan = ([(24, 0, True)] * 4 + [(24, 9, True)] * 3 + [(7, 0, False)] * 2 + [(120, 40, True)] + [(24, 0, True)] * 2
            + [(24, 9, True)] * 2)

    def run(graphs):
        cache = CacheManager(model.cache_specs(), 16, 90, enable_prefix_caching=False)
        cache.allocate(rt.dtype, rt.device)
        runner = ModelRunner(model, cache, rt, graphs=graphs)
        seqs = [cache.new_sequence() for _ in ids]
        at = [0, 0, 0]
        outs = []
        for n0, n1, single in plan:
            entries = []
            for s, n in ((0, n0), (1, n1), (2, 1 if single else 0)):
                if n:
                    cache.append(seqs[s], at[s], n)
                    want = [n - 1] if s != 1 else [0, n // 2]
                    entries.append(StepEntry(seqs[s], ids[s][at[s] : at[s] + n], at[s], want))
                    at[s] += n
            outs.append(runner.step(entries).cpu().clone())
            for s in range(3):
                cache.trim(seqs[s], at[s])
        return outs, runner

    plain_outs, plain_runner = run(False)
    listed_outs, listed_runner = run(True)
    assert plain_runner.list_replays == 0 and plain_runner.list_records == 0
    # shapes (24, 0), (24, 9), (7, 0), (120, 40), and (24, 0), (24, 9) once more after the large step
    assert listed_runner.list_records == 6 and listed_runner.list_replays == len(plan) - 6
    for a, b in zip(plain_outs, listed_outs):
        assert torch.isfinite(a).all() and torch.equal(a, b)


def test_a_model_with_a_part_that_decides_on_the_host_is_never_run_from_a_list(model_root):
    """Only parts that say their launches follow from the step's shape are recorded."""
    from shrike_amd.cache import CacheManager
    from shrike_amd.engine.loading import load_model
    from shrike_amd.engine.runner import ModelRunner

    model, rt, _ = load_model(make_model_dir("A", model_root), "float32")
    cache = CacheManager(model.cache_specs(), 4, 8, enable_prefix_caching=False)
    assert ModelRunner(model, cache, rt).use_call_lists
    model.blocks[0].ffn.launches_follow_shape = False  # as a part of the user's own would have it
    assert not model.launches_follow_shape()
    assert not ModelRunner(model, cache, rt).use_call_lists
