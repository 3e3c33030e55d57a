"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L] [--shape 7b]
    python bench.py --shape 14b --mixed 32      # a mixed step instead (a line of its own)

The model has the layer sizes of the Qwen2.5-7B shape (28 layers, hidden 3584,
28 query heads over 4 key/value heads of 128, intermediate 18944, vocabulary
152064) with random weights in bfloat16.  A "step" is one decode step of
the whole serving path (LLMEngine.step: schedule, forward from the paged cache,
sample, book-keeping) for `batch` requests that were each prefilled with 2,048
random tokens; decoding runs towards context 4,096 (`--context N` starts it at
N tokens instead).  One JSON line is printed: `value` is decoded tokens per
second; `prefill` is a 2,048-token prompt in one step; `roofline` prices the
decode step's unavoidable HBM reads (every weight once, the live requests'
cache) against 8 TB/s, and against the bandwidth that a plain device copy
reaches on this GPU (`achievable`); `prefill.achievable_frac` prices the prompt
against the rate of the engine's own 4096^3 product; `points` holds batch 1 and
64, the same batches at a context near 4,000, a 2,048-token prompt taken in
portions under the reference's 512-token budget, batch 8 at a context of 16,000,
and, with the layer sizes of two larger published models (`config.points_shapes`),
a step of 32 decodes beside a prompt portion (14B) and decode at batch 64 (32B);
`breakdown_us` is the decode step's time by kernel, from events around every
launch of a step that runs kernel by kernel.  The larger models' points are left
out when the run has already taken two minutes.
"""

from __future__ import annotations

import argparse
import json
import os
import random
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# Qwen2.5-7B shape
# layer sizes: the config.json files that the package ships as data
def _shape(name: str) -> dict:
    from shrike_amd.config.presets import load_preset

    return load_preset(f"qwen2.5-{name}")


SHAPE_NAMES = ("0.5b", "7b", "14b", "32b")
PROMPT_LEN = 2048
CONTEXT_END = 4096
PAGE_SIZE = 16
HBM_PEAK_GBS = 8000.0
BF16_PEAK_FLOPS = 2.5e15


def matmul_params(cfg) -> tuple[int, int]:
    """(elements of all per-layer matrices, elements of the output matrix)."""
    h, d = cfg.hidden_size, cfg.head_dim
    per_layer = (
        (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * d * h
        + cfg.num_attention_heads * d * h
        + 3 * h * cfg.intermediate_size
    )
    return per_layer * cfg.num_hidden_layers, cfg.vocab_size * h


def kv_bytes_per_token(cfg) -> int:
    return cfg.num_hidden_layers * 2 * cfg.num_key_value_heads * cfg.head_dim * 2


def prefill_flops(cfg, n: int) -> float:
    layers, head = matmul_params(cfg)
    linear = 2.0 * n * layers + 2.0 * head  # the output matrix runs on one row
    # causal attention: token p reads p + 1 keys, 2 products of head_dim each per head
    attn = 4.0 * cfg.head_dim * cfg.num_attention_heads * cfg.num_hidden_layers * n * (n + 1) / 2
    return linear + attn


def run_offline(cfg, spec, requests: int, seed: int) -> dict:
    """The reference's offline throughput run (bench/bench_engine.py:47-63, lengths as
    bench/workload.py:15-22): `requests` short prompts, 32 to 256 new tokens each, greedy,
    all handed to generate() at once, the engine with its defaults (512-token budget,
    prefix caching on).  The prompts are random ids of 24 to 72 tokens instead of the
    reference's sentences."""
    import torch

    from shrike_amd import SamplingParams
    from shrike_amd.config import EngineConfig
    from shrike_amd.engine.llm_engine import LLMEngine
    from shrike_amd.engine.loading import random_model

    model, runtime = random_model(spec, seed=seed, dtype="bfloat16")
    rng = random.Random(seed)
    prompts = [[rng.randrange(cfg.vocab_size) for _ in range(rng.randint(24, 72))] for _ in range(requests)]
    sampling = [SamplingParams(max_new_tokens=rng.randint(32, 256), ignore_eos=True) for _ in range(requests)]
    defaults = EngineConfig(dtype="bfloat16", seed=seed)
    pages = requests * (-(-(72 + 256) // defaults.block_size) + 1)
    engine = LLMEngine(None, EngineConfig(dtype="bfloat16", seed=seed, num_kv_blocks=pages), model=model,
                       runtime=runtime)
    engine.generate(prompts[:4], SamplingParams(max_new_tokens=4, ignore_eos=True), chat=False)  # first launches
    torch.cuda.synchronize()
    steps_before = engine.metrics()["steps"]
    t0 = time.perf_counter()
    outputs = engine.generate(prompts, sampling, chat=False)
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t0
    tokens = sum(len(o) for o in outputs)
    assert [len(o) for o in outputs] == [s.max_new_tokens for s in sampling]
    m = engine.metrics()
    return {"tokens": tokens, "seconds": round(seconds, 4), "tok_s": round(tokens / seconds, 1),
            "steps": m["steps"] - steps_before, "preemptions": m["preemptions"],
            "prefix_cache_hit_rate": m["prefix_cache_hit_rate"], "max_running": defaults.max_running,
            "token_budget": defaults.max_tokens_per_step, "page_size": defaults.block_size}


def make_engine(cfg, spec, max_batch: int, seed: int, budget: int | None = None):
    import torch

    from shrike_amd.config import EngineConfig
    from shrike_amd.engine.llm_engine import LLMEngine
    from shrike_amd.engine.loading import random_model

    t0 = time.perf_counter()
    model, runtime = random_model(spec, seed=seed, dtype="bfloat16")
    torch.cuda.synchronize()
    print(f"[bench] random weights on the device in {time.perf_counter() - t0:.1f}s", file=sys.stderr)
    pages = max_batch * (CONTEXT_END // PAGE_SIZE + 2)
    config = EngineConfig(
        block_size=PAGE_SIZE, num_kv_blocks=pages,
        # a whole prompt, of any context this program asks for, beside every running request's token
        max_tokens_per_step=budget if budget is not None else CONTEXT_END + max_batch,
        max_running=max_batch, enable_prefix_caching=False, dtype="bfloat16", seed=seed,
    )
    return LLMEngine(None, config, model=model, runtime=runtime)


def run_decode(engine, cfg, batch: int, steps: int, warmup: int, seed: int,
               prompt_len: int = PROMPT_LEN, temperature: float = 0.0, top_p: float = 1.0) -> dict:
    """Prefill `batch` prompts of `prompt_len` tokens, then time `steps` decode steps."""
    import torch

    from shrike_amd import SamplingParams

    rng = random.Random(seed)
    # the first requests decode while the later ones' prompts are taken in, portion by portion
    prefill_steps = batch * -(-prompt_len // engine.scheduler.max_tokens_per_step)
    sampling = SamplingParams(max_new_tokens=prefill_steps + batch + warmup + steps + 8, ignore_eos=True,
                              temperature=temperature, top_p=top_p)
    for _ in range(batch):
        engine.add_request([rng.randrange(cfg.vocab_size) for _ in range(prompt_len)], sampling)
    while engine.scheduler.waiting or not all(r.prefill_done for r in engine.scheduler.running):
        engine.step()
    for _ in range(warmup):
        engine.step()
    torch.cuda.synchronize()
    context_start = sum(r.num_computed_tokens for r in engine.scheduler.running) / batch
    t0 = time.perf_counter()
    produced = 0
    for _ in range(steps):
        produced += len(engine.step())
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    context_end = sum(r.num_computed_tokens for r in engine.scheduler.running) / batch
    assert produced == batch * steps, f"{produced} tokens from {steps} steps of {batch}"
    for req in list(engine.scheduler.running):
        engine.abort(req.req_id)
    layer_w, head_w = matmul_params(cfg)
    mean_ctx = (context_start + context_end) / 2 + 1
    step_bytes = 2.0 * (layer_w + head_w) + batch * mean_ctx * kv_bytes_per_token(cfg)
    ms = elapsed / steps * 1e3
    return {
        "tok_s": produced / elapsed, "ms_per_step": ms, "context_start": context_start,
        "context_end": context_end, "step_bytes": step_bytes,
        "gb_s": step_bytes / (ms * 1e-3) / 1e9,
    }


def run_chunked_prefill(engine, cfg, seed: int, budget: int = 512, prompt_len: int = PROMPT_LEN) -> float:
    """Milliseconds until a prompt of `prompt_len` tokens has its first token when the
    scheduler cuts it into portions of `budget` tokens (the reference's default: 512)."""
    import torch

    from shrike_amd import SamplingParams

    rng = random.Random(seed + 3)
    saved, engine.scheduler.max_tokens_per_step = engine.scheduler.max_tokens_per_step, budget
    best = None
    try:
        for _ in range(2):
            engine.add_request([rng.randrange(cfg.vocab_size) for _ in range(prompt_len)],
                               SamplingParams(max_new_tokens=1, ignore_eos=True))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            steps = 0
            while engine.has_work:
                engine.step()
                steps += 1
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            assert steps == -(-prompt_len // budget)
            best = dt if best is None else min(best, dt)
    finally:
        engine.scheduler.max_tokens_per_step = saved
    return best * 1e3


def other_shapes(args, started: float, limit: float = 120.0) -> tuple[dict, str]:
    """Points with the layer sizes of larger published models, each skipped once the
    whole run has taken `limit` seconds: a step of 32 decodes beside a portion of a
    2,048-token prompt under a 512-token budget (14B), decode at batch 64 (32B)."""
    import torch

    from shrike_amd.models.qwen2 import Qwen2Config, build_spec

    points, named = {}, []
    for shape, what in (("14b", "mixed"), ("32b", "decode")):
        if time.perf_counter() - started > limit:
            print(f"[bench] {shape} point skipped: the run has taken {time.perf_counter() - started:.0f}s", file=sys.stderr)
            continue
        cfg = Qwen2Config.from_dict(_shape(shape))
        spec = build_spec(cfg)
        named.append(f"{shape}: {cfg.num_hidden_layers} layers, hidden {cfg.hidden_size}, {cfg.num_attention_heads} heads "
                     f"over {cfg.num_key_value_heads} of {cfg.head_dim}, intermediate {cfg.intermediate_size}")
        if what == "mixed":
            engine = make_engine(cfg, spec, 33, args.seed, budget=512)
            mixed = run_mixed(engine, cfg, 32, 512, args.seed)
            points["mixed_14b_ms"] = mixed["mixed_step_ms"]
            points["decode_b32_14b_ms"] = mixed["decode_only_ms"]
            print(f"[bench] 14B sizes, 32 decodes + a portion under a 512-token budget: {mixed}", file=sys.stderr)
        else:
            engine = make_engine(cfg, spec, 64, args.seed)
            run = run_decode(engine, cfg, 64, min(args.steps, 40), args.warmup, args.seed + 64)
            points["decode_b64_32b"] = round(run["tok_s"], 1)
            points["decode_b64_32b_hbm_frac"] = round(run["gb_s"] / HBM_PEAK_GBS, 4)
            print(f"[bench] 32B sizes, batch 64: {run['tok_s']:.1f} tok/s, {run['ms_per_step']:.3f} ms/step, "
                  f"{run['gb_s']:.0f} GB/s", file=sys.stderr)
        del engine
        torch.cuda.empty_cache()
    return points, "; ".join(named)


def run_prefill(engine, cfg, seed: int, repeats: int = 3) -> dict:
    import torch

    from shrike_amd import SamplingParams

    rng = random.Random(seed + 1)
    best = None
    for _ in range(repeats):
        engine.add_request([rng.randrange(cfg.vocab_size) for _ in range(PROMPT_LEN)],
                           SamplingParams(max_new_tokens=1, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        outs = engine.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert len(outs) == 1 and outs[0].finished
        best = dt if best is None else min(best, dt)
    flops = prefill_flops(cfg, PROMPT_LEN)
    return {"value": round(PROMPT_LEN / best, 1), "tokens": PROMPT_LEN, "ms": round(best * 1e3, 3),
            "frac": round(flops / best / BF16_PEAK_FLOPS, 4)}


def measure_peaks(device="cuda:0") -> dict:
    """What this GPU reaches on the plainest work of each kind: bytes per second
    of a device-to-device copy of 2 GiB (read + write), of a read-only stream
    (the engine's one-row product with a 1 GiB matrix), and flop/s of the engine's own bfloat16 product
    at 4096 x 4096 x 4096."""
    import torch

    from shrike_amd.kernels import ops

    out = {}
    src = torch.empty(1 << 30, dtype=torch.bfloat16, device=device).normal_()
    dst = torch.empty_like(src)

    def timed(fn, repeats):
        fn()
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(repeats):
            fn()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end) / repeats * 1e-3

    nbytes = src.numel() * 2
    out["copy_gbs"] = round(2 * nbytes / timed(lambda: dst.copy_(src), 5) / 1e9, 1)
    del src, dst
    # a read-only stream: the engine's own product of one row with a 1 GiB matrix
    rows, width = 131072, 4096
    big = ops.retile_weight(torch.empty(rows, width, dtype=torch.bfloat16, device=device).normal_())
    x = torch.randn(1, width, device=device).to(torch.bfloat16)
    y = torch.empty(1, rows, dtype=torch.bfloat16, device=device)
    out["read_gbs"] = round(rows * width * 2 / timed(lambda: ops.gemm_tiled_weight(x, big, rows, width, y), 5) / 1e9, 1)
    del big
    # the matrix units alone on random operands: the power limit's ceiling for every product
    operands = torch.randn(32768, device=device).to(torch.bfloat16)
    flop = ops.mfma_alone(operands, 2048, 2048)
    out["mfma_tflops"] = round(flop / timed(lambda: ops.mfma_alone(operands, 2048, 2048), 3) / 1e12, 1)
    n = 4096
    a = torch.randn(n, n, device=device).to(torch.bfloat16)
    wt = ops.retile_weight(torch.randn(n, n, device=device).to(torch.bfloat16))
    c = torch.empty(n, n, dtype=torch.bfloat16, device=device)
    out["gemm_tflops"] = round(2.0 * n**3 / timed(lambda: ops.gemm_tiled_weight(a, wt, n, n, c), 10) / 1e12, 1)
    return out


def kernel_breakdown(engine, steps: int = 3) -> dict:
    """Microseconds per decode step by kernel: the running requests' next steps
    run kernel by kernel (no graph) with an event before and after every launch."""
    import torch

    from shrike_amd.kernels import ops

    names = ["embed", "add_rmsnorm", "act_mul", "gemm", "gemm_tiled_weight", "rope_kv_store", "attention",
             "attention_decode", "attention_prefill", "attention_prefill_shared", "argmax", "sample"]
    spans: list[tuple[str, object, object]] = []
    saved = {n: getattr(ops, n) for n in names}

    def wrap(name, fn):
        def timed(*args, **kwargs):
            label = name
            if name == "gemm_tiled_weight":  # told apart by the matrix: [m, k]
                label = f"gemm {args[2]}x{args[3]}" + (" gated" if kwargs.get("gated") else "")
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            out = fn(*args, **kwargs)
            b.record()
            spans.append((label, a, b))
            return out
        return timed

    runner = engine.runner
    # no step may be in flight or planned from before: the next ones are to run kernel by kernel
    overlap, engine.config.overlap_steps = engine.config.overlap_steps, False
    engine.step()  # takes in the step that was launched ahead, if one was, and launches none
    graphs, runner.use_graphs = runner.use_graphs, False
    lists, runner.use_call_lists = runner.use_call_lists, False
    engine._planned = None
    try:
        for n, fn in saved.items():
            setattr(ops, n, wrap(n, fn))
        engine.step()  # buffers of the kernel-by-kernel path
        spans.clear()
        for _ in range(steps):
            # the device is held back while the host queues the step's launches and
            # events, so that an event pair brackets its kernel and not the host's pace
            torch.cuda.synchronize()
            torch.cuda._sleep(30_000_000)
            engine.step()
        torch.cuda.synchronize()
    finally:
        for n, fn in saved.items():
            setattr(ops, n, fn)
        runner.use_graphs = graphs
        runner.use_call_lists = lists
        engine.config.overlap_steps = overlap
        engine._planned = None
    total: dict[str, float] = {}
    for label, a, b in spans:
        total[label] = total.get(label, 0.0) + a.elapsed_time(b) * 1e3 / steps
    return {k: round(v, 1) for k, v in sorted(total.items(), key=lambda kv: -kv[1])}


def run_mixed(engine, cfg, decodes: int, budget: int, seed: int) -> dict:
    """`decodes` requests decoding at a context of about PROMPT_LEN while one more
    PROMPT_LEN-token prompt is admitted under a token budget of `budget` a step:
    the time of the steps that hold `decodes` single tokens and a prompt portion."""
    import torch

    from shrike_amd import SamplingParams

    rng = random.Random(seed)
    sampling = SamplingParams(max_new_tokens=400, ignore_eos=True)
    for _ in range(decodes):
        engine.add_request([rng.randrange(cfg.vocab_size) for _ in range(PROMPT_LEN)], sampling)
    while engine.scheduler.waiting or not all(r.prefill_done for r in engine.scheduler.running):
        engine.step()
    for _ in range(20):
        engine.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(50):
        engine.step()
    torch.cuda.synchronize()
    decode_ms = (time.perf_counter() - t0) / 50 * 1e3
    late = engine.requests[engine.add_request([rng.randrange(cfg.vocab_size) for _ in range(PROMPT_LEN)],
                                              SamplingParams(max_new_tokens=8, ignore_eos=True))]
    full = []  # steps that use the whole budget
    while engine.scheduler.waiting or not all(r.prefill_done for r in engine.scheduler.running):
        done = late.num_computed_tokens
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step()
        torch.cuda.synchronize()
        # (a decode step that was already running when the prompt arrived is not one of them)
        if late.num_computed_tokens - done >= budget - decodes:
            full.append((time.perf_counter() - t0) * 1e3)
    for req in list(engine.scheduler.running):
        engine.abort(req.req_id)
    mean = sum(full) / len(full)
    return {"decode_only_ms": round(decode_ms, 3), "mixed_step_ms": round(mean, 3), "mixed_steps": len(full),
            "tokens_per_s": round(budget / mean * 1e3, 1)}


def run_products(cfg, tokens: list[int]) -> dict:
    """Microseconds of each of a layer's four products (and of the output head) with
    the engine's kernels and, beside them, with the vendor library's matrix product
    (torch.matmul) on the same sizes: a yardstick only, the engine never calls it.
    The engine's gate/up product includes the gate's activation and writes half the
    columns; its products of few tokens include no reader of their shares of k."""
    import statistics

    import torch

    from shrike_amd.kernels import ops

    dev = "cuda:0"

    def graph_us(fn, repeats=5):
        fn()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(repeats):
                fn()
        times = []
        for _ in range(5):
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            graph.replay()
            b.record()
            torch.cuda.synchronize()
            times.append(a.elapsed_time(b) * 1e3 / repeats)
        return statistics.median(times)

    h, inter = cfg.hidden_size, cfg.intermediate_size
    qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim
    shapes = [("qkv", qkv, h, False), ("o", h, cfg.num_attention_heads * cfg.head_dim, False),
              ("gate_up", inter, h, True), ("down", h, inter, False), ("lm_head", cfg.vocab_size, h, False)]
    out = {}
    for n in tokens:
        for name, m, k, gated in shapes:
            if name == "lm_head" and n > 64:
                continue  # the head only ever sees the rows whose logits are wanted
            rows = 2 * m if gated else m
            w = (torch.randn(rows, k, device=dev) * k**-0.5).to(torch.bfloat16)
            x = torch.randn(n, k, device=dev).to(torch.bfloat16)
            y = torch.empty(n, rows, device=dev, dtype=torch.bfloat16)
            library = graph_us(lambda: torch.matmul(x, w.t(), out=y))
            if gated:
                tiled = ops.interleave_gate_up(w[:m].contiguous(), w[m:].contiguous())
            else:
                tiled = ops.retile_weight(w)
            del w
            splits = 1 if gated else ops.gemm_splits(n, m, k)
            z = (torch.empty(splits, n, m, device=dev) if splits > 1
                 else torch.empty(n, m, device=dev, dtype=torch.bfloat16))
            if gated:
                own = graph_us(lambda: ops.gemm_tiled_weight(x, tiled, m, k, z, gated="silu"))
            else:
                own = graph_us(lambda: ops.gemm_tiled_weight(x, tiled, m, k, z, splits=splits))
            out[f"{name}_n{n}"] = {"own_us": round(own, 1), "library_us": round(library, 1), "k_shares": splits}
            print(f"[bench] {n:5d} tokens {name:8s} {rows:6d} x {k:5d}: own {own:7.1f} us ({splits} shares of k), "
                  f"library {library:7.1f} us", file=sys.stderr)
            del tiled, x, y, z
    return out


def main() -> int:
    global CONTEXT_END
    started = time.perf_counter()
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--gpus", type=int, default=int(os.environ.get("WORLD_SIZE", "1")))
    ap.add_argument("--steps", type=int, default=1900,
                    help="timed decode steps; 1900 after 2048-token prompts reach context 4,000")
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None,
                    help="run fewer layers than the configuration has (both numbers are reported)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points")
    ap.add_argument("--context", type=int, default=PROMPT_LEN, metavar="N",
                    help="start decoding at a context of N tokens (N-token prompts) instead of 2,048")
    ap.add_argument("--context-end", type=int, default=CONTEXT_END, metavar="N",
                    help="the context length the cache is made for (the configuration's 4,096; more for runs "
                         "at longer contexts)")
    ap.add_argument("--far-context", type=int, default=4000 - 64, metavar="N",
                    help="context of the extra points decode_b*_ctx4000 (0: leave them out)")
    ap.add_argument("--no-peaks", action="store_true",
                    help="skip the measurement of this GPU's copy bandwidth and product rate")
    ap.add_argument("--shape", choices=SHAPE_NAMES, default="7b",
                    help="layer sizes: Qwen2.5-7B (the default and the reported figure), 0.5B, 14B or 32B")
    ap.add_argument("--mixed", type=int, default=0, metavar="DECODES",
                    help="instead: time steps of DECODES single tokens plus a portion of a 2,048-token "
                         "prompt under a 512-token budget (prints its own JSON line)")
    ap.add_argument("--offline", type=int, default=0, metavar="REQUESTS",
                    help="instead: the reference's offline throughput run, REQUESTS short prompts with 32 to "
                         "256 new tokens each through generate() (prints its own JSON line)")
    ap.add_argument("--products", action="store_true",
                    help="instead: time a layer's matrix products at 1 to 2,048 tokens with the engine's kernels "
                         "and, as a yardstick, with the vendor library (prints its own JSON line)")
    ap.add_argument("--seed", type=int, default=0)
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    if args.steps < 1 or args.warmup < 0 or args.batch < 1:
        print("bench.py: --steps and --batch must be positive, --warmup non-negative")
        return 2
    CONTEXT_END = args.context_end
    if not 1 <= args.context < CONTEXT_END:
        print(f"bench.py: --context must lie in [1, {CONTEXT_END})")
        return 2
    room = CONTEXT_END - args.context - args.warmup - max(args.batch, 1 if args.no_points else 64) - 2
    if args.steps > room:
        print(f"bench.py: at most {room} steps fit between context {args.context} and {CONTEXT_END}")
        return 2

    import torch

    import shrike_amd.models  # noqa: F401
    from shrike_amd.models.qwen2 import Qwen2Config, build_spec

    raw = _shape(args.shape)
    layers_of_config = raw["num_hidden_layers"]
    if args.layers is not None:
        raw["num_hidden_layers"] = args.layers
    cfg = Qwen2Config.from_dict(raw)
    spec = build_spec(cfg)
    if args.products:
        products = run_products(cfg, [1, 8, 64, 512, PROMPT_LEN])
        print(json.dumps({
            "metric": f"us of a layer's matrix products, own kernels and vendor library (Qwen2.5-{args.shape.upper()} shape)",
            "unit": "us", "n_gpus": 1, "higher_is_better": False, "dtype": "bf16",
            "data": "synthetic: random operands", "products": products}))
        return 0
    if args.offline:
        offline = run_offline(cfg, spec, args.offline, args.seed)
        print(json.dumps({
            "metric": f"generated tok/s of {args.offline} requests with 32 to 256 new tokens each through "
                      f"generate() (Qwen2.5-{args.shape.upper()} shape)",
            "value": offline["tok_s"], "unit": "tok/s", "n_gpus": 1, "higher_is_better": True, "dtype": "bf16",
            "data": "synthetic: random weights N(0, 0.02), prompts of 24 to 72 random ids",
            "config": {"model": f"Qwen2.5-{args.shape.upper()} shape (Qwen2ForCausalLM)",
                       "layers": cfg.num_hidden_layers, "layers_of_config": layers_of_config,
                       "requests": args.offline, "sampling": "greedy"},
            **offline}))
        return 0
    if args.mixed:
        engine = make_engine(cfg, spec, args.mixed + 1, args.seed, budget=512)
        mixed = run_mixed(engine, cfg, args.mixed, 512, args.seed)
        print(json.dumps({
            "metric": f"ms of a step of {args.mixed} decodes plus a prompt portion, 512-token budget "
                      f"(Qwen2.5-{args.shape.upper()} shape)",
            "value": mixed["mixed_step_ms"], "unit": "ms", "n_gpus": 1, "higher_is_better": False,
            "dtype": "bf16", "data": "synthetic: random weights N(0, 0.02), prompt ids uniform in [0, vocab)",
            "config": {"model": f"Qwen2.5-{args.shape.upper()} shape (Qwen2ForCausalLM)",
                       "layers": cfg.num_hidden_layers, "layers_of_config": layers_of_config,
                       "decodes": args.mixed, "token_budget": 512, "prompt_len": PROMPT_LEN,
                       "page_size": PAGE_SIZE},
            **mixed}))
        return 0
    batches = [args.batch] if args.no_points else sorted({1, args.batch, 64})
    engine = make_engine(cfg, spec, max(batches), args.seed)

    results = {}
    for b in batches:
        results[b] = run_decode(engine, cfg, b, args.steps, args.warmup, args.seed + b, args.context)
        print(f"[bench] batch {b}: {results[b]['tok_s']:.1f} tok/s, "
              f"{results[b]['ms_per_step']:.3f} ms/step, {results[b]['gb_s']:.0f} GB/s",
              file=sys.stderr)
    # the same batches near the end of the 4,096-token context, a short run each
    far = {}
    far_steps = min(args.steps, 40)
    if args.far_context and not args.no_points and args.far_context + far_steps + args.warmup + 66 <= CONTEXT_END:
        for b in batches:
            far[b] = run_decode(engine, cfg, b, far_steps, args.warmup, args.seed + 100 + b, args.far_context)
            print(f"[bench] batch {b} at context {far[b]['context_start']:.0f}: {far[b]['tok_s']:.1f} tok/s, "
                  f"{far[b]['ms_per_step']:.3f} ms/step, {far[b]['gb_s']:.0f} GB/s", file=sys.stderr)
    # the main batch once more with temperature and a nucleus instead of the argmax, a short run
    sampled = None
    if not args.no_points:
        sampled = run_decode(engine, cfg, args.batch, min(args.steps, 200), args.warmup, args.seed + 200 + args.batch,
                             args.context, temperature=0.8, top_p=0.95)
        print(f"[bench] batch {args.batch}, temperature 0.8, top_p 0.95: {sampled['tok_s']:.1f} tok/s, "
              f"{sampled['ms_per_step']:.3f} ms/step", file=sys.stderr)
    prefill = run_prefill(engine, cfg, args.seed)
    print(f"[bench] prefill: {prefill}", file=sys.stderr)
    more_points = {}
    if not args.no_points and args.shape == "7b":
        more_points["prefill_2048_budget512_ms"] = round(run_chunked_prefill(engine, cfg, args.seed), 3)
        print(f"[bench] 2,048-token prompt in portions of 512: {more_points['prefill_2048_budget512_ms']} ms",
              file=sys.stderr)
        if 8 * (16000 // PAGE_SIZE + 16) <= engine.cache.num_pages:
            long_ms = run_chunked_prefill(engine, cfg, args.seed, budget=PROMPT_LEN, prompt_len=16000)
            more_points["prefill_16000_budget2048_ms"] = round(long_ms, 2)
            more_points["prefill_16000_bf16_frac"] = round(
                prefill_flops(cfg, 16000) / (long_ms * 1e-3) / BF16_PEAK_FLOPS, 4)
            print(f"[bench] 16,000-token prompt in portions of {PROMPT_LEN}: {long_ms:.1f} ms", file=sys.stderr)
            long_run = run_decode(engine, cfg, 8, min(args.steps, 40), args.warmup, args.seed + 300, 16000)
            more_points["decode_b8_ctx16000"] = round(long_run["tok_s"], 1)
            more_points["decode_b8_ctx16000_hbm_frac"] = round(long_run["gb_s"] / HBM_PEAK_GBS, 4)
            print(f"[bench] batch 8 at context {long_run['context_start']:.0f}: {long_run['tok_s']:.1f} tok/s, "
                  f"{long_run['ms_per_step']:.3f} ms/step, {long_run['gb_s']:.0f} GB/s", file=sys.stderr)
    # one batch left running for the per-kernel times
    from shrike_amd import SamplingParams

    rng = random.Random(args.seed + 7)
    for _ in range(args.batch):
        engine.add_request([rng.randrange(cfg.vocab_size) for _ in range(args.context)],
                           SamplingParams(max_new_tokens=64, ignore_eos=True))
    while engine.scheduler.waiting or not all(r.prefill_done for r in engine.scheduler.running):
        engine.step()
    breakdown = kernel_breakdown(engine)
    for req in list(engine.scheduler.running):
        engine.abort(req.req_id)
    print(f"[bench] decode step by kernel (us): {breakdown}", file=sys.stderr)
    peaks = None if args.no_peaks else measure_peaks()
    if peaks:
        print(f"[bench] this GPU: {peaks}", file=sys.stderr)
        prefill["gemm_tflops"] = peaks["gemm_tflops"]
        prefill["mfma_tflops"] = peaks["mfma_tflops"]  # the matrix units alone, random operands
        prefill["achievable_frac"] = round(
            prefill_flops(cfg, PROMPT_LEN) / (prefill["ms"] * 1e-3) / (peaks["gemm_tflops"] * 1e12), 4)

    graphs_on = bool(engine.config.graphs and engine.runner.use_graphs)
    points_shapes = ""
    if not args.no_points and args.shape == "7b":
        del engine
        torch.cuda.empty_cache()
        extra, points_shapes = other_shapes(args, started)
        more_points.update(extra)

    main_run = results[args.batch]
    line = {
        "metric": f"decode tok/s at batch {args.batch} (Qwen2.5-{args.shape.upper()} shape, "
                  f"{args.context}-token prompts, decoding from context "
                  f"{main_run['context_start']:.0f} to {main_run['context_end']:.0f})",
        "value": round(main_run["tok_s"], 1),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(main_run["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic: random weights N(0, 0.02), prompt ids uniform in [0, vocab)",
        "config": {
            "model": f"Qwen2.5-{args.shape.upper()} shape (Qwen2ForCausalLM)",
            "layers": cfg.num_hidden_layers,
            "layers_of_config": layers_of_config,
            "hidden": cfg.hidden_size,
            "heads": cfg.num_attention_heads,
            "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim,
            "intermediate": cfg.intermediate_size,
            "vocab": cfg.vocab_size,
            "global_batch": args.batch,
            "seq_len": CONTEXT_END,
            "prompt_len": args.context,
            "context_start": round(main_run["context_start"], 1),
            "context_end": round(main_run["context_end"], 1),
            "page_size": PAGE_SIZE,
            "parallelism": "single GPU",
            "sampling": "greedy",
            "hip_graphs": graphs_on,
            "points_shapes": points_shapes,
        },
        "prefill": prefill,
        "roofline": {
            "bound": "hbm",
            "achieved": round(main_run["gb_s"], 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(main_run["gb_s"] / HBM_PEAK_GBS, 4),
        },
        "points": {f"decode_b{b}": round(r["tok_s"], 1) for b, r in results.items() if b != args.batch},
        "breakdown_us": breakdown,
    }
    line["points"][f"decode_b{args.batch}"] = round(main_run["tok_s"], 1)
    for b, r in far.items():
        line["points"][f"decode_b{b}_ctx4000"] = round(r["tok_s"], 1)
    if sampled:
        line["points"][f"decode_b{args.batch}_top_p"] = round(sampled["tok_s"], 1)
    line["points"].update(more_points)
    if peaks:
        line["roofline"]["achievable"] = peaks["copy_gbs"]
        line["roofline"]["achievable_read"] = peaks["read_gbs"]
        line["roofline"]["achievable_frac"] = round(main_run["gb_s"] / max(peaks["copy_gbs"], peaks["read_gbs"]), 4)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
