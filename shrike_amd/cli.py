"""Interactive terminal chat with the in-process engine: python -m shrike_amd.cli

The commands and defaults are those of the reference's shrike/cli.py
(temperature 0.7, top_p 0.9, 512 new tokens; /help /clear /metrics /reset
/temp /max /cache /budget /bench /system /exit); /spec is absent because
speculative decoding is not part of this engine.  A model folder without a
tokenizer is driven with lines of token ids instead of text.
"""

from __future__ import annotations

import argparse
import sys
import time

from .config import DEFAULT_MODEL_DIR
from .engine.request import SamplingParams

HELP = """Commands:
  /help                Show this help
  /clear               Clear conversation history
  /metrics             Show engine metrics (cache hits, blocks, preemptions)
  /reset               Zero the metrics counters
  /temp <float>        Set temperature; 0 uses greedy decoding
  /max <int>           Set maximum new tokens
  /cache on|off        Toggle prefix caching live
  /budget <int>        Set scheduler token budget per step (chunked prefill)
  /bench <n> [tokens]  Fire n concurrent requests (default 64 tokens each)
                       and report aggregate throughput
  /system <text>       Set or replace the system message
  /exit                Quit"""


def _parse_args(argv=None) -> argparse.Namespace:
    parser = argparse.ArgumentParser(description="Chat with a local model")
    parser.add_argument("--model", default=DEFAULT_MODEL_DIR)
    parser.add_argument("--dtype", default=None)
    parser.add_argument("--num-kv-blocks", type=int, default=None)
    return parser.parse_args(argv)


def _run_bench(engine, count: int, tokens: int) -> None:
    import random

    rng = random.Random(0)
    vocab = engine.model.spec.vocab_size
    sampling = SamplingParams(max_new_tokens=tokens, temperature=0.0, ignore_eos=True)
    try:
        for _ in range(count):
            engine.add_request([rng.randrange(vocab) for _ in range(16)], sampling)
    except ValueError as error:
        print(f"[error] {error}")
        return
    started, generated, steps = time.perf_counter(), 0, 0
    while engine.has_work:
        generated += len(engine.step())
        steps += 1
    elapsed = time.perf_counter() - started
    hit = engine.metrics()["prefix_cache_hit_rate"]
    print(
        f"{count} reqs x {tokens} tok -> {generated} tok in {elapsed:.2f}s = "
        f"{generated / elapsed:.0f} tok/s aggregate ({generated / elapsed / count:.1f} tok/s per "
        f"request, {steps} steps, cache_hit={hit})"
    )


def _reply(engine, token_ids, temperature, max_new_tokens):
    """Run one request to its end, streaming its text (or ids); returns (text, ids)."""
    sampling = SamplingParams(max_new_tokens=max_new_tokens, temperature=temperature, top_p=0.9)
    try:
        req_id = engine.add_request(token_ids, sampling, chat=False)
    except ValueError as error:
        print(f"[error] {error}")
        return None
    generated, buf, parts = [], [], []
    started, first = time.perf_counter(), None
    try:
        while engine.has_work:
            for out in engine.step():
                if out.req_id != req_id:
                    continue
                first = first or time.perf_counter()
                generated.append(out.token_id)
                if engine.tokenizer is None:
                    print(out.token_id, end=" ", flush=True)
                    continue
                buf.append(out.token_id)
                text = engine.tokenizer.decode(buf, skip_special_tokens=True)
                if not text.endswith("�"):
                    print(text, end="", flush=True)
                    parts.append(text)
                    buf.clear()
    except KeyboardInterrupt:
        engine.abort(req_id)
        print("\n[aborted]")
        return None
    elapsed = time.perf_counter() - started
    ttft = (first - started) * 1000 if first else 0.0
    print(f"\n[{len(generated)} tok, {elapsed:.1f}s, {len(generated) / max(elapsed, 1e-9):.0f} tok/s, "
          f"TTFT {ttft:.0f}ms]")
    return "".join(parts), generated


def main(argv=None) -> None:
    args = _parse_args(argv)
    from .engine.llm_engine import EngineStats, LLMEngine, apply_chat_template

    print(f"Loading {args.model} ...", flush=True)
    t0 = time.perf_counter()
    engine = LLMEngine(args.model, dtype=args.dtype, num_kv_blocks=args.num_kv_blocks)
    print(f"ready: {args.model}, {engine.cache.num_pages} KV blocks, "
          f"loaded in {time.perf_counter() - t0:.1f}s")
    messages: list[dict[str, str]] = []
    temperature, max_new_tokens = 0.7, 512
    while True:
        try:
            line = input("shrike> ")
        except EOFError:
            print()
            break
        except KeyboardInterrupt:
            print("\nUse /exit to quit.")
            continue
        if not line.strip():
            continue
        if line.startswith("/"):
            command, _, argument = line.strip().partition(" ")
            argument = argument.strip()
            if command == "/exit":
                break
            if command == "/help":
                print(HELP)
            elif command == "/clear":
                messages.clear()
                print("Conversation cleared.")
            elif command == "/metrics":
                for key, value in engine.metrics().items():
                    print(f"{key:<24}{value}")
            elif command == "/reset":
                engine.stats = EngineStats()
                engine.cache.cache_hit_blocks = engine.cache.cache_query_blocks = 0
                engine.scheduler.num_preemptions = 0
                print("Metrics counters reset.")
            elif command == "/temp":
                try:
                    value = float(argument)
                    if not 0 <= value < float("inf"):
                        raise ValueError
                    temperature = value
                    print(f"Temperature set to {temperature:g}.")
                except ValueError:
                    print("Usage: /temp <non-negative float>")
            elif command == "/max":
                try:
                    value = int(argument)
                    if value <= 0:
                        raise ValueError
                    max_new_tokens = value
                    print(f"Maximum new tokens set to {max_new_tokens}.")
                except ValueError:
                    print("Usage: /max <positive int>")
            elif command == "/cache":
                if argument in ("on", "off"):
                    engine.cache.enable_prefix_caching = argument == "on"
                    print(f"Prefix caching {argument}.")
                else:
                    print("Usage: /cache on|off")
            elif command == "/budget":
                try:
                    value = int(argument)
                    if value < 1:
                        raise ValueError
                    engine.scheduler.max_tokens_per_step = value
                    print(f"Scheduler token budget set to {value} per step.")
                except ValueError:
                    print("Usage: /budget <positive int>")
            elif command == "/bench":
                parts = argument.split()
                try:
                    count = int(parts[0])
                    tokens = int(parts[1]) if len(parts) > 1 else 64
                    if count < 1 or tokens < 1:
                        raise ValueError
                    _run_bench(engine, count, tokens)
                except (IndexError, ValueError):
                    print("Usage: /bench <num_requests> [tokens_each]")
            elif command == "/system":
                if not argument:
                    print("Usage: /system <text>")
                elif messages and messages[0]["role"] == "system":
                    messages[0]["content"] = argument
                    print("System message updated.")
                else:
                    messages.insert(0, {"role": "system", "content": argument})
                    print("System message set.")
            else:
                print(f"Unknown command: {command}. Type /help for commands.")
            continue

        if engine.tokenizer is None:
            try:
                token_ids = [int(t) for t in line.replace(",", " ").split()]
            except ValueError:
                print("this model folder has no tokenizer: type token ids separated by spaces")
                continue
            _reply(engine, token_ids, temperature, max_new_tokens)
            continue
        messages.append({"role": "user", "content": line})
        text = apply_chat_template(args.model, messages)
        token_ids = list(engine.tokenizer.encode(text, add_special_tokens=False).ids)
        result = _reply(engine, token_ids, temperature, max_new_tokens)
        if result is None:
            messages.pop()
        else:
            messages.append({"role": "assistant", "content": result[0]})


if __name__ == "__main__":
    main()
