"""python -m shrike_amd: stream one completion through the engine.

The options are those of the reference's scripts/chat.py (prompt, --max-tokens,
--temperature, --model) and of its server's engine flags
(--max-tokens-per-step, --max-running, --no-prefix-caching); the rest expose
the engine's own options.  Without a tokenizer in the model folder, give the
prompt as token ids (--prompt-ids) or as a length of random ids (--prompt-len).
"""

from __future__ import annotations

import argparse
import random
import sys
import time

from .config import DEFAULT_MODEL_DIR
from .engine.request import SamplingParams


def parse_args(argv=None) -> argparse.Namespace:
    ap = argparse.ArgumentParser(prog="python -m shrike_amd", description=__doc__.split("\n\n")[0])
    ap.add_argument("prompt", nargs="?", default=None, help="text prompt (needs tokenizer.json)")
    ap.add_argument("--model", default=DEFAULT_MODEL_DIR)
    ap.add_argument("--random-config", default=None, metavar="CONFIG_JSON",
                    help="instead of --model: a config.json (or a folder with one, or the name of a preset: "
                         "qwen2.5-0.5b, -7b, -14b, -32b) whose architecture is built with random weights "
                         "drawn on the device from --seed")
    ap.add_argument("--prompt-ids", default=None, help="comma-separated token ids")
    ap.add_argument("--prompt-len", type=int, default=None, help="that many random token ids")
    ap.add_argument("--max-tokens", type=int, default=128)
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--ignore-eos", action="store_true")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-chat", action="store_true", help="do not wrap a text prompt in the chat template")
    ap.add_argument("--dtype", choices=["bfloat16", "float32", "bf16", "fp32"], default=None)
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--num-kv-blocks", type=int, default=None)
    ap.add_argument("--gpu-mem-util", type=float, default=0.85)
    ap.add_argument("--max-tokens-per-step", type=int, default=512)
    ap.add_argument("--max-running", type=int, default=256)
    ap.add_argument("--no-prefix-caching", action="store_true")
    ap.add_argument("--no-graphs", action="store_true", help="run decode steps kernel by kernel")
    ap.add_argument("--no-overlap", action="store_true",
                    help="launch a decode step only when the tokens of the step before are on the host")
    ap.add_argument("--metrics", action="store_true", help="print engine metrics at the end")
    return ap.parse_args(argv)


def main(argv=None) -> int:
    args = parse_args(argv)
    from .engine.llm_engine import LLMEngine

    t0 = time.perf_counter()
    options = dict(
        block_size=args.block_size, gpu_mem_util=args.gpu_mem_util,
        max_tokens_per_step=args.max_tokens_per_step, max_running=args.max_running,
        enable_prefix_caching=not args.no_prefix_caching, num_kv_blocks=args.num_kv_blocks,
        dtype=args.dtype, seed=args.seed, graphs=not args.no_graphs, overlap_steps=not args.no_overlap,
    )
    if args.random_config is not None:
        import json
        import os

        from .config import EngineConfig, architecture_name, canonical_dtype, get_architecture
        from .engine.loading import random_model

        from .config.presets import load_preset, preset_names

        path = args.random_config
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        try:
            if not os.path.exists(path) and path.lower() in preset_names():
                raw = load_preset(path)
            else:
                with open(path) as f:
                    raw = json.load(f)
        except (OSError, ValueError) as e:
            print(f"[error] --random-config {path}: {e} (presets: {', '.join(preset_names())})", file=sys.stderr)
            return 2
        arch = get_architecture(architecture_name(raw))
        spec = arch.build_spec(arch.config_cls.from_dict(raw))
        dtype = canonical_dtype(args.dtype) if args.dtype else spec.stored_dtype
        model, runtime = random_model(spec, seed=args.seed, dtype=dtype)
        engine = LLMEngine(None, EngineConfig(**dict(options, dtype=dtype)), model=model, runtime=runtime)
    else:
        engine = LLMEngine(args.model, **options)
    print(f"[engine up in {time.perf_counter() - t0:.1f}s, {engine.cache.num_pages} KV blocks]",
          file=sys.stderr)
    if args.prompt_ids is not None:
        prompt = [int(t) for t in args.prompt_ids.replace(" ", "").split(",") if t]
    elif args.prompt_len is not None:
        rng = random.Random(args.seed)
        prompt = [rng.randrange(engine.model.spec.vocab_size) for _ in range(args.prompt_len)]
    elif args.prompt is not None:
        prompt = args.prompt
    else:
        print("give a prompt, --prompt-ids or --prompt-len", file=sys.stderr)
        return 2
    sampling = SamplingParams(args.max_tokens, args.temperature, args.top_p, args.ignore_eos, args.seed)
    try:
        engine.add_request(prompt, sampling, chat=not args.no_chat)
    except ValueError as e:
        print(f"[error] {e}", file=sys.stderr)
        return 2

    buf: list[int] = []
    t0, n = time.perf_counter(), 0
    while engine.has_work:
        for out in engine.step():
            n += 1
            if engine.tokenizer is None:
                print(out.token_id, end=" ", flush=True)
                continue
            buf.append(out.token_id)
            text = engine.tokenizer.decode(buf, skip_special_tokens=True)
            if not text.endswith("�"):  # wait for the rest of a split character
                print(text, end="", flush=True)
                buf.clear()
    dt = time.perf_counter() - t0
    print(f"\n[{n} tokens in {dt:.2f}s = {n / max(dt, 1e-9):.1f} tok/s]", file=sys.stderr)
    if args.metrics:
        for key, value in engine.metrics().items():
            print(f"{key:<24}{value}", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
