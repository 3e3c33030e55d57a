"""Trace replay: feeds given token ids through a model step by step and writes
the logits at the wanted places.  It samples nothing and owns no model code:
it drives the same model, step function, cache manager and kernels that
generation uses.

Input, one JSON object a line on standard input:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step in which something is wanted, OUT/<step>.f32 holds the logits at
the wanted places, in the order of the entries and of `want`, as little-endian
float32 [wanted, vocab].  After every step a line `done <step>` is printed.

--poison fills every cache page with NaN before the first step, and again each
page that a request gives back (at its end, or when a window has passed it):
a read through a stale table or beyond a request's length then shows as NaN.
--pages writes OUT/<step>.pages.json: for each entry of the step the page ids
of its block tables (one list per page group, -1 for a page given back) and
the pages this step's tokens were written to.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path


def _say(msg: str) -> None:
    print(f"[trace_run] {msg}", file=sys.stderr, flush=True)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--no-graphs", action="store_true", help="launch every step kernel by kernel")
    ap.add_argument("--poison", action="store_true",
                    help="fill pages that no request holds with NaN (at start and when given back)")
    ap.add_argument("--pages", action="store_true", help="write <step>.pages.json with the page ids used")
    args = ap.parse_args(argv)

    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)

    _say("loading kernels (compiled at the first call of a fresh checkout)")
    from ..kernels import load as load_kernels

    load_kernels()
    import numpy as np
    import torch

    from ..cache import CacheManager
    from ..engine.loading import load_model
    from ..engine.runner import ModelRunner, StepEntry
    from .poison import PagePoisoner

    _say(f"loading {args.model} as {args.dtype}")
    model, runtime, _cfg = load_model(args.model, args.dtype)
    page = args.block_size
    num_pages = max(1, -(-args.max_tokens // page))
    cache = CacheManager(model.cache_specs(), page, num_pages, max_slots=64,
                         enable_prefix_caching=False)
    cache.allocate(runtime.dtype, runtime.device)
    runner = ModelRunner(model, cache, runtime, graphs=not args.no_graphs)
    poisoner = PagePoisoner(cache) if args.poison else None
    if poisoner is not None:
        poisoner.poison_everything()
    _say(f"ready: {num_pages} pages of {page} tokens" + (", poisoned" if poisoner else ""))

    live: dict[str, tuple] = {}  # id -> (SequenceCache, tokens so far)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        msg = json.loads(line)
        step = msg["step"]
        entries, lengths, used = [], [], []
        for e in msg.get("entries", []):
            rid = str(e["id"])
            if rid not in live:
                live[rid] = [cache.new_sequence(), 0]
            seq, have = live[rid]
            tokens = [int(t) for t in e["tokens"]]
            if not tokens:
                continue
            if not cache.can_append(seq, have, len(tokens)):
                raise RuntimeError(
                    f"step {step}: request {rid!r} needs more pages than --max-tokens "
                    f"{args.max_tokens} provides ({cache.num_free} free)"
                )
            cache.append(seq, have, len(tokens))
            entries.append(StepEntry(seq, tokens, have, [int(w) for w in e.get("want", [])]))
            live[rid][1] = have + len(tokens)
            lengths.append(have + len(tokens))
            first, last = have // page, (have + len(tokens) - 1) // page
            used.append({"id": rid, "start": have, "tokens": len(tokens),
                         "tables": [list(t) for t in seq.tables],
                         "written": [list(t[first : last + 1]) for t in seq.tables]})
        if args.pages and entries:
            (out_dir / f"{step}.pages.json").write_text(json.dumps(used) + "\n")
        if entries:
            logits = runner.step(entries)
            if logits.shape[0]:
                arr = logits.detach().to("cpu", torch.float32).numpy()
                arr.astype("<f4", copy=False).tofile(out_dir / f"{step}.f32")
            else:
                torch.cuda.synchronize()
            for e, length in zip(entries, lengths):
                before = poisoner.held(e.cache) if poisoner else None
                if cache.trim(e.cache, length) and poisoner:
                    torch.cuda.synchronize()  # the step that still read them is done
                    poisoner.poison_released(before, e.cache)
        for rid in msg.get("end", []):
            rid = str(rid)
            if rid in live:
                seq = live.pop(rid)[0]
                before = poisoner.held(seq) if poisoner else None
                cache.free(seq)
                if poisoner:
                    torch.cuda.synchronize()
                    poisoner.poison_released(before)
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
