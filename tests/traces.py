"""Builds replay traces (the four ways of cutting a set of requests) and runs
bin/trace_run on them."""

from __future__ import annotations

import json
import os
import random
import subprocess
import sys
from pathlib import Path

import numpy as np

REPO = Path(__file__).resolve().parent.parent
TRACE_RUN = REPO / "bin" / "trace_run"


def run_trace(model_dir, dtype: str, steps: list[dict], max_tokens: int, out_dir, vocab: int,
              timeout: int = 600, block_size: int | None = None, poison: bool = False,
              pages: bool = False) -> dict[int, np.ndarray]:
    """-> {step: float32 [wanted, vocab]} for the steps that wanted something."""
    out_dir = Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    text = "".join(json.dumps(s) + "\n" for s in steps)
    extra = ([] if block_size is None else ["--block-size", str(block_size)]) \
        + (["--poison"] if poison else []) + (["--pages"] if pages else [])
    proc = subprocess.run(
        [sys.executable, str(TRACE_RUN), "--model", str(model_dir), "--dtype", dtype,
         "--out", str(out_dir), "--max-tokens", str(max_tokens), *extra],
        input=text, capture_output=True, text=True, timeout=timeout, env=dict(os.environ),
    )
    if proc.returncode != 0:
        raise RuntimeError(f"trace_run exited with {proc.returncode}:\n{proc.stderr[-3000:]}")
    done = [int(line.split()[1]) for line in proc.stdout.splitlines() if line.startswith("done ")]
    assert done == [s["step"] for s in steps], "every step must be acknowledged in order"
    out = {}
    for s in steps:
        wanted = sum(len(e.get("want", [])) for e in s["entries"])
        path = out_dir / f"{s['step']}.f32"
        if wanted:
            out[s["step"]] = np.fromfile(path, dtype="<f4").reshape(wanted, vocab)
        else:
            assert not path.exists()
    return out


class TraceBuilder:
    """Collects steps and remembers which (request, position) each written row is."""

    def __init__(self):
        self.steps: list[dict] = []
        self.rows: dict[int, list[tuple[str, int]]] = {}

    def add(self, entries: list[tuple[str, list[int], int, list[int]]], end=()):
        """entries: (id, tokens, position of the first token, wanted offsets)."""
        step = len(self.steps)
        self.steps.append({
            "step": step,
            "entries": [{"id": rid, "tokens": toks, "want": want} for rid, toks, _, want in entries],
            "end": list(end),
        })
        self.rows[step] = [(rid, start + w) for rid, _, start, want in entries for w in want]
        return step

    def collect(self, outputs: dict[int, np.ndarray]) -> dict[tuple[str, int], np.ndarray]:
        got = {}
        for step, rows in self.rows.items():
            for i, key in enumerate(rows):
                assert key not in got, f"{key} written twice"
                got[key] = outputs[step][i]
        return got


def read_pages(out_dir, steps: list[dict]) -> dict[int, list[dict]]:
    """{step: what --pages wrote for it}."""
    out = {}
    for s in steps:
        path = Path(out_dir) / f"{s['step']}.pages.json"
        if path.exists():
            out[s["step"]] = json.loads(path.read_text())
    return out


def check_pages(steps: list[dict], pages: dict[int, list[dict]], page_size: int, num_pages: int) -> int:
    """What the page ids of a replay must satisfy: tables cover the tokens, ids lie
    in the pool, no page is held by two live requests, and a request keeps its
    pages from step to step.  Returns how many times a page was handed to a
    request after another request had held it."""
    reused = 0
    groups = max((len(rec["tables"]) for recs in pages.values() for rec in recs), default=0)
    for g in range(groups):
        owner: dict[int, str] = {}  # page -> live request that holds it
        seen_before: set[int] = set()
        last_table: dict[str, list[int]] = {}
        for s in steps:
            for rec in pages.get(s["step"], []):
                rid, table = rec["id"], rec["tables"][g]
                assert len(table) * page_size >= rec["start"] + rec["tokens"]
                assert all(-1 <= p < num_pages for p in table)
                prev = last_table.get(rid, [])
                assert all(a == b or b == -1 for a, b in zip(prev, table)), "a request's pages changed under it"
                for a, b in zip(prev, table):  # given back by a window
                    if a >= 0 and b == -1:
                        seen_before.add(a)
                        owner.pop(a, None)
                for p in table[len(prev):]:
                    if p == -1:
                        continue  # taken and passed by the window within one step
                    assert owner.get(p, rid) == rid, f"group {g}: page {p} is held twice"
                    reused += p in seen_before
                    owner[p] = rid
                last_table[rid] = table
                first = rec["start"] // page_size
                written = rec["written"][g]
                assert written == table[first : first + len(written)] and min(written) >= 0
            for rid in s.get("end", []):
                for p in last_table.pop(rid, []):
                    if p >= 0:
                        seen_before.add(p)
                        owner.pop(p, None)
    return reused


def round64(n: int) -> int:
    return -(-n // 64) * 64


def whole(tb: TraceBuilder, prefix: str, seqs: dict[str, list[int]]):
    for name, ids in seqs.items():
        tb.add([(prefix + name, ids, 0, list(range(len(ids))))], end=[prefix + name])
    return max(round64(len(ids)) for ids in seqs.values())


def last_one_by_one(tb: TraceBuilder, prefix: str, seqs: dict[str, list[int]], tail: int = 32):
    for name, ids in seqs.items():
        rid, head = prefix + name, max(1, len(ids) - tail)
        tb.add([(rid, ids[:head], 0, list(range(head)))])
        for p in range(head, len(ids)):
            tb.add([(rid, [ids[p]], p, [0])], end=[rid] if p == len(ids) - 1 else [])
        if head == len(ids):
            tb.add([], end=[rid])
    return max(round64(len(ids)) for ids in seqs.values())


def changing_portions(tb: TraceBuilder, prefix: str, seqs: dict[str, list[int]],
                      sizes=(7, 2, 5, 3, 2, 16, 1, 9, 2, 31, 4)):
    for name, ids in seqs.items():
        rid, p, k = prefix + name, 0, 0
        while p < len(ids):
            n = min(sizes[k % len(sizes)], len(ids) - p)
            k += 1
            tb.add([(rid, ids[p : p + n], p, list(range(n)))], end=[rid] if p + n == len(ids) else [])
            p += n
    return max(round64(len(ids)) for ids in seqs.values())


def mixed(tb: TraceBuilder, prefix: str, seqs: dict[str, list[int]], max_tokens: int, seed: int = 0,
          max_live: int = 4):
    """Up to four live requests, portions of some beside single tokens of
    others; a request starts as soon as its rounded length fits under
    max_tokens, so pages of finished requests are used again."""
    rng = random.Random(seed)
    waiting = list(seqs.items())
    live: dict[str, list] = {}  # name -> [ids, cursor]
    held = 0
    while waiting or live:
        while waiting and len(live) < max_live and held + round64(len(waiting[0][1])) <= max_tokens:
            name, ids = waiting.pop(0)
            live[name] = [ids, 0]
            held += round64(len(ids))
        assert live, "max_tokens is too small for the next request"
        entries, end = [], []
        for name, item in list(live.items()):
            ids, p = item
            if rng.random() < 0.15 and len(live) > 1:
                continue  # left out of this step, goes on later
            left = len(ids) - p
            in_prompt = p < len(ids) * 2 // 3
            n = min(left, rng.choice([2, 3, 5, 8, 13, 21]) if in_prompt else 1)
            want = list(range(n)) if n <= 4 else sorted(rng.sample(range(n), 3)) + [n - 1]
            want = sorted(set(want))
            entries.append((prefix + name, ids[p : p + n], p, want))
            item[1] = p + n
            if item[1] == len(ids):
                end.append(prefix + name)
                held -= round64(len(ids))
                del live[name]
        if entries or end:
            tb.add(entries, end=end)
