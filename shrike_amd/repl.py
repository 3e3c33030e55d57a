"""An interactive session on the in-process engine: python -m shrike_amd.repl

A line of text is a chat turn (a model folder without a tokenizer takes lines
of token ids instead); a line that starts with "/" is a command.  The command
names and the chat defaults (temperature 0.7, top_p 0.9, 512 new tokens) are
the reference's (shrike/cli.py:29-52, :107-111); /spec is absent because this
engine has no speculative decoding.  Every command is a method of `Session`
named `do_<name>`; its docstring is its line in /help.
"""

from __future__ import annotations

import argparse
import random
import sys
import time

from .config import DEFAULT_MODEL_DIR
from .engine.request import SamplingParams


class Quit(Exception):
    """Raised by /exit."""


class BadArgument(ValueError):
    """A command's argument could not be used; the message says what is wanted."""


def _number(text: str, kind, lowest, what: str):
    try:
        value = kind(text)
    except ValueError:
        raise BadArgument(f"{what}: {text!r} is not a number") from None
    if not value >= lowest or value == float("inf"):
        raise BadArgument(f"{what}: must be at least {lowest}, got {text}")
    return value


class Session:
    def __init__(self, engine, model_dir, out=sys.stdout):
        self.engine = engine
        self.model_dir = model_dir
        self.out = out
        self.history: list[dict[str, str]] = []
        self.temperature = 0.7
        self.top_p = 0.9
        self.max_new_tokens = 512

    def say(self, text: str = "", end: str = "\n") -> None:
        print(text, end=end, file=self.out, flush=True)

    # ---------------------------------------------------------------- commands

    def do_help(self, arg: str) -> None:
        """/help                 this list"""
        for name in sorted(n for n in dir(self) if n.startswith("do_")):
            self.say("  " + (getattr(self, name).__doc__ or name[3:]).strip())

    def do_clear(self, arg: str) -> None:
        """/clear                forget the conversation so far"""
        self.history.clear()
        self.say("history dropped")

    def do_metrics(self, arg: str) -> None:
        """/metrics              counters of the engine (steps, pages, preemptions, prefix hits)"""
        for key, value in self.engine.metrics().items():
            self.say(f"  {key} = {value}")

    def do_reset(self, arg: str) -> None:
        """/reset                set the counters of /metrics back to zero"""
        from .engine.llm_engine import EngineStats

        self.engine.stats = EngineStats()
        self.engine.cache.cache_hit_blocks = self.engine.cache.cache_query_blocks = 0
        self.engine.scheduler.num_preemptions = 0
        self.say("counters are zero again")

    def do_temp(self, arg: str) -> None:
        """/temp T               sampling temperature; 0 takes the most likely token"""
        self.temperature = _number(arg, float, 0.0, "/temp T")
        self.say(f"temperature {self.temperature:g}")

    def do_max(self, arg: str) -> None:
        """/max N                most tokens generated per turn"""
        self.max_new_tokens = _number(arg, int, 1, "/max N")
        self.say(f"up to {self.max_new_tokens} tokens per turn")

    def do_cache(self, arg: str) -> None:
        """/cache on|off         share cached pages between requests with a common prefix"""
        if arg not in ("on", "off"):
            raise BadArgument("/cache takes on or off")
        self.engine.cache.enable_prefix_caching = arg == "on"
        self.say(f"prefix sharing is {arg}")

    def do_budget(self, arg: str) -> None:
        """/budget N             tokens the scheduler puts into one step (prompts are cut to fit)"""
        self.engine.scheduler.max_tokens_per_step = _number(arg, int, 1, "/budget N")
        self.say(f"{self.engine.scheduler.max_tokens_per_step} tokens per step")

    def do_bench(self, arg: str) -> None:
        """/bench N [TOKENS]     run N requests at once (64 tokens each unless given), report tokens/s"""
        words = arg.split()
        if not words or len(words) > 2:
            raise BadArgument("/bench N [TOKENS]")
        count = _number(words[0], int, 1, "/bench N")
        tokens = _number(words[1], int, 1, "/bench TOKENS") if len(words) == 2 else 64
        rng = random.Random(0)
        vocab = self.engine.model.spec.vocab_size
        sampling = SamplingParams(max_new_tokens=tokens, ignore_eos=True)
        for _ in range(count):
            self.engine.add_request([rng.randrange(vocab) for _ in range(16)], sampling)
        t0, made, steps = time.perf_counter(), 0, 0
        while self.engine.has_work:
            made += len(self.engine.step())
            steps += 1
        dt = time.perf_counter() - t0
        self.say(f"  {count} requests, {made} tokens, {steps} steps, {dt:.2f} s: "
                 f"{made / dt:.0f} tokens/s in all, {made / dt / count:.1f} per request; "
                 f"prefix hit rate {self.engine.metrics()['prefix_cache_hit_rate']}")

    def do_system(self, arg: str) -> None:
        """/system TEXT          the system message that opens the conversation"""
        if not arg:
            raise BadArgument("/system needs the message text")
        replaced = bool(self.history) and self.history[0]["role"] == "system"
        if replaced:
            self.history[0]["content"] = arg
        else:
            self.history.insert(0, {"role": "system", "content": arg})
        self.say("system message " + ("replaced" if replaced else "set"))

    def do_exit(self, arg: str) -> None:
        """/exit                 leave"""
        raise Quit

    # ------------------------------------------------------------------- turns

    def command(self, line: str) -> None:
        name, _, arg = line[1:].strip().partition(" ")
        handler = getattr(self, "do_" + name, None)
        if handler is None:
            self.say(f"no command /{name}; /help lists them")
            return
        try:
            handler(arg.strip())
        except (BadArgument, ValueError) as error:
            self.say(f"  {error}")

    def complete(self, token_ids: list[int]):
        """Runs one request to its end, printing as it goes; (text, ids) or None."""
        sampling = SamplingParams(self.max_new_tokens, self.temperature, self.top_p)
        req_id = self.engine.add_request(token_ids, sampling, chat=False)
        tokenizer = self.engine.tokenizer
        ids, pending, text = [], [], []
        t0 = t_first = time.perf_counter()
        try:
            while self.engine.has_work:
                for out in self.engine.step():
                    if out.req_id != req_id:
                        continue
                    if not ids:
                        t_first = time.perf_counter()
                    ids.append(out.token_id)
                    if tokenizer is None:
                        self.say(str(out.token_id), end=" ")
                        continue
                    pending.append(out.token_id)
                    piece = tokenizer.decode(pending, skip_special_tokens=True)
                    if not piece.endswith("�"):  # else: a character is still incomplete
                        self.say(piece, end="")
                        text.append(piece)
                        pending.clear()
        except KeyboardInterrupt:
            self.engine.abort(req_id)
            self.say("\n(interrupted; the turn is dropped)")
            return None
        dt = time.perf_counter() - t0
        self.say(f"\n  ({len(ids)} tokens in {dt:.1f} s, {len(ids) / max(dt, 1e-9):.0f} tokens/s, "
                 f"first after {(t_first - t0) * 1e3:.0f} ms)")
        return "".join(text), ids

    def turn(self, line: str) -> None:
        if self.engine.tokenizer is None:
            try:
                token_ids = [int(t) for t in line.replace(",", " ").split()]
            except ValueError:
                self.say("no tokenizer in this model folder: give token ids, separated by spaces")
                return
            try:
                self.complete(token_ids)
            except ValueError as error:
                self.say(f"  {error}")
            return
        from .engine.llm_engine import apply_chat_template

        self.history.append({"role": "user", "content": line})
        prompt = apply_chat_template(self.model_dir, self.history)
        token_ids = list(self.engine.tokenizer.encode(prompt, add_special_tokens=False).ids)
        try:
            result = self.complete(token_ids)
        except ValueError as error:
            self.say(f"  {error}")
            result = None
        if result is None:
            self.history.pop()
        else:
            self.history.append({"role": "assistant", "content": result[0]})

    def run(self, lines) -> None:
        for line in lines:
            line = line.strip()
            if not line:
                continue
            try:
                self.command(line) if line.startswith("/") else self.turn(line)
            except Quit:
                return


def _prompted_lines(prompt: str):
    while True:
        try:
            yield input(prompt)
        except EOFError:
            print()
            return
        except KeyboardInterrupt:
            print("\n(/exit leaves)")


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m shrike_amd.repl", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", default=DEFAULT_MODEL_DIR)
    ap.add_argument("--dtype", default=None)
    ap.add_argument("--num-kv-blocks", type=int, default=None)
    args = ap.parse_args(argv)
    from .engine.llm_engine import LLMEngine

    t0 = time.perf_counter()
    engine = LLMEngine(args.model, dtype=args.dtype, num_kv_blocks=args.num_kv_blocks)
    print(f"{args.model}: {engine.cache.num_pages} cache pages, up in {time.perf_counter() - t0:.1f} s; "
          "/help lists the commands")
    Session(engine, args.model).run(_prompted_lines("shrike> "))
    return 0


if __name__ == "__main__":
    sys.exit(main())
