"""The interactive session's commands, on a stand-in engine (CPU)."""

import io
from types import SimpleNamespace

from shrike_amd.repl import Session


class FakeEngine:
    def __init__(self):
        self.tokenizer = None
        self.cache = SimpleNamespace(enable_prefix_caching=True, cache_hit_blocks=3, cache_query_blocks=4)
        self.scheduler = SimpleNamespace(max_tokens_per_step=512, num_preemptions=2)
        self.model = SimpleNamespace(spec=SimpleNamespace(vocab_size=100))
        self.added, self.pending, self.stats = [], [], None

    def metrics(self):
        return {"steps": 7, "prefix_cache_hit_rate": 0.75}

    def add_request(self, ids, sampling, chat=True):
        if not ids:
            raise ValueError("empty prompt")
        self.added.append((list(ids), sampling))
        self.pending.append([len(self.added) - 1, sampling.max_new_tokens])
        return len(self.added) - 1

    @property
    def has_work(self):
        return bool(self.pending)

    def step(self):
        outs = []
        for item in list(self.pending):
            item[1] -= 1
            outs.append(SimpleNamespace(req_id=item[0], token_id=40 + item[0], finished=item[1] == 0))
            if item[1] == 0:
                self.pending.remove(item)
        return outs


def run(lines):
    engine, out = FakeEngine(), io.StringIO()
    session = Session(engine, None, out=out)
    session.run(lines)
    return engine, session, out.getvalue()


def test_settings_commands_change_the_session_and_the_engine():
    engine, session, text = run(["/temp 0", "/max 3", "/budget 64", "/cache off", "5 6 7"])
    assert session.temperature == 0.0 and session.max_new_tokens == 3
    assert engine.scheduler.max_tokens_per_step == 64
    assert engine.cache.enable_prefix_caching is False
    ids, sampling = engine.added[0]
    assert ids == [5, 6, 7] and sampling.max_new_tokens == 3 and sampling.temperature == 0.0
    assert "40 40 40" in text and "3 tokens" in text


def test_bad_arguments_are_explained_and_change_nothing():
    engine, session, text = run(["/temp -1", "/max zero", "/cache maybe", "/budget 0", "/nosuch", "/bench"])
    assert session.temperature == 0.7 and session.max_new_tokens == 512
    assert engine.scheduler.max_tokens_per_step == 512 and engine.cache.enable_prefix_caching
    for needle in ("/temp T", "/max N", "on or off", "/budget N", "no command /nosuch", "/bench N"):
        assert needle in text


def test_help_lists_every_command_and_exit_stops_the_session():
    engine, session, text = run(["/help", "/exit", "1 2 3"])
    for name in ("help", "clear", "metrics", "reset", "temp", "max", "cache", "budget", "bench",
                 "system", "exit"):
        assert f"/{name}" in text
    assert engine.added == []  # the line after /exit was never read


def test_reset_metrics_bench_and_system():
    engine, session, text = run(["/metrics", "/reset", "/bench 3 2", "/system be brief", "/system be kind",
                                 "/clear", "not numbers"])
    assert "steps = 7" in text and engine.scheduler.num_preemptions == 0
    assert engine.cache.cache_hit_blocks == 0 and engine.stats is not None
    assert len(engine.added) == 3 and "3 requests, 6 tokens" in text
    assert "system message set" in text and "system message replaced" in text
    assert session.history == []
    assert "give token ids" in text
