"""The scheduler's decisions (CPU): budget, portions, admission order, what
happens when pages run out.  Vectors marked with a reference file are the ones
the reference's own tests hold."""

import random

import pytest

from shrike_amd.cache import CacheManager
from shrike_amd.engine.request import Request, SamplingParams, Status
from shrike_amd.engine.scheduler import Scheduler
from shrike_amd.parts import kv_cache_spec

SPEC = kv_cache_spec(num_kv_heads=1, head_dim=16)


def req(tokens, max_new=8) -> Request:
    return Request(token_ids=list(tokens), sampling=SamplingParams(max_new_tokens=max_new))


def cache(num_pages=8, page_size=4, prefix=False, specs=(SPEC,)) -> CacheManager:
    return CacheManager(list(specs), page_size, num_pages, max_slots=16, enable_prefix_caching=prefix)


def ids(batch):
    return [(r.req_id, n) for r, n in batch]


def test_has_work_and_empty_schedule():
    # tests/test_scheduler.py:21-26
    sched = Scheduler(cache())
    assert sched.has_work is False and sched.schedule() == []
    sched.add(req(range(4)))
    assert sched.has_work is True


def test_max_running_caps_concurrency():
    # tests/test_scheduler.py:29-39
    sched = Scheduler(cache(20), max_tokens_per_step=64, max_running=1)
    a, b = req(range(4)), req(range(100, 104))
    sched.add(a)
    sched.add(b)
    assert ids(sched.schedule()) == [(a.req_id, 4)]
    assert len(sched.running) == 1 and len(sched.waiting) == 1 and b.status is Status.WAITING


def test_first_come_first_served_head_of_line_blocking():
    # tests/test_scheduler.py:42-53: the head needs 3 pages of 2; nothing overtakes it
    sched = Scheduler(cache(2), max_tokens_per_step=64, max_running=8)
    big, small = req(range(12)), req(range(4))
    sched.add(big)
    sched.add(small)
    assert sched.schedule() == []
    assert sched.running == [] and small.status is Status.WAITING
    assert sched.cache.num_free == 2 and sched.cache.slots.num_free == 16  # nothing kept


def test_chunked_prompts_and_preemption():
    # tests/test_block_manager.py:60-99 of the reference
    cm = cache(6, 4)
    sched = Scheduler(cm, max_tokens_per_step=8, max_running=4)
    long, short = req(range(20)), req(range(200, 206))
    sched.add(long)
    sched.add(short)

    batch = sched.schedule()  # budget 8: long gets 8, nothing is left
    assert ids(batch) == [(long.req_id, 8)]
    sched.postprocess(batch)
    assert long.num_computed_tokens == 8
    batch = sched.schedule()
    assert ids(batch) == [(long.req_id, 8)]
    sched.postprocess(batch)
    batch = sched.schedule()  # long ends its prompt (4), short is admitted with 4
    assert ids(batch) == [(long.req_id, 4), (short.req_id, 4)]
    sched.postprocess(batch)
    assert long.prefill_done and short.num_computed_tokens == 4

    long.token_ids.append(1000)  # a sampled token; its page is the 6th, the pool is dry
    batch = sched.schedule()
    assert ids(batch) == [(long.req_id, 1)]
    assert sched.num_preemptions == 1
    assert short.status is Status.WAITING and short.num_computed_tokens == 0 and short.cache is None
    assert sched.waiting[0] is short
    sched.postprocess(batch)

    sched.finish(long, "stop")
    assert cm.num_free == 6
    batch = sched.schedule()
    assert ids(batch) == [(short.req_id, 6)]  # recomputes its whole prompt in one portion
    sched.postprocess(batch)
    assert short.prefill_done


def test_single_tokens_come_first_and_the_budget_holds():
    sched = Scheduler(cache(32), max_tokens_per_step=10, max_running=8)
    a, b, c = req(range(3)), req(range(10, 17)), req(range(20, 40))
    for r in (a, b, c):
        sched.add(r)
    batch = sched.schedule()
    assert ids(batch) == [(a.req_id, 3), (b.req_id, 7)]
    sched.postprocess(batch)
    a.token_ids.append(1)
    b.token_ids.append(2)
    batch = sched.schedule()  # two decodes cost 2, c's prompt is cut to the remaining 8
    assert ids(batch) == [(a.req_id, 1), (b.req_id, 1), (c.req_id, 8)]
    assert sum(n for _, n in batch) <= 10


def test_a_request_that_is_itself_the_newest_sits_out():
    cm = cache(2, 4)
    sched = Scheduler(cm, max_tokens_per_step=64)
    a = req(range(8))
    sched.add(a)
    sched.postprocess(sched.schedule())
    a.token_ids.append(7)  # needs a third page; a is the only and newest running request
    assert sched.schedule() == []  # it preempted itself, and the pool is too small to re-admit 9
    assert sched.num_preemptions == 1 and a.status is Status.WAITING and cm.num_free == 2


def test_resumed_request_recomputes_prompt_and_generated_tokens_in_portions():
    cm = cache(8, 4)
    sched = Scheduler(cm, max_tokens_per_step=6)
    a = req(range(5))
    sched.add(a)
    sched.postprocess(sched.schedule())
    a.token_ids += [50, 51, 52]  # generated before a preemption
    sched._preempt_newest()
    assert a.num_computed_tokens == 0 and a.cache is None
    batch = sched.schedule()
    assert ids(batch) == [(a.req_id, 6)]
    sched.postprocess(batch)
    batch = sched.schedule()
    assert ids(batch) == [(a.req_id, 2)]  # reaches its last known token: the engine samples here
    sched.postprocess(batch)
    assert a.num_computed_tokens == a.num_tokens == 8


def test_failed_admission_rolls_back_prefix_references():
    # tests/test_review_regressions.py:17-39
    cm = cache(2, 4, prefix=True)
    first = cm.new_sequence()
    cm.append(first, 0, 5)
    cm.register_full_pages(first, list(range(5)), 5)
    cm.free(first)
    hog = cm.new_sequence()
    cm.append(hog, 0, 4)
    assert cm.num_free == 1
    sched = Scheduler(cm, max_tokens_per_step=64)
    b = req(list(range(5)) + [99, 98, 97])  # hits the cached first page, but its tail needs two more
    sched.add(b)
    assert sched.schedule() == []
    assert b.cache is None and b.num_computed_tokens == 0 and b.block_table == []
    assert cm.num_free == 1
    cm.check([hog])


def test_prefix_hit_shortens_the_first_portion():
    cm = cache(8, 4, prefix=True)
    sched = Scheduler(cm, max_tokens_per_step=64)
    a = req(range(10))
    sched.add(a)
    sched.postprocess(sched.schedule())
    sched.finish(a, "stop")
    b = req(list(range(10)) + [77])
    sched.add(b)
    assert ids(sched.schedule()) == [(b.req_id, 3)]  # two pages of 4 are shared
    assert b.num_computed_tokens == 8
    assert cm.cache_hit_blocks == 2


def test_window_pages_come_back_during_a_long_request():
    win = kv_cache_spec(num_kv_heads=1, head_dim=16, window=5)
    cm = cache(4, 4, specs=(win,))
    sched = Scheduler(cm, max_tokens_per_step=4)
    a = req(range(40), max_new=1)  # 10 pages worth of prompt through a pool of 4
    sched.add(a)
    steps = 0
    while not a.prefill_done:
        batch = sched.schedule()
        assert batch, "a window must let a long prompt through a small pool"
        sched.postprocess(batch)
        steps += 1
    assert steps == 10 and sched.num_preemptions == 0


@pytest.mark.parametrize("seed", range(4))
def test_random_workloads_keep_the_invariants(seed):
    rng = random.Random(seed)
    cm = cache(10, 4)
    sched = Scheduler(cm, max_tokens_per_step=12, max_running=3)
    todo = [req([rng.randrange(100) for _ in range(rng.randint(1, 14))], max_new=rng.randint(1, 6))
            for _ in range(12)]
    for r in todo:
        sched.add(r)
    finished, steps = 0, 0
    while sched.has_work:
        steps += 1
        assert steps < 2000
        batch = sched.schedule()
        assert sum(n for _, n in batch) <= 12 and len(sched.running) <= 3
        singles = [n == 1 for _, n in batch]
        assert singles == sorted(singles, reverse=True)  # single tokens first
        assert len({r.req_id for r, _ in batch}) == len(batch)
        for r, n in batch:
            assert r.status is Status.RUNNING
            assert len(r.cache.tables[0]) * 4 >= r.num_computed_tokens + n
        sched.postprocess(batch)
        for r, n in batch:
            if r.num_computed_tokens == r.num_tokens:
                r.token_ids.append(rng.randrange(100))
                if r.num_generated >= r.sampling.max_new_tokens:
                    sched.finish(r, "length")
                    finished += 1
        cm.check([r.cache for r in sched.running])
    assert finished == 12 and cm.num_free == 10 and cm.slots.num_free == 16


@pytest.mark.parametrize("seed", range(6))
def test_a_planned_decode_step_is_the_step_that_schedule_would_give(seed):
    """Two schedulers get the same requests, arrivals and tokens.  One plans its
    next step ahead whenever plan_decode_step() offers one (before the step's
    tokens exist); the other always calls schedule().  Their batches and their
    pools agree at every step, through admissions, ends and preemptions."""
    rng = random.Random(seed)
    cms = [cache(9, 4), cache(9, 4)]
    scheds = [Scheduler(cm, max_tokens_per_step=10, max_running=4) for cm in cms]
    arrivals = sorted((rng.randrange(60), [rng.randrange(50) for _ in range(rng.randint(1, 9))],
                       rng.randint(1, 12)) for _ in range(10))
    reqs = [{}, {}]  # arrival number -> request, per scheduler
    planned, steps, plans_used = None, 0, 0
    while arrivals or any(s.has_work for s in scheds):
        steps += 1
        assert steps < 3000
        while arrivals and arrivals[0][0] <= steps:
            _, tokens, max_new = arrivals.pop(0)
            for which in (0, 1):
                r = req(tokens, max_new)
                reqs[which][len(reqs[which])] = r
                scheds[which].add(r)
            planned = None  # as the engine does when a request arrives
        if planned is not None:
            plans_used += 1
        batches = [planned if planned is not None else scheds[0].schedule(), scheds[1].schedule()]
        number = [{r.req_id: k for k, r in reqs[w].items()} for w in (0, 1)]
        assert [(number[0][r.req_id], n) for r, n in batches[0]] == \
               [(number[1][r.req_id], n) for r, n in batches[1]]
        assert cms[0].num_free == cms[1].num_free
        for w in (0, 1):
            scheds[w].postprocess(batches[w])
        ends = [r.num_computed_tokens == r.num_tokens for r, _ in batches[0]]
        planned = scheds[0].plan_decode_step() if all(ends) and batches[0] else None
        token = rng.randrange(50)
        for w in (0, 1):
            for (r, _), end in zip(list(batches[w]), ends):
                if end:
                    r.token_ids.append(token)
                    if r.num_generated >= r.sampling.max_new_tokens:
                        scheds[w].finish(r, "length")
                        if w == 0:
                            planned = None
            cms[w].check([r.cache for r in scheds[w].running])
    assert plans_used > 5
    assert all(cm.num_free == 9 for cm in cms)
