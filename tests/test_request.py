"""Request bookkeeping and sampling parameters (CPU).  The vectors are those of
the reference's tests/test_request.py."""

import pytest

from shrike_amd import SamplingParams
from shrike_amd.engine.request import Request, Status
from shrike_amd.sampling import uniform


def _req(tokens, **sp) -> Request:
    return Request(token_ids=list(tokens), sampling=SamplingParams(**sp))


def test_prompt_length_is_fixed_at_construction():
    r = _req([1, 2, 3])
    r.token_ids.extend([4, 5])
    assert (r.num_prompt_tokens, r.num_tokens, r.num_generated) == (3, 5, 2)


def test_defaults():
    r = _req([7])
    assert r.status is Status.WAITING and r.num_computed_tokens == 0
    assert r.block_table == [] and r.finish_reason is None and r.cache is None


def test_prefill_done_follows_computed_tokens():
    r = _req([1, 2, 3, 4])
    r.num_computed_tokens = 3
    assert not r.prefill_done
    r.num_computed_tokens = 4
    assert r.prefill_done


def test_ids_are_unique_and_increase():
    a, b, c = _req([1]), _req([1]), _req([1])
    assert a.req_id < b.req_id < c.req_id


def test_sampling_defaults_are_greedy():
    sp = SamplingParams()
    assert (sp.temperature, sp.top_p, sp.ignore_eos, sp.max_new_tokens) == (0.0, 1.0, False, 128)
    SamplingParams(max_new_tokens=1, temperature=0.0, top_p=1.0)
    SamplingParams(temperature=2.5, top_p=0.01)


@pytest.mark.parametrize(
    ("kwargs", "match"),
    [
        ({"max_new_tokens": 0}, "max_new_tokens"),
        ({"max_new_tokens": -1}, "max_new_tokens"),
        ({"temperature": -0.1}, "temperature"),
        ({"top_p": 0.0}, "top_p"),
        ({"top_p": 1.5}, "top_p"),
    ],
)
def test_sampling_rejects_out_of_range(kwargs, match):
    with pytest.raises(ValueError, match=match):
        SamplingParams(**kwargs)


def test_uniform_numbers_are_a_pure_function_of_seed_and_draw():
    xs = [uniform(7, i) for i in range(2000)]
    assert xs == [uniform(7, i) for i in range(2000)]
    assert all(0.0 <= x < 1.0 for x in xs)
    assert abs(sum(xs) / len(xs) - 0.5) < 0.03
    assert len(set(xs)) > 1990
    assert [uniform(8, i) for i in range(5)] != xs[:5]
