"""The cache manager on the CPU: pages, block tables, groups, windows, state
slots, prefix sharing.  The vectors marked with a reference file are the ones
the reference's own tests hold."""

import random

import pytest

from shrike_amd.cache import CacheManager, PageError, PagePool
from shrike_amd.parts import kv_cache_spec
from shrike_amd.parts.base import StateSpec

FULL = kv_cache_spec(num_kv_heads=2, head_dim=16)
WIN = kv_cache_spec(num_kv_heads=2, head_dim=16, window=6)


def manager(num_pages=8, page_size=4, specs=(FULL, FULL), **kw):
    return CacheManager(list(specs), page_size, num_pages, **kw)


def test_allocate_by_delta_and_free():
    # tests/test_block_manager.py:11-23 of the reference
    cm = manager(8, 4)
    seq = cm.new_sequence()
    assert cm.pages_needed(seq, 0, 10) == [3]
    cm.append(seq, 0, 10)
    assert len(seq.tables[0]) == 3 and cm.num_free == 5
    assert cm.pages_needed(seq, 10, 1) == [0]
    assert cm.pages_needed(seq, 12, 1) == [1]  # three pages hold 12 tokens
    cm.free(seq)
    assert cm.num_free == 8 and seq.tables == [[]]


def test_can_append_boundary():
    # tests/test_block_manager_edges.py:23-28
    cm = manager(2, 4)
    seq = cm.new_sequence()
    assert cm.pages_needed(seq, 0, 8) == [2]
    assert cm.can_append(seq, 0, 8) is True
    assert cm.can_append(seq, 0, 9) is False
    with pytest.raises(PageError):
        cm.append(seq, 0, 9)
    assert cm.num_free == 2  # a refused append takes nothing


def test_layers_with_the_same_need_share_a_group_others_get_their_own_pages():
    cm = manager(6, 4, specs=(FULL, WIN, FULL, None, WIN))
    assert [g.layers for g in cm.groups] == [[0, 2], [1, 4]]
    seq = cm.new_sequence()
    cm.append(seq, 0, 9)
    assert [len(t) for t in seq.tables] == [3, 3]
    assert [g.pool.num_free for g in cm.groups] == [3, 3]
    assert cm.layer_cache(2).group == 0 and cm.layer_cache(4).group == 1
    assert not cm.owns_cache(3)


def test_window_gives_pages_back_when_it_has_passed_them():
    cm = manager(6, 4, specs=(FULL, WIN))  # window 6
    seq = cm.new_sequence()
    cm.append(seq, 0, 16)
    # after 16 tokens the next query (position >= 16) reads keys > 10: pages 0 and 1 are done
    assert cm.trim(seq, 16) == 2
    assert seq.tables[1][:2] == [-1, -1] and all(p >= 0 for p in seq.tables[1][2:])
    assert all(p >= 0 for p in seq.tables[0])  # the group without a window keeps everything
    assert cm.groups[1].pool.num_free == 4 and cm.groups[0].pool.num_free == 2
    assert cm.trim(seq, 16) == 0  # nothing twice
    cm.check([seq])
    cm.free(seq)
    assert [g.pool.num_free for g in cm.groups] == [6, 6]


def test_trimmed_pages_are_used_again():
    cm = manager(3, 4, specs=(WIN,))
    seq = cm.new_sequence()
    done = 0
    used = set()
    for _ in range(20):  # 40 tokens through 3 pages of 4 with a window of 6
        assert cm.can_append(seq, done, 2)
        cm.append(seq, done, 2)
        done += 2
        cm.trim(seq, done)
        used.update(p for p in seq.tables[0] if p >= 0)
        cm.check([seq])
    assert used == {0, 1, 2} and len(seq.tables[0]) == 10


def test_state_slots_one_per_request():
    cm = manager(4, 4, specs=(FULL, StateSpec((8,))), max_slots=2)
    assert [g.layers for g in cm.state_groups] == [[1]]
    a, b = cm.new_sequence(), cm.new_sequence()
    assert {a.state_slot, b.state_slot} == {0, 1} and a.fresh_state
    with pytest.raises(PageError, match="slot"):
        cm.new_sequence()
    cm.free(a)
    c = cm.new_sequence()
    assert c.state_slot == 0
    cm.check([b, c])


def test_slots_exist_even_without_state_layers():
    cm = manager(4, 4, max_slots=3)
    assert cm.state_groups == [] and cm.slots.num_free == 3
    seq = cm.new_sequence()
    assert seq.state_slot == 0 and cm.slots.num_free == 2


def test_double_free_is_an_error():
    pool = PagePool(2)
    p = pool.take()
    pool.release(p)
    with pytest.raises(PageError, match="nobody holds"):
        pool.release(p)
    cm = manager(4, 4)
    seq = cm.new_sequence()
    cm.append(seq, 0, 5)
    cm.free(seq)
    cm.free(seq)  # tables are empty and the slot is gone: nothing happens twice
    assert cm.num_free == 4 and cm.slots.num_free == cm.slots.num_slots


def test_oldest_freed_page_is_handed_out_first():
    # shrike/engine/block_manager.py:38,51: deque, popleft
    pool = PagePool(3)
    a, b, c = pool.take(), pool.take(), pool.take()
    pool.release(b)
    pool.release(a)
    assert pool.take() == b and pool.take() == a


@pytest.mark.parametrize("seed", range(5))
def test_no_page_lost_held_twice_or_freed_twice_under_random_orders(seed):
    rng = random.Random(seed)
    cm = manager(12, 4, specs=(FULL, WIN, StateSpec((2,))), max_slots=4,
                 enable_prefix_caching=False)
    live: list = []  # (seq, tokens computed)
    for _ in range(400):
        action = rng.random()
        if action < 0.25 and len(live) < 4:
            live.append([cm.new_sequence(), 0])
        elif action < 0.8 and live:
            item = rng.choice(live)
            n = rng.choice([1, 1, 1, 2, 3, 7, 11])
            if cm.can_append(item[0], item[1], n):
                cm.append(item[0], item[1], n)
                item[1] += n
                cm.trim(item[0], item[1])
                first_needed = max(0, item[1] - 6 + 1) // 4
                assert all(p >= 0 for p in item[0].tables[1][first_needed:])
                assert all(p >= 0 for p in item[0].tables[0])
                assert all(len(t) * 4 >= item[1] for t in item[0].tables)
            else:
                assert any(
                    n_ > g.pool.num_free
                    for n_, g in zip(cm.pages_needed(item[0], item[1], n), cm.groups)
                )
        elif live:
            item = live.pop(rng.randrange(len(live)))
            cm.free(item[0])
        cm.check([s for s, _ in live])
        for gi, g in enumerate(cm.groups):
            held = sum(1 for s, _ in live for p in s.tables[gi] if p >= 0)
            assert g.pool.num_free + held == g.pool.num_pages
    for s, _ in live:
        cm.free(s)
    assert all(g.pool.num_free == g.pool.num_pages for g in cm.groups)
    assert cm.slots.num_free == 4


# ------------------------------------------------------------------ prefix sharing


def computed(cm, tokens):
    seq = cm.new_sequence()
    cm.append(seq, 0, len(tokens))
    cm.register_full_pages(seq, tokens, len(tokens))
    return seq


def test_prefix_hit_and_eviction():
    # tests/test_block_manager.py:26-57
    cm = manager(4, 4, specs=(FULL,))
    a = computed(cm, list(range(9)))
    cm.free(a)

    b = cm.new_sequence()
    cached = cm.match_prefix(b, list(range(9)))
    assert cached == 8 and len(b.tables[0]) == 2  # never the whole prompt
    cm.append(b, cached, 1)
    assert len(b.tables[0]) == 3

    c = cm.new_sequence()
    cached_c = cm.match_prefix(c, list(range(4)) + [99, 98, 97, 96, 95])
    assert cached_c == 4 and len(c.tables[0]) == 1
    assert cm.groups[0].pool.ref_count[c.tables[0][0]] == 2  # shared with b
    cm.check([b, c])

    cm.free(b)
    cm.free(c)
    d = cm.new_sequence()
    cm.append(d, 0, 16)  # an unrelated request takes every page: cached pages are evicted
    assert cm.num_free == 0
    e = cm.new_sequence()
    assert cm.match_prefix(e, list(range(9))) == 0


def test_never_matches_the_whole_prompt():
    # tests/test_block_manager_edges.py:55-67
    cm = manager(4, 4, specs=(FULL,))
    cm.free(computed(cm, list(range(8))))
    assert cm.match_prefix(cm.new_sequence(), list(range(8))) == 4


def test_chain_hash_depends_on_what_came_before():
    # tests/test_block_manager_edges.py:15-20
    h = CacheManager.chain_hash(None, [1, 2, 3])
    assert h == CacheManager.chain_hash(None, [1, 2, 3])
    assert CacheManager.chain_hash(h, [4, 5, 6]) != CacheManager.chain_hash(None, [4, 5, 6])


def test_prefix_sharing_switched_off_is_inert():
    # tests/test_block_manager_edges.py:31-37
    cm = manager(4, 4, specs=(FULL,), enable_prefix_caching=False)
    cm.free(computed(cm, list(range(9))))
    assert cm.match_prefix(cm.new_sequence(), list(range(9))) == 0


def test_prefix_sharing_is_off_where_a_window_or_state_exists():
    assert manager(4, 4, specs=(FULL, WIN)).enable_prefix_caching is False
    assert manager(4, 4, specs=(FULL, StateSpec((2,)))).enable_prefix_caching is False
    assert manager(4, 4, specs=(FULL, FULL)).enable_prefix_caching is True


def test_release_reveals_a_free_page_again():
    # tests/test_block_manager_edges.py:40-52
    cm = manager(4, 4, specs=(FULL,))
    cm.free(computed(cm, list(range(9))))
    b = cm.new_sequence()
    cm.match_prefix(b, list(range(9)))
    page = b.tables[0][0]
    assert cm.groups[0].pool.ref_count[page] == 1
    cm.release_pages(b)
    assert cm.groups[0].pool.ref_count[page] == 0 and cm.num_free == 4


def test_registration_continues_where_it_stopped():
    cm = manager(8, 4, specs=(FULL,))
    tokens = list(range(14))
    seq = cm.new_sequence()
    cm.append(seq, 0, 14)
    n, h = cm.register_full_pages(seq, tokens, 6)
    assert n == 1
    n, h = cm.register_full_pages(seq, tokens, 14, n, h)
    assert n == 3
    cm.free(seq)
    assert cm.match_prefix(cm.new_sequence(), tokens) == 12


def test_poisoned_free_pages_show_through_a_shifted_table():
    """The replay tool's poisoner on CPU tensors: keys written through a request's
    own table read back finite; the same read through a table whose entry is
    shifted to a free page, or to a page the request gave back, meets NaN."""
    import torch

    from shrike_amd.parts import kv_cache_spec
    from shrike_amd.replay.poison import PagePoisoner

    cache = CacheManager([kv_cache_spec(2, 32), kv_cache_spec(2, 32, window=8)], 4, 12, enable_prefix_caching=False)
    cache.allocate(torch.float32, "cpu")
    poisoner = PagePoisoner(cache)
    poisoner.poison_everything()
    assert all(torch.isnan(g.tensors["k"]).all() and torch.isnan(g.tensors["v"]).all() for g in cache.groups)

    def write(seq, group, first, last):
        g = cache.groups[group]
        for p in range(first, last):
            page = seq.tables[group][p // 4]
            g.tensors["k"][0, page, :, :, p % 4, :] = float(p)
            g.tensors["v"][0, page, :, :, p % 4] = float(p)

    def read(table, group, first, last):
        g = cache.groups[group]
        return torch.stack([g.tensors["k"][0, table[p // 4], :, :, p % 4, :].flatten() for p in range(first, last)])

    a, b = cache.new_sequence(), cache.new_sequence()
    cache.append(a, 0, 10)
    cache.append(b, 0, 6)
    for seq, n in ((a, 10), (b, 6)):
        write(seq, 0, 0, n)
        write(seq, 1, 0, n)
    assert torch.isfinite(read(a.tables[0], 0, 0, 10)).all()
    free_page = next(p for p in range(12) if cache.groups[0].pool.ref_count[p] == 0)
    shifted = list(a.tables[0])
    shifted[1] = free_page
    assert torch.isnan(read(shifted, 0, 4, 8)).all()  # a stale entry reads poison, not old numbers
    # the slots of a's last page beyond its 10 tokens were never written
    assert torch.isnan(read(a.tables[0], 0, 10, 12)).all()

    # the window passes a's first page: given back and poisoned, the others untouched
    before = poisoner.held(a)
    old_first = a.tables[1][0]
    cache.append(a, 10, 2)
    write(a, 0, 10, 12)
    write(a, 1, 10, 12)
    assert cache.trim(a, 12) == 1 and a.tables[1][0] == -1
    assert poisoner.poison_released(before, a) == [[], [old_first]]
    assert torch.isnan(cache.groups[1].tensors["k"][0, old_first]).all()
    assert torch.isfinite(read(a.tables[1], 1, 5, 12)).all()

    # b ends: its pages are poisoned, a's are not
    before = poisoner.held(b)
    cache.free(b)
    assert poisoner.poison_released(before) == before
    for gi, pages in enumerate(before):
        assert torch.isnan(cache.groups[gi].tensors["v"][0, pages]).all()
    assert torch.isfinite(read(a.tables[0], 0, 0, 12)).all()
    cache.free(a)
    cache.check([])
