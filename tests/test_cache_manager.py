"""The cache manager: no page lost, held twice or freed twice, under random orders of requests."""
import random

import pytest

from xyntetik_runner_amd.cache import CacheManager, OutOfPages, Pool, first_needed_position
from xyntetik_runner_amd.parts.base import KVSpec

FULL = KVSpec(2, 16, None)
WIN = KVSpec(1, 32, 10)


def test_pool_basics():
    p = Pool(3, first=1)
    a, b, c = p.take(), p.take(), p.take()
    assert sorted([a, b, c]) == [1, 2, 3] and p.n_free == 0
    with pytest.raises(OutOfPages):
        p.take()
    p.give(b)
    with pytest.raises(ValueError):
        p.give(b)                      # freed twice
    with pytest.raises(ValueError):
        p.give(99)                     # never handed out
    assert p.take() == b               # the page just freed is used again first
    with pytest.raises(OutOfPages):
        p.take_many(2)
    p.check()


def test_reserve_is_all_or_nothing_across_groups():
    m = CacheManager([FULL, WIN], page_size=4, pages_per_group=3, n_slots=2)
    m.admit("a")
    m.reserve("a", 8)
    m.advance("a", 8)
    before = [m.free_pages(0), m.free_pages(1)]
    with pytest.raises(OutOfPages):
        m.reserve("a", 20)             # 5 pages wanted, 3 exist
    assert [m.free_pages(0), m.free_pages(1)] == before and len(m.get("a").tables[0]) == 2
    m.check()


def test_block_table_addresses_every_position():
    m = CacheManager([FULL], page_size=4, pages_per_group=8, n_slots=4)
    m.admit("a"); m.admit("b")
    m.reserve("a", 5); m.advance("a", 5)
    m.reserve("b", 9); m.advance("b", 9)
    m.reserve("a", 13); m.advance("a", 13)
    ta, tb = m.get("a").tables[0], m.get("b").tables[0]
    assert len(ta) == 4 and len(tb) == 3 and not set(ta) & set(tb) and 0 not in ta + tb
    m.check()
    m.release("a")
    assert m.free_pages(0) == 8 - 3
    m.admit("c")
    m.reserve("c", 4)
    assert m.get("c").tables[0][0] in ta          # a freed page is used again
    assert m.get("c").fresh
    m.advance("c", 4)
    assert not m.get("c").fresh
    m.check()


def test_window_group_gives_pages_back_as_the_window_passes():
    m = CacheManager([FULL, WIN], page_size=4, pages_per_group=6, n_slots=1)
    m.admit("a")
    n = 0
    for step in (3, 2, 7, 1, 1, 5, 1):
        m.reserve("a", n + step)
        n += step
        m.advance("a", n)
        m.check()
        lo = first_needed_position(n, WIN.window)
        t_full, t_win = m.get("a").tables
        assert all(p >= 0 for p in t_full)
        for i, p in enumerate(t_win):
            assert (p < 0) == ((i + 1) * 4 <= lo), (n, i, p, lo)
    assert n == 20 and m.free_pages(1) == 6 - 3 and m.free_pages(0) == 6 - 5
    m.release("a")
    assert m.free_pages(0) == 6 and m.free_pages(1) == 6 and m.slots.n_free == 1
    m.check()


def test_first_needed_position():
    assert first_needed_position(0, None) == 0 and first_needed_position(100, None) == 0
    assert first_needed_position(5, 10) == 0 and first_needed_position(10, 10) == 1 and first_needed_position(25, 10) == 16


def test_slots_run_out_and_come_back():
    m = CacheManager([FULL], page_size=4, pages_per_group=8, n_slots=2)
    a, b = m.admit("a"), m.admit("b")
    assert a.slot != b.slot and not m.can_admit()
    with pytest.raises(OutOfPages):
        m.admit("c")
    with pytest.raises(ValueError):
        m.admit("a")
    m.release("a")
    assert m.admit("c").slot == a.slot
    m.check()


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_keep_every_invariant(seed):
    rng = random.Random(seed)
    page_size = rng.choice([1, 2, 4, 16])
    groups = [FULL, WIN] if seed % 2 else [FULL]
    m = CacheManager(groups, page_size=page_size, pages_per_group=rng.randint(6, 20), n_slots=4)
    live, next_id = {}, 0
    for _ in range(400):
        op = rng.random()
        if op < 0.25 and m.can_admit():
            m.admit(next_id)
            live[next_id] = 0
            next_id += 1
        elif op < 0.8 and live:
            rid = rng.choice(list(live))
            grow = rng.randint(1, 3 * page_size + 2)
            free_before = [m.free_pages(g) for g in range(len(groups))]
            ok = m.can_reserve(rid, live[rid] + grow)
            try:
                m.reserve(rid, live[rid] + grow)
                assert ok
                live[rid] += grow
                m.advance(rid, live[rid])
            except OutOfPages:
                assert not ok
                assert [m.free_pages(g) for g in range(len(groups))] == free_before
        elif live:
            rid = rng.choice(list(live))
            m.release(rid)
            del live[rid]
        m.check()
        assert m.tokens_held() == sum(live.values())
    for rid in list(live):
        m.release(rid)
    m.check()
    assert all(m.free_pages(g) == m.pages_per_group for g in range(len(groups))) and m.slots.n_free == 4


def test_trim_gives_back_what_a_step_reserved_and_did_not_run():
    m = CacheManager([FULL, WIN], page_size=4, pages_per_group=8, n_slots=2)
    m.admit("a")
    m.reserve("a", 6); m.advance("a", 6)
    free = [m.free_pages(0), m.free_pages(1)]
    m.reserve("a", 19)                 # three more pages in each group; then the step fails
    assert m.free_pages(0) == free[0] - 3
    m.trim("a")
    assert [m.free_pages(0), m.free_pages(1)] == free and m.get("a").n_tokens == 6
    assert m.pages_needed_new(9) == [3, 3]
    m.check()
    m.reserve("a", 7); m.advance("a", 7)
    m.check()


def test_a_reader_may_not_look_further_back_than_the_cache_it_reads_keeps():
    """An entry of the run order that reads another entry's cache with a wider window, or with
    none, would look up pages that the owner's window has given back."""
    import torch
    from xyntetik_runner_amd.cache import CacheStorage
    dev = torch.device("cpu")
    own, narrow, wide, full = KVSpec(1, 16, 8), KVSpec(1, 16, 4), KVSpec(1, 16, 12), KVSpec(1, 16, None)
    ok = CacheStorage([own, narrow, own], [None] * 3, [None, 0, 0], 4, 3, 2, torch.float32, dev)
    assert [lc.owns for lc in ok.layers] == [True, False, False] and ok.layers[1].k is ok.layers[0].k
    for reader in (wide, full):
        with pytest.raises(ValueError, match="keeps only the last 8 keys"):
            CacheStorage([own, reader], [None] * 2, [None, 0], 4, 3, 2, torch.float32, dev)
    # an owner that keeps every key serves any reader
    CacheStorage([full, narrow, full], [None] * 3, [None, 0, 0], 4, 3, 2, torch.float32, dev)


# ----------------------------------------------------------------------------- pools of different sizes
def test_groups_have_pools_of_their_own_size():
    from xyntetik_runner_amd.cache import pages_for_spec
    # 2 requests, steps of at most 8 tokens, pages of 4: a window of 10 touches 3 pages, plus the one
    # being filled and the one not yet given back, plus the step's own 2
    assert pages_for_spec(WIN, 4, max_tokens=4000, max_requests=2, max_step_tokens=8) == 2 * (3 + 2) + 2
    assert pages_for_spec(FULL, 4, max_tokens=4000, max_requests=2, max_step_tokens=8) == 1000
    assert pages_for_spec(WIN, 4, max_tokens=4000, max_requests=2) == 1000         # steps of any size
    assert pages_for_spec(WIN, 4, max_tokens=20, max_requests=2, max_step_tokens=8) == 5      # never more than the tokens' pages
    m = CacheManager([FULL, WIN], page_size=4, pages_per_group=[40, 10], n_slots=2)
    assert [g.pool.size for g in m.groups] == [40, 10]
    assert m.capacity_tokens() == 160                       # the group that keeps every key sets the limit
    assert m.max_portion() == (10 - 4) * 4                  # the windowed one what a step can bring
    with pytest.raises(ValueError):
        CacheManager([FULL, WIN], page_size=4, pages_per_group=[40], n_slots=2)
    with pytest.raises(ValueError):
        CacheManager([FULL, WIN], page_size=4, pages_per_group=[40, 0], n_slots=2)


def test_a_windowed_pool_carries_a_request_longer_than_itself():
    """Only windowed groups: a request grows to many times the pool's positions in portions no larger
    than ``max_portion``, and never holds more pages than its window and its portion touch."""
    m = CacheManager([WIN], page_size=4, pages_per_group=8, n_slots=1)
    assert m.capacity_tokens() >= 1 << 60
    step = m.max_portion()
    assert step == (8 - 4) * 4
    m.admit("a")
    n = 0
    while n < 600:
        k = min(step, 600 - n)
        m.reserve("a", n + k)
        assert m.groups[0].pool.n_out <= 8
        n += k
        m.advance("a", n)
        m.check()
        assert m.groups[0].pool.n_out <= 4
    # one token more than max_portion does not fit at this point
    with pytest.raises(OutOfPages):
        m.reserve("a", n + step + 5)
    m.release("a")
    assert m.all_free()


def test_trim_is_counted():
    """Who keeps a copy of a block table (a recorded step does) sees from ``version`` that pages
    went back from its end, even when its length is later the same again."""
    m = CacheManager([FULL], page_size=4, pages_per_group=8, n_slots=2)
    m.admit("a"); m.admit("b")
    m.reserve("a", 4); m.advance("a", 4)
    m.reserve("b", 4); m.advance("b", 4)
    m.reserve("a", 5); m.reserve("b", 5)
    before = [list(m.get(r).tables[0]) for r in "ab"]
    va = m.get("a").version
    m.trim("a"); m.trim("b")
    assert m.get("a").version > va
    m.reserve("a", 5); m.reserve("b", 5)
    after = [list(m.get(r).tables[0]) for r in "ab"]
    assert [len(t) for t in after] == [len(t) for t in before] and after != before      # same lengths, other pages
    m.check()
