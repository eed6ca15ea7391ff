"""The scheduler's decisions, without a model: budget, order, admission, preemption, finishing."""
import random

import pytest

from xyntetik_runner_amd.cache import CacheManager
from xyntetik_runner_amd.engine.request import Request
from xyntetik_runner_amd.engine.scheduler import Scheduler
from xyntetik_runner_amd.parts.base import KVSpec
from xyntetik_runner_amd.sampling import SamplingParams

SPEC = KVSpec(2, 16, None)


def make(pages=16, page_size=4, budget=8, max_running=4, max_len=64, slots=8, stop=()):
    m = CacheManager([SPEC], page_size=page_size, pages_per_group=pages, n_slots=slots)
    return m, Scheduler(m, max_batched_tokens=budget, max_running=max_running, max_model_len=max_len, stop_ids=stop)


def req(i, n, new=8, **kw):
    return Request(i, list(range(1, n + 1)), SamplingParams(max_new_tokens=new, **kw))


def run_step(s, token=7):
    """Plan, pretend the step ran, and give every ready request ``token``."""
    plan = s.schedule()
    for r in s.ran(plan):
        s.accept(r, token)
    s.manager.check()
    return plan


def test_budget_is_never_exceeded_and_prompts_are_cut():
    m, s = make(budget=8)
    s.add(req("a", 20))
    sizes = []
    while s.running or s.waiting:
        plan = run_step(s)
        assert plan.n_tokens <= 8
        sizes.append([n for _, n in plan.entries])
        if len(sizes) > 40:
            break
    assert sizes[:3] == [[8], [8], [4]]            # 20 prompt tokens in portions of 8, 8, 4
    assert all(x == [1] for x in sizes[3:]) and len(sizes) == 3 + 7   # then 7 more decode steps (8 new tokens)


def test_decode_comes_before_prompt_portions_and_admission_is_fifo():
    m, s = make(budget=6, pages=32)
    s.add(req("a", 3)); s.add(req("b", 9)); s.add(req("c", 2))
    p1 = s.schedule()
    assert [(r.id, n) for r, n in p1.entries] == [("a", 3), ("b", 3)]         # c waits: no budget left
    for r in s.ran(p1):
        s.accept(r, 5)
    p2 = s.schedule()
    # a decodes (1), b's prompt goes on (5 of its 6 left); c still waits behind b
    assert [(r.id, n) for r, n in p2.entries] == [("a", 1), ("b", 5)]
    for r in s.ran(p2):
        s.accept(r, 5)
    p3 = s.schedule()
    assert [(r.id, n) for r, n in p3.entries] == [("a", 1), ("b", 1), ("c", 2)]
    assert p3.n_tokens <= 6


def test_max_running_and_slots_limit_admission():
    m, s = make(budget=64, max_running=2, pages=64)
    for i in range(4):
        s.add(req(i, 2, new=2))
    p = s.schedule()
    assert [r.id for r, _ in p.entries] == [0, 1] and len(s.waiting) == 2
    for r in s.ran(p):
        s.accept(r, 3)
    p = run_step(s)                      # both finish here (2 new tokens each)
    assert not s.running
    p = s.schedule()
    assert [r.id for r, _ in p.entries] == [2, 3]


def test_finishing_rules():
    m, s = make(stop=(99,), max_len=12)
    a = req("a", 4, new=3)
    s.add(a)
    run_step(s, token=5)
    assert a.output == [5] and not a.finished
    s.ran(s.schedule()); assert s.accept(a, 99)                    # stop token: not kept
    assert a.finish_reason == "stop" and a.output == [5] and m.free_pages() == 16 and not s.running
    b = req("b", 4, new=2)
    s.add(b)
    run_step(s, 1); run_step(s, 1)
    assert b.finish_reason == "length" and b.output == [1, 1]
    c = req("c", 4, new=-1, ignore_eos=True)
    s.add(c)
    for _ in range(20):
        if c.finished:
            break
        run_step(s, 99)
    assert c.finish_reason == "context" and c.n_tokens == 12 and c.output == [99] * 8
    with pytest.raises(ValueError) as e:
        s.add(req("d", 12))
    assert "13" in str(e.value)                                    # names a context that fits


def test_running_out_of_pages_preempts_the_last_admitted_and_recomputes():
    m, s = make(pages=6, page_size=4, budget=16, max_len=64)       # 24 positions
    a, b = req("a", 8, new=12), req("b", 8, new=12)
    s.add(a); s.add(b)
    preempted_at = None
    for step in range(60):
        plan = run_step(s, token=3)
        if plan.preempted:
            assert [r.id for r in plan.preempted] == ["b"]          # the request admitted last
            assert s.waiting[0] is b and b.n_computed == 0 and b.n_preempted == 1
            assert all(r is not b for r, _ in plan.entries)
            preempted_at = step
            kept = list(b.output)
        if a.finished and b.finished:
            break
    assert preempted_at is not None
    assert a.finish_reason == b.finish_reason == "length"
    assert len(a.output) == 12 and len(b.output) == 12 and b.output[:len(kept)] == kept
    assert a.n_preempted == 0
    assert m.free_pages() == 6 and m.slots.n_free == 8


def test_a_request_that_cannot_fit_alone_fails_and_frees():
    m, s = make(pages=2, page_size=4, budget=16, max_len=64)       # 8 positions
    with pytest.raises(ValueError):
        s.add(req("x", 8))                                          # prompt + 1 > capacity: refused at the door
    a = req("a", 6, new=10)
    s.add(a)
    reasons = []
    for _ in range(10):
        plan = run_step(s, 1)
        reasons += [r.finish_reason for r in plan.failed]
        if a.finished:
            break
    assert reasons == ["cache_full"] and a.n_computed == 8 and a.n_tokens == 9 and m.free_pages() == 2 and not s.running


def test_no_starvation_under_random_load():
    rng = random.Random(3)
    m, s = make(pages=12, page_size=4, budget=10, max_running=3, max_len=48)
    reqs = [req(i, rng.randint(1, 14), new=rng.randint(1, 10)) for i in range(12)]
    for r in reqs:
        s.add(r)
    for step in range(2000):
        if not s.has_work():
            break
        plan = run_step(s, token=rng.randint(0, 50))
        assert plan.n_tokens <= 10 and (plan.entries or plan.failed)
        ids = [r.id for r, _ in plan.entries]
        assert len(ids) == len(set(ids))
    assert all(r.finished and r.finish_reason == "length" for r in reqs), [(r.id, r.finish_reason) for r in reqs]
    assert m.free_pages() == 12


def test_a_slice_of_a_requests_tokens():
    """Prompt and output are two lists; a slice across them equals the slice of both together."""
    req = Request("r", [5, 6, 7, 8], SamplingParams())
    req.output.extend([20, 21, 22])
    whole = req.tokens
    assert whole == [5, 6, 7, 8, 20, 21, 22] and req.n_tokens == 7
    for a in range(9):
        for b in range(a, 10):
            assert req.token_slice(a, b) == whole[a:b], (a, b)
    req.n_computed = 5
    assert req.remaining == 2


def run_step_as_the_runner_does(s, token=7):
    """``run_step``, and the cache manager is told what is cached now, as the step function tells
    it (pages that a window has passed go back then)."""
    plan = s.schedule()
    for r, n in plan.entries:
        s.manager.advance(r.id, r.n_computed + n)
    for r in s.ran(plan):
        s.accept(r, token)
    s.manager.check()
    return plan


def test_portions_are_cut_to_what_the_windowed_pools_can_hold():
    """Every layer keeps a window of 10 keys, the pool has 8 pages of 4: a prompt of 200 tokens is no
    longer than the cache holds (windowed layers set no limit), runs in portions of at most
    (8 - 4) x 4 = 16 tokens although the budget is 64, nobody is preempted and nothing fails."""
    m = CacheManager([KVSpec(1, 32, 10)], page_size=4, pages_per_group=8, n_slots=2)
    s = Scheduler(m, max_batched_tokens=64, max_running=2, max_model_len=1024)
    assert s.capacity_tokens() > 1 << 60
    s.add(req("a", 200, new=4))
    sizes = []
    while s.running or s.waiting:
        plan = run_step_as_the_runner_does(s)
        assert not plan.preempted and not plan.failed
        sizes.append(plan.n_tokens)
        assert len(sizes) < 60
    assert sizes[:13] == [16] * 12 + [8] and sizes[13:] == [1] * 3
    assert m.all_free()


def test_a_full_attention_group_still_limits_the_length():
    m = CacheManager([SPEC, KVSpec(1, 32, 10)], page_size=4, pages_per_group=[10, 8], n_slots=2)
    s = Scheduler(m, max_batched_tokens=64, max_running=2, max_model_len=1024)
    assert s.capacity_tokens() == 40
    with pytest.raises(ValueError, match="does not fit the cache"):
        s.add(req("a", 40))
    s.add(req("b", 39, new=1))
    while s.running or s.waiting:
        plan = run_step_as_the_runner_does(s)
        assert not plan.failed
    assert m.all_free()
