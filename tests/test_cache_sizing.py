"""How the cache is sized from the memory that is left (host arithmetic only)."""
import pytest

from xyntetik_runner_amd.cache import CacheTooSmall, cache_groups, memory_budget, page_bytes, size_pools
from xyntetik_runner_amd.parts import KVSpec

GIB = 1 << 30
FULL = KVSpec(8, 128, None)
WIN = KVSpec(8, 128, 1024)


def test_groups_of_a_run_order():
    # four entries: two own a cache of every key, one a windowed one, one reads the first entry's
    specs, owners = cache_groups([FULL, WIN, FULL, FULL, None], [None, None, None, 0, None])
    assert specs == [FULL, WIN] and owners == [2, 1]


def test_page_bytes():
    # keys and values of 32 layers, 8 heads of 128, 64 positions, 2 bytes: 128 KiB a token
    assert page_bytes(FULL, 32, 64, 2) == 64 * 128 * 1024


def test_budget():
    total = 288 * GIB
    assert memory_budget(total, total - 16 * GIB, 0.9, 2 * GIB) == int(0.9 * total) - 16 * GIB - 2 * GIB
    with pytest.raises(ValueError):
        memory_budget(total, total, 1.5, 0)


def test_the_8b_shape_with_its_real_context_takes_what_is_left():
    """Llama-3.1-8B names a context of 131,072: 64 requests of that length would be 1 TiB, so the
    pool is what the card has left (src/model.h:516-592 caps the context instead; here the pool is shared)."""
    budget = memory_budget(288 * GIB, (288 - 16) * GIB, 0.9, 2 * GIB)
    (pages,) = size_pools([FULL], [32], 64, 2, max_requests=64, max_step_tokens=2048, budget_bytes=budget,
                          max_model_len=131072)
    per_page = page_bytes(FULL, 32, 64, 2)
    assert pages == budget // per_page - 1                          # all of it but the null page
    assert pages * 64 >= 131072                                     # one request of the full context fits
    assert (pages + 1) * per_page <= budget


def test_no_more_than_the_requests_can_fill():
    (pages,) = size_pools([FULL], [2], 64, 2, max_requests=4, budget_bytes=100 * GIB, max_model_len=1000)
    assert pages == 4 * 16


def test_too_small_is_a_named_error():
    """The 70B shape with a context of 131,072 beside 141 GB of weights, at a fraction that leaves 30 GiB."""
    spec = KVSpec(8, 128, None)
    with pytest.raises(CacheTooSmall, match="131072 tokens"):
        size_pools([spec], [80], 64, 2, max_requests=64, budget_bytes=30 * GIB, max_model_len=131072)
    with pytest.raises(CacheTooSmall):
        size_pools([spec], [80], 64, 2, max_requests=64, budget_bytes=-5, max_model_len=128)
    # and with room for exactly one request it is sized for one
    need = (2048 + 1) * page_bytes(spec, 80, 64, 2)
    assert size_pools([spec], [80], 64, 2, max_requests=64, budget_bytes=need, max_model_len=131072) == [2048]


def test_windowed_groups_take_a_fixed_share_first():
    per_full, per_win = page_bytes(FULL, 24, 64, 2), page_bytes(WIN, 8, 64, 2)
    sizes = size_pools([FULL, WIN], [24, 8], 64, 2, max_requests=16, max_step_tokens=2048, budget_bytes=40 * GIB,
                       max_model_len=32768)
    win_pages = 16 * (1024 // 64 + 2) + 2048 // 64
    assert sizes[1] == win_pages
    assert sizes[0] == (40 * GIB - (win_pages + 1) * per_win - per_full) // per_full
    # given tokens instead of memory, both follow from the tokens
    assert size_pools([FULL, WIN], [24, 8], 64, 2, max_requests=16, max_step_tokens=2048, max_tokens=100_000) == \
        [-(-100_000 // 64), win_pages]
    with pytest.raises(ValueError):
        size_pools([FULL], [1], 64, 2, max_requests=1)
