"""The cache manager without a GPU: the reference's vectors, window release,
state slots, and that under random orders of requests no page is lost, held
twice or freed twice."""

from __future__ import annotations

import random

import pytest

from llmserve_amd import CacheConfig, CacheFullError, Qwen2Config
from llmserve_amd.cache import CacheManager, PagePool
from llmserve_amd.registry import ARCHITECTURES
from tests.tiny import TINY_A, TINY_B


def manager(config: Qwen2Config, block_size: int, num_blocks: int, max_sequences: int = 8, length: int = 64):
    spec = ARCHITECTURES["Qwen2ForCausalLM"].build_spec(config)
    cache_config = CacheConfig(block_size=block_size, num_blocks=num_blocks, max_sequences=max_sequences)
    return CacheManager(spec, cache_config, max_sequence_length=length)


def test_pool_reuses_freed_pages_and_checks_the_owner():
    """reference tests/test_kv_cache.py:22-31"""
    pool = PagePool(2)
    first = pool.allocate("a")
    pool.allocate("b")
    with pytest.raises(CacheFullError):
        pool.allocate("c")
    with pytest.raises(ValueError):
        pool.free(first, "b")
    pool.free(first, "a")
    with pytest.raises(ValueError):
        pool.free(first, "a")  # twice
    assert pool.allocate("c") == first
    assert (pool.used_pages, pool.free_pages) == (2, 0)


def test_block_table_fragmentation_and_eviction():
    """reference tests/test_kv_cache.py:34-46"""
    cache = manager(TINY_A, 4, 4, length=32)
    cache.create("short")
    for _ in range(5):
        cache.reserve("short", 1)
    assert cache.block_table("short") == [0, 1]
    assert cache.stats(32)["paged_fragmentation_pct"] == 37.5
    cache.create("long")
    cache.reserve("long", 8)
    assert cache.evict("largest") == ("long", 8)
    assert cache.groups[0].pool.free_pages == 2
    cache.check_invariants()


def test_slots_cross_page_boundaries():
    """reference tests/test_kv_cache.py:114-134: pages [0,0,1 | 2,2], offsets [0,1,0 | 0,1]"""
    cache = manager(TINY_A, 2, 8)
    cache.create("a")
    cache.create("b")
    a = cache.reserve("a", 3)
    b = cache.reserve("b", 2)
    assert (a.slot, b.slot) == (0, 1)
    assert (a.slots[0] // 2).tolist() == [0, 0, 1] and (a.slots[0] % 2).tolist() == [0, 1, 0]
    assert (b.slots[0] // 2).tolist() == [2, 2] and (b.slots[0] % 2).tolist() == [0, 1]
    assert (a.start, b.start) == (0, 0)
    more = cache.reserve("a", 2)
    assert more.start == 3 and (more.slots[0] // 2).tolist() == [1, 3]
    assert cache.block_table("a") == [0, 1, 3]


def test_freed_rows_are_cleared_and_the_next_request_gets_another_row():
    """reference tests/test_kv_cache.py:77-111"""
    cache = manager(TINY_A, 2, 4)
    row = cache.create("first")
    cache.reserve("first", 3)
    assert cache.groups[0].tables[row, :4].tolist() == [0, 1, -1, -1]
    cache.free("first")
    assert (cache.groups[0].tables[row] == -1).all()
    assert cache.create("replacement") != row
    with pytest.raises(ValueError):
        cache.create("replacement")
    with pytest.raises(KeyError):
        cache.free("first")
    cache.check_invariants()


def test_full_cache_raises_and_holds_nothing_new():
    cache = manager(TINY_A, 4, 3, length=64)
    cache.create("a")
    cache.reserve("a", 9)
    cache.create("b")
    assert not cache.fits([("b", 1)])
    assert cache.pages_short([("b", 5)]) == 2
    with pytest.raises(CacheFullError):
        cache.reserve("b", 1)
    assert cache.sequences["b"].length == 0
    cache.check_invariants()
    cache.reserve("a", 3)  # room left inside a's last page
    with pytest.raises(CacheFullError):
        cache.reserve("a", 1)
    cache.free("a")
    cache.reserve("b", 12)
    bounded = manager(TINY_A, 4, 64, length=8)
    bounded.create("x")
    with pytest.raises(CacheFullError, match="longest sequence"):
        bounded.reserve("x", 9)


def test_groups_have_pages_of_their_own_and_a_window_gives_them_back():
    cache = manager(TINY_B, 8, 16, length=512)  # layer 0 sees all keys, layers 1 and 2 the last 24
    assert [(g.need.window, g.cells) for g in cache.groups] == [(None, [(0, None)]), (24, [(1, None), (2, None)])]
    assert cache.groups[1].storage["keys"].shape == (2, 16, 1, 4, 8, 8) and cache.groups[1].storage["values"].shape == (2, 16, 1, 1, 32, 8)
    cache.create("r")
    cache.reserve("r", 40)  # nothing to give back yet: the step starts at position 0
    assert [g.pool.used_pages for g in cache.groups] == [5, 5]
    # the next token sits at position 40 and reads keys 17..40: blocks 0 and 1 (keys 0..15) have passed
    assert cache.pages_needed("r", 1) == [(1, 0), (1, 2)]
    cache.reserve("r", 1)
    assert [g.pool.used_pages for g in cache.groups] == [6, 4]
    assert cache.groups[1].tables[0, :6].tolist() == [-1, -1, 2, 3, 4, 5]
    cache.check_invariants()
    for _ in range(60):
        cache.reserve("r", 1)
    assert cache.groups[1].pool.used_pages <= 5  # never more than a window's worth (+ the page being filled)
    assert cache.groups[0].pool.used_pages == 13
    cache.check_invariants()
    cache.free("r")
    assert [g.pool.free_pages for g in cache.groups] == [16, 16]


def test_a_window_lets_a_long_request_live_in_few_pages():
    cache = manager(TINY_B, 8, 6, length=512)
    cache.create("r")
    with pytest.raises(CacheFullError):
        cache.reserve("r", 56)  # the full-attention group needs 7 pages
    cache.reserve("r", 40)
    assert cache.fits([("r", 8)]) and not cache.fits([("r", 9)])


@pytest.mark.parametrize("config,block", [(TINY_A, 4), (TINY_B, 8)])
def test_random_orders_lose_nothing(config, block):
    rng = random.Random(17)
    cache = manager(config, block, 24, max_sequences=5, length=200)
    live: dict[str, int] = {}
    counter = 0
    for _ in range(3000):
        action = rng.random()
        if action < 0.15 and len(live) < 5:
            name = f"r{counter}"
            counter += 1
            cache.create(name)
            live[name] = 0
        elif action < 0.85 and live:
            name = rng.choice(sorted(live))
            count = rng.choice([1, 1, 1, 2, 3, 7, 16, 33])
            fits = cache.fits([(name, count)])
            if fits:
                before = (cache.used_pages, cache.stats(200)["used_tokens"])
                reservation = cache.reserve(name, count)
                assert reservation.start == live[name]
                if rng.random() < 0.25:  # taken back unused: as if it had never been made
                    cache.cancel(reservation)
                    # (a page that the window has passed at this position stays given back)
                    assert cache.used_pages <= before[0] and cache.stats(200)["used_tokens"] == before[1]
                    assert cache.sequences[name].length == live[name]
                    with pytest.raises(ValueError):
                        cache.cancel(reservation)
                else:
                    live[name] += count
            else:
                before = cache.used_pages
                with pytest.raises(CacheFullError):
                    cache.reserve(name, count)
                assert cache.used_pages == before
        elif live:
            name = rng.choice(sorted(live))
            if rng.random() < 0.5:
                cache.free(name)
            else:
                name, recompute = cache.evict("largest")
                assert recompute == live[name]
            del live[name]
        cache.check_invariants()
        assert {n: cache.sequences[n].length for n in live} == live
    for name in list(live):
        cache.free(name)
    cache.check_invariants()
    assert cache.used_pages == 0 and all((g.tables == -1).all() for g in cache.groups)
    with pytest.raises(CacheFullError):
        for index in range(6):
            cache.create(f"slot{index}")
