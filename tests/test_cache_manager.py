"""The cache manager on the host: pages, block tables, prefix reuse, windows, state slots.

Reference: test/engine.test.ts:61-123 for prefix reuse and eviction.
"""
import random

import pytest

from sprout_lm_amd.cache import FREED, CacheManager, PagedKVSpec, PageError, PagePool, StateSpec

FULL = PagedKVSpec(2, 16)
WINDOWED = PagedKVSpec(2, 16, window=10)


def invariants(cache: CacheManager):
    """No page lost or held twice: every page is free, or referenced exactly as often as it is held."""
    for gi, g in enumerate(cache.groups):
        held = {}
        for seq in cache.live:
            for page in seq.blocks[gi]:
                if page != FREED:
                    held[page] = held.get(page, 0) + 1
        for entry in cache._prefixes.values():
            held[entry.pages[gi]] = held.get(entry.pages[gi], 0) + 1
        free = list(g.pool._free)
        assert len(free) == len(set(free)), "a page is on the free list twice"
        for page in range(g.pool.num_pages):
            assert g.pool.refs[page] == held.get(page, 0), f"page {page}: refs {g.pool.refs[page]} held {held.get(page, 0)}"
            assert (page in free) == (g.pool.refs[page] == 0)


def test_pool_hands_out_page_zero_first_and_reuses_last_freed():
    pool = PagePool(3)
    assert [pool.allocate(), pool.allocate()] == [0, 1]
    pool.release(0)
    assert pool.allocate() == 0 and pool.allocate() == 2 and pool.allocate() is None
    with pytest.raises(PageError):
        pool.release(1); pool.release(1)
    with pytest.raises(PageError):
        PagePool(2).retain(0)


def test_reserve_is_all_or_nothing_over_groups():
    cache = CacheManager([FULL, WINDOWED, FULL], block_size=4, num_blocks=3, max_sequences=2, prefix_caching=False)
    assert len(cache.groups) == 2 and cache.groups[0].slots == [0, 2] and cache.groups[1].slots == [1]
    a = cache.create()
    assert cache.reserve(a, 9) and [len(b) for b in a.blocks] == [3, 3]
    b = cache.create()
    assert not cache.reserve(b, 1) and b.blocks == [[], []]
    invariants(cache)
    a.release()
    assert cache.reserve(b, 12)
    invariants(cache)
    b.release(); b.release()          # idempotent
    assert cache.free_pages() == [3, 3]
    with pytest.raises(PageError):
        cache.reserve(b, 1)           # use after release


def test_window_gives_pages_back_as_it_passes_them():
    cache = CacheManager([WINDOWED], block_size=4, num_blocks=5, max_sequences=1, prefix_caching=True)
    assert not cache.prefix_caching      # a window cannot share prefixes
    seq = cache.create()
    for length in range(1, 41):
        assert cache.reserve(seq, length), f"window of 10 must fit 5 pages of 4 at length {length}"
        cache.commit(seq, length)
        first_needed = max(0, length - 10 + 1)
        for i, page in enumerate(seq.blocks[0]):
            assert (page == FREED) == ((i + 1) * 4 <= first_needed)
        invariants(cache)
    assert cache.groups[0].pool.num_free >= 1
    seq.release()
    assert cache.free_pages() == [5]


def test_table_versions_change_exactly_when_a_table_changes():
    """Mirrors of a block table on the device are rewritten when its version moves: it must move with every page
    that is added or given back (also by a window, which leaves the table's length as it was), and only then."""
    cache = CacheManager([FULL, WINDOWED], block_size=4, num_blocks=6, max_sequences=2, prefix_caching=False)
    seq = cache.create()
    seen = [(list(b), v) for b, v in zip(seq.blocks, seq.table_versions)]
    for length in range(1, 25):
        assert cache.reserve(seq, length)
        cache.commit(seq, length)
        for gi, (blocks, version) in enumerate(zip(seq.blocks, seq.table_versions)):
            assert (blocks != seen[gi][0]) == (version != seen[gi][1]), f"group {gi} at length {length}"
            seen[gi] = (list(blocks), version)
    assert FREED in seq.blocks[1] and FREED not in seq.blocks[0]
    other = cache.create()
    assert not cache.reserve(other, 24)                    # group 0 has no page left: nothing is kept
    assert other.blocks == [[], []]


def test_prefix_reuse_leaves_the_last_token_to_compute():
    cache = CacheManager([FULL], block_size=2, num_blocks=8, max_sequences=4)
    tokens = [5, 6, 7, 8]                                   # exactly two pages
    a = cache.create()
    assert cache.reserve(a, 4)
    cache.commit(a, 2); cache.publish(tokens, a)
    cache.commit(a, 4); cache.publish(tokens, a)
    b = cache.reuse_prefix(tokens)
    assert b.length == 2 and b.blocks[0] == a.blocks[0][:1]  # one page reused, the last token recomputed
    c = cache.reuse_prefix(tokens + [9])
    assert c.length == 4 and c.blocks[0] == a.blocks[0]
    d = cache.reuse_prefix([9, 9, 7, 8, 1])                  # same later page under another context
    assert d.length == 0
    assert cache.snapshot()["pages"][a.blocks[0][0]]["active_refs"] == 3
    invariants(cache)
    for s in (a, b, c, d):
        s.release()
    assert cache.snapshot()["cached_pages"] == 2 and cache.free_pages() == [6]
    cache.clear_prefixes()
    assert cache.free_pages() == [8]


def test_lru_eviction_takes_only_pages_no_request_uses():
    cache = CacheManager([FULL], block_size=2, num_blocks=3, max_sequences=4)
    a = cache.create()
    tokens = [1, 2, 3, 4, 5]
    assert cache.reserve(a, 5)
    cache.commit(a, 2); cache.publish(tokens, a)
    cache.commit(a, 4); cache.publish(tokens, a)
    a.release()                                               # both full pages stay cached
    reused = cache.reuse_prefix([1, 2, 9])
    protected = reused.blocks[0][0]
    other = cache.create()
    assert cache.reserve(other, 4)                            # takes the free page and evicts the unused one
    assert cache.evictions == 1 and protected not in other.blocks[0]
    assert not cache.reserve(other, 5)                        # the protected page is not evicted
    invariants(cache)
    other.release(); reused.release(); cache.clear_prefixes()
    assert cache.free_pages() == [3]


def test_state_slots_are_per_request_and_come_back():
    cache = CacheManager([FULL, StateSpec((4, 3))], block_size=4, num_blocks=4, max_sequences=2)
    assert not cache.prefix_caching and cache.slot_location[1] == ("state", 0, 0)
    a, b = cache.create(), cache.create()
    assert {a.state_slot, b.state_slot} == {0, 1}
    with pytest.raises(PageError):
        cache.create()
    a.release()
    assert cache.create().state_slot == a.state_slot


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_never_lose_or_double_a_page(seed):
    rng = random.Random(seed)
    specs = [FULL, WINDOWED] if seed % 2 else [FULL]
    cache = CacheManager(specs, block_size=4, num_blocks=12, max_sequences=5, prefix_caching=True)
    live = []
    prompts = [[rng.randrange(3) for _ in range(rng.randrange(1, 30))] for _ in range(8)]
    for _ in range(400):
        action = rng.random()
        if action < 0.25 and len(live) < 5:
            tokens = rng.choice(prompts)
            live.append((cache.reuse_prefix(tokens), tokens))
        elif action < 0.8 and live:
            seq, tokens = rng.choice(live)
            if seq.length < len(tokens):
                new = min(len(tokens), seq.length + rng.randrange(1, 7))
                if cache.reserve(seq, new):
                    old = seq.length
                    cache.commit(seq, new)
                    for boundary in range((old // 4 + 1) * 4, new + 1, 4):
                        cache.publish(tokens, seq, boundary)
        elif live:
            seq, _ = live.pop(rng.randrange(len(live)))
            seq.release()
        invariants(cache)
    for seq, _ in live:
        seq.release()
    cache.clear_prefixes()
    invariants(cache)
    assert cache.free_pages() == [12] * len(cache.groups)
