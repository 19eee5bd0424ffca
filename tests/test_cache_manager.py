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
            for page in entry.pages[gi] or ():
                held[page] = held.get(page, 0) + 1
        free = g.pool.free_list()
        assert len(free) == len(set(free)) == g.pool.num_free, "a page is on the free list twice"
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


def test_a_pool_costs_what_it_has_handed_out_not_what_it_could():
    """A pool of two billion pages (a mistyped option) is built at once and without memory for its pages: the
    memory budget is what refuses it, and it has to get that far."""
    import time
    start = time.time()
    pool = PagePool(2_000_000_000)
    assert pool.num_free == 2_000_000_000 and pool.refs[1_999_999_999] == 0 and len(pool.refs) == 2_000_000_000
    assert [pool.allocate() for _ in range(3)] == [0, 1, 2]
    pool.release(1)
    assert pool.num_free == 1_999_999_998 and pool.allocate() == 1 and pool.allocate() == 3
    cache = CacheManager([FULL, WINDOWED], block_size=16, num_blocks=2_000_000_000, max_sequences=4)
    assert cache.storage_bytes(2) == CacheManager.pool_bytes([FULL, WINDOWED], 16, 2_000_000_000, 4, 2)
    assert time.time() - start < 1.0


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
    cache = CacheManager([WINDOWED], block_size=4, num_blocks=5, max_sequences=1, prefix_caching=False)
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


def feed(cache, seq, tokens, portion):
    """Compute `tokens` in portions, publishing every full page as the scheduler does after a step."""
    bs = cache.block_size
    while seq.length < len(tokens):
        old, new = seq.length, min(len(tokens), seq.length + portion)
        assert cache.reserve(seq, new)
        cache.commit(seq, new)
        for boundary in range((old // bs + 1) * bs, new + 1, bs):
            cache.publish(tokens, seq, boundary)


def test_a_windowed_group_shares_the_pages_its_window_still_covers():
    """A group with a window of 10 beside one that keeps every key, pages of 4.  A second request with the same
    first 21 tokens takes over five pages: all five in the full group; in the windowed group those from key
    20 - 10 + 1 = 11 on (pages 2..4), the earlier places of its table marked as given back."""
    cache = CacheManager([FULL, WINDOWED], block_size=4, num_blocks=12, max_sequences=3)
    assert cache.prefix_caching
    tokens = list(range(100, 123))                            # 23 tokens: five full pages and three more
    a = cache.create()
    feed(cache, a, tokens, portion=3)                         # portions shorter than the window: every page is live when offered
    assert a.blocks[1][:3] == [FREED] * 3                     # a's own window (from key 14) has passed pages 0..2
    b = cache.reuse_prefix(tokens[:21] + [7, 7])
    assert b.length == 20 and b.blocks[0] == a.blocks[0][:5]
    assert b.blocks[1][:2] == [FREED, FREED] and all(p != FREED for p in b.blocks[1][2:5])
    assert b.blocks[1][3:5] == a.blocks[1][3:5]               # the very pages a wrote
    invariants(cache)
    # b goes on: its window passes pages like anyone's, the cache keeps its own reference
    feed(cache, b, tokens[:21] + [7, 7], portion=2)
    assert b.length == 23 and b.blocks[1][2] == FREED
    invariants(cache)
    a.release(); b.release()
    assert cache.free_pages()[0] == 12 - 5                    # the five shared pages stay cached
    cache.clear_prefixes()
    assert cache.free_pages() == [12, 12]


def test_a_long_portion_offers_what_its_window_has_left_and_reuse_stops_where_keys_are_missing():
    """Computed in one step, a prompt of 24 tokens has given back the windowed pages before key 15 when its pages
    are offered: the entries of pages 0..2 hold no page of that group.  A request that shares 8 tokens would
    read keys from 8 - 10 + 1 < 0 on, which nobody holds: it shares nothing.  One that shares all 24 shares
    five pages (one token is left to compute) and reads keys from 11 on: page 2 is missing, so it steps back
    until its window is whole, which it never is here: nothing either.  After the same prompt came in short
    portions, both share."""
    cache = CacheManager([FULL, WINDOWED], block_size=4, num_blocks=16, max_sequences=4)
    tokens = list(range(24))
    a = cache.create()
    feed(cache, a, tokens, portion=24)
    assert [e.pages[1] is None for e in sorted(cache._prefixes.values(), key=lambda e: e.last_used)] == [True] * 3 + [False] * 3
    assert cache.reuse_prefix(tokens[:8] + [99]).length == 0
    assert cache.reuse_prefix(tokens).length == 0
    invariants(cache)
    for seq in list(cache.live):
        seq.release()
    cache.clear_prefixes()
    a = cache.create()
    feed(cache, a, tokens, portion=4)
    assert cache.reuse_prefix(tokens[:8] + [99]).length == 8 and cache.reuse_prefix(tokens).length == 20
    invariants(cache)


def test_a_short_windowed_pool_takes_cached_pages_back_one_at_a_time():
    """When a windowed group's pool is empty, the least recently used entry gives back that group's page alone
    and stays a link of its chain; a request whose window would need the missing page shares less."""
    cache = CacheManager([WINDOWED], block_size=4, num_blocks=6, max_sequences=3)
    tokens = list(range(16))
    a = cache.create()
    feed(cache, a, tokens, portion=4)
    a.release()                                               # four pages cached
    assert cache.free_pages() == [2]
    b = cache.create()
    assert cache.reserve(b, 12)                               # three pages: one more than are free
    assert cache.evictions == 1 and len(cache._prefixes) == 4
    first = min(cache._prefixes.values(), key=lambda e: e.last_used)
    assert first.pages == [None]                              # the oldest entry gave its page back and stays
    invariants(cache)
    c = cache.reuse_prefix(tokens)     # three pages offered; a window of 10 at key 12 begins at key 3, in page 0
    assert c.length == 0
    d = cache.reuse_prefix(tokens + [1] * 8)   # four pages: at key 16 the window begins at key 7, in page 1
    assert d.length == 16 and d.blocks[0][0] == FREED and FREED not in d.blocks[0][1:]
    invariants(cache)
    for seq in (b, c, d):
        seq.release()
    cache.clear_prefixes()
    assert cache.free_pages() == [6]


def test_a_prefix_published_again_restores_the_pages_an_entry_gave_back():
    """An entry that gave a windowed group's page back under pressure stays in its chain.  When a later request
    computes the same tokens and offers the page again, the entry takes the new page, and the prefix is shared
    whole again."""
    cache = CacheManager([WINDOWED], block_size=4, num_blocks=8, max_sequences=3)
    tokens = list(range(16))
    a = cache.create()
    feed(cache, a, tokens, portion=4)
    a.release()
    b = cache.create()
    assert cache.reserve(b, 20)                               # one page more than are free: the oldest entry gives its own
    b.release()
    assert sum(e.pages == [None] for e in cache._prefixes.values()) == 1
    assert cache.reuse_prefix(tokens).length == 0             # a window at key 12 needs page 0, which is gone
    for seq in list(cache.live):
        seq.release()
    again = cache.create()
    feed(cache, again, tokens, portion=4)                     # computes and offers the same four pages
    assert all(e.pages != [None] for e in cache._prefixes.values())
    invariants(cache)
    again.release()
    assert cache.reuse_prefix(tokens).length == 12
    invariants(cache)
    for seq in list(cache.live):
        seq.release()
    cache.clear_prefixes()
    assert cache.free_pages() == [8]


def test_a_prefix_hit_is_believed_only_with_the_same_tokens(monkeypatch):
    """The index is keyed by a hash; a hit is taken only if the entry holds the very tokens behind the very
    parent (the reference keys by the tokens themselves, src/kv-cache.ts:103,118).  With a hash that maps
    everything to one value, other prompts share nothing, and the same prompt still shares."""
    monkeypatch.setattr(CacheManager, "_chain", staticmethod(lambda parent, tokens: b"same"))
    cache = CacheManager([FULL], block_size=4, num_blocks=8, max_sequences=4)
    tokens = [1, 2, 3, 4, 5]
    a = cache.create()
    feed(cache, a, tokens, portion=5)
    assert len(cache._prefixes) == 1
    assert cache.reuse_prefix([9, 9, 9, 9, 5]).length == 0
    assert cache.reuse_prefix([1, 2, 3, 4, 9]).length == 4
    # a second page hashes to the same key: it is not the first page's entry, and is not taken for it
    assert cache.reuse_prefix([1, 2, 3, 4, 1, 2, 3, 4, 0]).length == 4
    invariants(cache)


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
    # whether a model with state shares prefixes is its plan's word; the manager does what it is told
    assert cache.prefix_caching and cache.slot_location[1] == ("state", 0, 0)
    a, b = cache.create(), cache.create()
    assert {a.state_slot, b.state_slot} == {0, 1}
    with pytest.raises(PageError):
        cache.create()
    a.release()
    assert cache.create().state_slot == a.state_slot


@pytest.mark.parametrize("seed", range(12))
def test_random_orders_never_lose_or_double_a_page(seed):
    rng = random.Random(seed)
    specs = [[FULL], [FULL, WINDOWED], [WINDOWED], [PagedKVSpec(1, 8, window=5), FULL, WINDOWED],
             [FULL, PagedKVSpec(2, 16, window=10, page_tokens=2)], [PagedKVSpec(2, 16, page_tokens=1), WINDOWED]][seed % 6]
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
    assert cache.free_pages() == [g.pool.num_pages for g in cache.groups]


def test_groups_with_pages_of_their_own_size():
    """A windowed group asks for pages of 2 tokens in a cache whose pages (and prefix unit) are 8: it holds the same
    number of tokens in four times the pages, gives back what its window of 10 has passed two tokens at a time,
    and shares a prefix as four of its pages beside one of the other group's."""
    small = PagedKVSpec(2, 16, window=10, page_tokens=2)
    cache = CacheManager([FULL, small], block_size=8, num_blocks=6, max_sequences=3)
    assert [g.page_tokens for g in cache.groups] == [8, 2] and [g.pool.num_pages for g in cache.groups] == [6, 24]
    with pytest.raises(ValueError, match="do not divide"):
        CacheManager([PagedKVSpec(2, 16, page_tokens=3)], block_size=8, num_blocks=4, max_sequences=1)
    tokens = list(range(30))
    a = cache.create()
    assert cache.pages_needed(a, 17) == [3, 9]
    feed(cache, a, tokens, portion=3)
    assert [len(b) for b in a.blocks] == [4, 15]
    # length 30: the next token reads keys from 21 on; pages of 2 before key 20 are back
    assert a.blocks[1][:10] == [FREED] * 10 and FREED not in a.blocks[1][10:]
    invariants(cache)
    b = cache.reuse_prefix(tokens[:26])
    # three units of 8 are offered (one token must stay); b computes position 24 next and reads keys from 15 on,
    # which lie in the second unit: all of its four small pages come along, the first unit's do not
    assert b.length == 24 and b.blocks[0] == a.blocks[0][:3]
    assert b.blocks[1][:4] == [FREED] * 4 and FREED not in b.blocks[1][4:12] and len(b.blocks[1]) == 12
    invariants(cache)
    feed(cache, b, tokens[:26], portion=1)
    assert b.blocks[1][:8] == [FREED] * 8                 # at length 26 keys before 17 are passed: pages up to key 15
    a.release(); b.release(); cache.clear_prefixes()
    assert cache.free_pages() == [6, 24]


def test_keys_and_values_of_different_widths_and_a_dtype_of_their_own():
    """A slot whose values are narrower than its keys, kept in float32 whatever the model computes in: a group
    of its own, pools of the asked shapes, and the bytes that the memory budget counts."""
    import torch
    odd = PagedKVSpec(1, 24, value_dim=8, dtype="float32")
    cache = CacheManager([FULL, odd, FULL], block_size=4, num_blocks=5, max_sequences=2)
    assert [g.slots for g in cache.groups] == [[0, 2], [1]]
    cache.attach_storage(torch.bfloat16, "cpu")
    full, other = cache.groups
    assert full.k.shape == (2, 5, 2, 4, 16) and full.v.shape == (2, 5, 2, 16, 4) and full.k.dtype == torch.bfloat16
    assert other.k.shape == (1, 5, 1, 4, 24) and other.v.shape == (1, 5, 1, 8, 4) and other.v.dtype == torch.float32
    want = sum(t.numel() * t.element_size() for g in cache.groups for t in (g.k, g.v))
    assert cache.storage_bytes(2) == want == CacheManager.pool_bytes([FULL, odd, FULL], 4, 5, 2, 2)
