"""The cache manager: paged keys and values in groups, block tables, prefix reuse, state slots.

Reference: KVCache and PagedSequence (src/kv-cache.ts:5-172).  Beyond the reference: cache slots
are sorted into groups by what they need (all keys, or a window of them); every group has a pool
and block tables of its own, and a windowed group gives pages back once the window has passed them.
Requests also hold a slot for per-request state of fixed size.
"""
from __future__ import annotations

import hashlib
import struct
from dataclasses import dataclass, field

from .pages import PageError, PagePool
from .spec import PagedKVSpec, StateSpec

FREED = -1  # block-table entry of a page that a window has passed
_DTYPE_BYTES = {"float32": 4, "bfloat16": 2, "float16": 2, "int32": 4, "float64": 8, "int64": 8}


@dataclass
class PagedGroup:
    spec: PagedKVSpec
    slots: list[int]              # cache slot ids that live in this group, in pool order
    pool: PagePool
    page_tokens: int = 0          # tokens in one page of this group
    k: object = None              # device tensor [len(slots), pages, kv_heads, page_size, head_dim]
    v: object = None              # device tensor [len(slots), pages, kv_heads, value_dim or head_dim, page_size]


@dataclass
class StateGroup:
    spec: StateSpec
    slots: list[int]
    data: object = None           # device tensor [len(slots), max_sequences, *shape]


class SequenceCache:
    """What one request holds: a block table per group, its computed length, a state slot."""

    _next_uid = 0

    def __init__(self, manager: "CacheManager", state_slot: int):
        self._manager = manager
        SequenceCache._next_uid += 1
        self.uid = SequenceCache._next_uid      # never reused, unlike id(): caches keyed by it stay valid
        self.blocks: list[list[int]] = [[] for _ in manager.groups]
        # bumped whenever a group's table changes (a page more, a page given back): mirrors of the table on
        # the device are rewritten only then
        self.table_versions: list[int] = [0 for _ in manager.groups]
        self.length = 0
        self.state_slot = state_slot
        self.released = False
        self.prefix_keys: list[bytes] = []   # chained keys of the full pages computed so far

    def _live(self):
        if self.released:
            raise PageError("Sequence cache was released.")

    def release(self) -> None:
        self._manager.release(self)


@dataclass
class _PrefixEntry:
    """`block_size` tokens of a prefix in every group: that group's pages of them, or None where a windowed
    group has given them back (the entry then still links the chain, and serves requests whose window lies
    behind it)."""
    pages: list
    last_used: int
    parent: bytes = b""        # key of the entry one page earlier in the chain
    tokens: tuple = ()         # the page's own tokens: a hit is believed only if they, and the parent, are the same


class CacheManager:
    def __init__(self, slot_specs: list[PagedKVSpec | StateSpec], block_size: int, num_blocks: int,
                 max_sequences: int, prefix_caching: bool = True):
        """`slot_specs[i]` is what cache slot i needs.  Storage is attached with `attach_storage`."""
        for name, value in (("block_size", block_size), ("num_blocks", num_blocks), ("max_sequences", max_sequences)):
            if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
                raise ValueError(f"{name} must be a positive integer.")
        self.block_size, self.num_blocks, self.max_sequences = block_size, num_blocks, max_sequences
        self.groups: list[PagedGroup] = []
        self.state_groups: list[StateGroup] = []
        self.slot_location: list[tuple[str, int, int]] = []   # slot -> ("paged" | "state", group, index in group)
        for slot, spec in enumerate(slot_specs):
            if isinstance(spec, PagedKVSpec):
                groups, kind = self.groups, "paged"
                tokens = spec.page_tokens or block_size
                if isinstance(tokens, bool) or not isinstance(tokens, int) or tokens <= 0 or block_size % tokens:
                    raise ValueError(f"Cache slot {slot}: pages of {tokens!r} tokens do not divide the cache's pages of "
                                     f"{block_size}.")
                # every group holds the same number of tokens, in pages of its own size
                make = lambda: PagedGroup(spec, [], PagePool(num_blocks * (block_size // tokens)), tokens)
            elif isinstance(spec, StateSpec):
                groups, kind = self.state_groups, "state"
                make = lambda: StateGroup(spec, [])
            else:
                raise TypeError(f"Cache slot {slot}: unknown cache spec {spec!r}.")
            for g, group in enumerate(groups):
                if group.spec == spec:
                    break
            else:
                groups.append(make())
                g = len(groups) - 1
            groups[g].slots.append(slot)
            self.slot_location.append((kind, g, len(groups[g].slots) - 1))
        # Whether pages may be shared between requests is the caller's decision (a model whose parts keep per-request
        # state that is no function of pages says no); there must be pages to share.  A group with a window
        # shares the pages its window still covers.
        self.prefix_caching = bool(prefix_caching and self.groups)
        self._prefixes: dict[bytes, _PrefixEntry] = {}
        self._clock = 0
        self.evictions = 0
        self._free_state_slots = list(range(max_sequences - 1, -1, -1))
        self.live: set[SequenceCache] = set()

    # ------------------------------------------------------------------ storage
    def attach_storage(self, dtype, device) -> None:
        """Allocate the pools on the device.  Host-only users (tests, planning) never call this."""
        import torch
        for g in self.groups:
            # keys [slot, page, head, token, dim]; values [slot, page, head, dim, token]: the keys of one
            # dimension lie together, which is how the P.V matrix product reads them
            n, kv, hd, vd = len(g.slots), g.spec.kv_heads, g.spec.head_dim, g.spec.value_dim or g.spec.head_dim
            kept = dtype if g.spec.dtype is None else getattr(torch, g.spec.dtype)
            g.k = torch.zeros((n, g.pool.num_pages, kv, g.page_tokens, hd), dtype=kept, device=device)
            g.v = torch.zeros((n, g.pool.num_pages, kv, vd, g.page_tokens), dtype=kept, device=device)
        for g in self.state_groups:
            # one slot more than requests can hold: `spare_state_slot`, where the padding rows of a recorded
            # step keep their state, so that no part has to tell them from real rows
            g.data = torch.zeros((len(g.slots), self.max_sequences + 1, *g.spec.shape),
                                 dtype=getattr(torch, g.spec.dtype), device=device)

    @property
    def spare_state_slot(self) -> int:
        """A state slot that no request ever holds (the last row of every state tensor)."""
        return self.max_sequences

    @staticmethod
    def pool_bytes(slot_specs, block_size: int, num_blocks: int, max_sequences: int, element_size: int) -> int:
        """Device bytes of the pools and state tensors that a manager of these options would allocate for cache
        elements of `element_size` bytes.  Plain arithmetic on the specs: nothing is built, so an absurd option
        costs nothing before the memory budget refuses it."""
        total = 0
        for spec in slot_specs:
            if isinstance(spec, PagedKVSpec):
                # every pool holds num_blocks * block_size tokens, whatever its page size
                size = element_size if spec.dtype is None else _DTYPE_BYTES[spec.dtype]
                total += num_blocks * block_size * spec.kv_heads * (spec.head_dim + (spec.value_dim or spec.head_dim)) * size
            elif isinstance(spec, StateSpec):
                count = 1
                for n in spec.shape:
                    count *= n
                total += (max_sequences + 1) * count * _DTYPE_BYTES.get(spec.dtype, 4)
            else:
                raise TypeError(f"Unknown cache spec {spec!r}.")
        return total

    def storage_bytes(self, element_size: int) -> int:
        """Device bytes of every pool and state tensor for cache elements of `element_size` bytes."""
        specs = [g.spec for g in self.groups for _ in g.slots] + [g.spec for g in self.state_groups for _ in g.slots]
        return self.pool_bytes(specs, self.block_size, self.num_blocks, self.max_sequences, element_size)

    # ------------------------------------------------------------------ sequences
    def create(self) -> SequenceCache:
        if not self._free_state_slots:
            raise PageError("No free sequence slot: more live sequences than max_sequences.")
        slot = self._free_state_slots.pop()
        for g in self.state_groups:
            if g.data is not None:
                g.data[:, slot].zero_()
        seq = SequenceCache(self, slot)
        self.live.add(seq)
        return seq

    @staticmethod
    def _chain(parent: bytes, tokens) -> bytes:
        return hashlib.blake2b(parent + struct.pack(f"<{len(tokens)}q", *tokens), digest_size=16).digest()

    def reuse_prefix(self, tokens) -> SequenceCache:
        """A new sequence that already holds the longest cached run of full pages of `tokens`.

        At least one token is always left to compute, also when the tokens end on a page edge
        (reference: src/kv-cache.ts:100-112).
        """
        seq = self.create()
        if not self.prefix_caching:
            return seq
        bs, key = self.block_size, b""
        keys, entries = [], []
        end = bs
        while end < len(tokens):
            parent, key = key, self._chain(key, tokens[end - bs:end])
            entry = self._prefixes.get(key)
            # The reference keys its index by the tokens themselves (src/kv-cache.ts:103,118) and cannot take one
            # prefix for another; a hash can, so a hit also has to show the same tokens behind the same parent.
            if entry is None or entry.parent != parent or entry.tokens != tuple(tokens[end - bs:end]):
                break
            keys.append(key)
            entries.append(entry)
            end += bs
        # The request computes position n * bs next and reads, in a group with a window, the keys from
        # n * bs - window + 1 on: the longest run of pages whose entries still hold those.
        n = len(entries)
        while n > 0 and not all(entries[i].pages[gi] is not None
                                for gi, g in enumerate(self.groups) if g.spec.window is not None
                                for i in range(self._first_needed(g, n * bs) // bs, n)):
            n -= 1
        for i in range(n):
            self._clock += 1
            entries[i].last_used = self._clock
        for gi, g in enumerate(self.groups):
            first = 0 if g.spec.window is None else self._first_needed(g, n * bs) // bs
            for i in range(n):
                if i >= first:
                    for page in entries[i].pages[gi]:
                        g.pool.retain(page)
                    seq.blocks[gi].extend(entries[i].pages[gi])
                else:
                    seq.blocks[gi].extend([FREED] * (bs // g.page_tokens))
            if n:
                seq.table_versions[gi] += 1
        seq.prefix_keys = keys[:n]
        seq.length = n * bs
        return seq

    @staticmethod
    def _first_needed(group, length: int) -> int:
        """The oldest key that the token at position `length` reads in `group`."""
        return 0 if group.spec.window is None else max(0, length - group.spec.window + 1)

    def publish(self, tokens, seq: SequenceCache, length: int | None = None) -> None:
        """Offer the full page of `seq` that ends at `length` (default: its computed length) for reuse.

        `tokens[:length]` are the tokens computed so far; the first publisher of a prefix wins
        (reference: src/kv-cache.ts:114-123).
        """
        length = seq.length if length is None else length
        if not self.prefix_caching or seq.released or length == 0 or length % self.block_size:
            return
        if len(tokens) < length or length > seq.length:
            raise ValueError("Prefix tokens must cover the published length, which must be computed.")
        bs = self.block_size
        n_pages = length // bs
        while len(seq.prefix_keys) < n_pages:
            i = len(seq.prefix_keys)
            parent = seq.prefix_keys[-1] if seq.prefix_keys else b""
            seq.prefix_keys.append(self._chain(parent, tokens[i * bs:(i + 1) * bs]))
        key = seq.prefix_keys[n_pages - 1]
        parent = seq.prefix_keys[n_pages - 2] if n_pages > 1 else b""
        mine_tokens = tuple(tokens[(n_pages - 1) * bs:n_pages * bs])
        # every group's pages of these `bs` tokens (a window may already have passed some of them, when a long
        # portion was computed in one step: then the entry holds none of that group)
        pages = []
        for g, blocks in zip(self.groups, seq.blocks):
            per = bs // g.page_tokens
            mine = blocks[(n_pages - 1) * per:n_pages * per]
            pages.append(None if FREED in mine else list(mine))
        known = self._prefixes.get(key)
        if known is not None:
            # The first publisher wins.  Where the entry has meanwhile given a windowed group's pages back (pool
            # pressure), a later publisher of the same tokens puts its own there, or that prefix would stay
            # half-shared for as long as its chain is in use.
            if known.parent == parent and known.tokens == mine_tokens:
                for gi, (g, mine) in enumerate(zip(self.groups, pages)):
                    if known.pages[gi] is None and mine is not None:
                        for page in mine:
                            g.pool.retain(page)
                        known.pages[gi] = mine
            return
        for g, mine in zip(self.groups, pages):
            for page in mine or ():
                g.pool.retain(page)   # the cache's own reference, beside the live requests'
        self._clock += 1
        self._prefixes[key] = _PrefixEntry(pages, self._clock, parent, mine_tokens)

    def _evict_one(self, group: int | None = None) -> bool:
        """Make a page free: drop the least recently used prefix entry that only the cache still holds.  For a
        group with a window (`group`) a lesser step comes first: the least recently used entry gives back its
        page of that group alone, if nobody else holds it, and stays as a link of its chain."""
        if group is not None and self.groups[group].spec.window is not None:
            pool, best = self.groups[group].pool, None
            for entry in self._prefixes.values():
                mine = entry.pages[group]
                if mine is not None and all(pool.refs[p] == 1 for p in mine) and (best is None or entry.last_used < best.last_used):
                    best = entry
            if best is not None:
                for page in best.pages[group]:
                    pool.release(page)
                best.pages[group] = None
                self.evictions += 1
                return True
        best_key, best = None, None
        for key, entry in self._prefixes.items():
            if all(g.pool.refs[p] == 1 for g, mine in zip(self.groups, entry.pages) for p in mine or ()):
                if best is None or entry.last_used < best.last_used:
                    best_key, best = key, entry
        if best is None:
            return False
        del self._prefixes[best_key]
        for g, mine in zip(self.groups, best.pages):
            for page in mine or ():
                g.pool.release(page)
        self.evictions += 1
        return True

    def pages_needed(self, seq: SequenceCache, new_length: int) -> list[int]:
        """Pages each group must still allocate so that `seq` can hold `new_length` tokens."""
        return [max(0, -(-new_length // g.page_tokens) - len(blocks)) for g, blocks in zip(self.groups, seq.blocks)]

    def reserve(self, seq: SequenceCache, new_length: int) -> bool:
        """Allocate pages in every group for tokens up to `new_length`.  All or nothing.

        When a pool is empty, cached prefix pages that no request uses are evicted, least recently
        used first (reference: src/kv-cache.ts:125-140).
        """
        seq._live()
        if new_length < seq.length:
            raise ValueError("A sequence cannot shrink.")
        taken: list[tuple[int, int]] = []
        for gi, (g, count) in enumerate(zip(self.groups, self.pages_needed(seq, new_length))):
            for _ in range(count):
                page = g.pool.allocate()
                while page is None and self._evict_one(gi):
                    page = g.pool.allocate()
                if page is None:
                    for gj, p in reversed(taken):
                        self.groups[gj].pool.release(p)
                        seq.blocks[gj].pop()
                        seq.table_versions[gj] += 1
                    return False
                seq.blocks[gi].append(page)
                seq.table_versions[gi] += 1
                taken.append((gi, page))
        return True

    def commit(self, seq: SequenceCache, new_length: int) -> None:
        """The step has written tokens up to `new_length`: record it and give back what windows have passed."""
        seq._live()
        if any(new_length > len(blocks) * g.page_tokens for g, blocks in zip(self.groups, seq.blocks)):
            raise PageError("Committed more tokens than pages were reserved for.")
        seq.length = new_length
        for gi, (g, blocks) in enumerate(zip(self.groups, seq.blocks)):
            if g.spec.window is None:
                continue
            # the next token (position new_length) reads keys >= new_length - window + 1
            for i in range(self._first_needed(g, new_length) // g.page_tokens):
                if blocks[i] != FREED:
                    g.pool.release(blocks[i])
                    blocks[i] = FREED
                    seq.table_versions[gi] += 1

    def release(self, seq: SequenceCache) -> None:
        if seq.released:
            return
        for g, blocks in zip(self.groups, seq.blocks):
            for page in blocks:
                if page != FREED:
                    g.pool.release(page)
            blocks.clear()
        self._free_state_slots.append(seq.state_slot)
        seq.released = True
        self.live.discard(seq)

    def clear_prefixes(self) -> None:
        for entry in self._prefixes.values():
            for g, mine in zip(self.groups, entry.pages):
                for page in mine or ():
                    g.pool.release(page)
        self._prefixes.clear()

    # ------------------------------------------------------------------ reports
    def free_pages(self) -> list[int]:
        return [g.pool.num_free for g in self.groups]

    def snapshot(self) -> dict:
        """Reference: src/kv-cache.ts:162-171, one record per group."""
        groups = []
        for gi, g in enumerate(self.groups):
            cached = {p for e in self._prefixes.values() for p in e.pages[gi] or ()}
            groups.append({
                "window": g.spec.window, "page_tokens": g.page_tokens, "slots": list(g.slots), "total_pages": g.pool.num_pages,
                "free_pages": g.pool.num_free, "cached_pages": len(cached),
                "pages": [{"id": i, "refs": r, "cached": i in cached, "active_refs": r - (i in cached)}
                          for i, r in enumerate(g.pool.refs)],
            })
        first = groups[0] if groups else {"total_pages": 0, "free_pages": 0, "cached_pages": 0, "pages": []}
        return {"total_pages": first["total_pages"], "free_pages": first["free_pages"],
                "cached_pages": first["cached_pages"], "evictions": self.evictions, "pages": first["pages"],
                "groups": groups, "free_sequence_slots": len(self._free_state_slots)}
