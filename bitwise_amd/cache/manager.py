"""The cache manager: for every request a block table per cache group and a state slot.

A *group* is a set of caches (one per layer call that writes one) with the same needs: all
keys, or a window of them.  Every group has a page pool of its own.  A request's pages are
given back when it ends, is preempted or cancelled, and, in a windowed group, as soon as the
window has passed them; cached full pages of a finished request stay until the space is
needed (reference: src/engine.cpp:146-220, src/block_manager.cpp).

Prefix reuse (src/engine.cpp:176-205) is only sound when the reused pages hold everything the
request has computed for its first tokens.  That is decided group by group: every group
registers its full pages under the request's hash chain; a request may start behind n cached
pages if every group still has the pages a query at position n * page_size reads there: all n
in a group that keeps all keys, the pages under the window in a windowed group (pages the
window has passed are given back, and stay findable until their space is needed).  State that
a mixer keeps in a slot is in no page, so a model with such a mixer has no prefix reuse.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence

from ..config.engine import Fault
from .pages import PagePool, StateSlots, block_hash


@dataclass(frozen=True)
class GroupSpec:
    window: Optional[int] = None       # None: all keys stay


@dataclass
class RequestCache:
    slot: int
    tables: List[List[int]]            # per group: page of positions [i*page, (i+1)*page); -1 once given back
    hashes: List[int] = field(default_factory=list)   # hash chain of this request's registered full pages
    computed: int = 0                  # tokens whose keys and values are in the cache


class CacheManager:
    def __init__(self, groups: Sequence[GroupSpec], num_pages: int, page_size: int, num_slots: int,
                 prefix_caching: bool = True, has_state: bool = False, fault: int = 0):
        self.groups = list(groups)
        self.fault = int(fault)            # a test-only bug for the simulator to catch (config.engine.Fault)
        self.page_size = page_size
        self.num_pages = num_pages
        self.prefix_caching = bool(prefix_caching) and not has_state and len(self.groups) > 0
        self.pools = [PagePool(num_pages, page_size, self.prefix_caching) for _ in self.groups]
        self.slots = StateSlots(num_slots)
        # called with (group, page) whenever a page becomes free (tests fill such pages with NaN, so that a
        # page that is handed out again must be written before it is read)
        self.on_free = None

    # ------------------------------------------------------------------ requests
    def open(self, seed: int = 0, stream: int = 0) -> Optional[RequestCache]:
        """Take a state slot; it records the request's position (0 now) and the key of its random draws."""
        slot = self.slots.allocate(seed, stream)
        if slot is None:
            return None
        return RequestCache(slot=slot, tables=[[] for _ in self.groups])

    def record(self, rc: RequestCache):
        return self.slots.records[rc.slot]

    def close(self, rc: RequestCache) -> None:
        """Give back every page and the slot."""
        self.release_pages(rc)
        self.slots.release(rc.slot)
        rc.slot = -1

    def release_pages(self, rc: RequestCache) -> None:
        for g, (pool, table) in enumerate(zip(self.pools, rc.tables)):
            for page in table:
                if page >= 0 and pool.release(page) and self.on_free is not None:
                    self.on_free(g, page)
        # new lists, not cleared ones: a table only ever grows at its end while it is the same object (the step
        # function's host copy of a block table relies on that)
        rc.tables = [[] for _ in self.pools]
        rc.hashes.clear()
        rc.computed = 0

    # ------------------------------------------------------------------ prefix reuse
    def admit_prefix(self, rc: RequestCache, tokens: Sequence[int]) -> int:
        """Take cached pages holding a prefix of ``tokens``.  The page holding the last token
        is never reused, so that its logits are computed (src/engine.cpp:178-179)."""
        if not self.prefix_caching or any(rc.tables):
            return rc.computed
        ps = self.page_size
        full = (len(tokens) - (0 if self.fault == Fault.PREFIX_COVERS_LAST_TOKEN else 1)) // ps
        chain: List[int] = []                       # the hash chain of the request's full pages
        parent = 0
        for i in range(full):
            parent = block_hash(parent, tokens[i * ps:(i + 1) * ps])
            chain.append(parent)

        def has(g: int, i: int) -> bool:
            return self.pools[g].peek(chain[i], tokens[i * ps:(i + 1) * ps]) is not None

        # groups that keep all keys need pages 0..n-1: n is at most their common run of hits from the start
        n = full
        for g, spec in enumerate(self.groups):
            if spec.window is None:
                n = next((i for i in range(n) if not has(g, i)), n)
        # windowed groups need the pages under the window of the next position: the longest n they all still hold
        while n > 0 and not all(has(g, i) for g, spec in enumerate(self.groups) if spec.window is not None
                                for i in range(self.first_needed_page(g, n * ps), n)):
            n -= 1
        for g, (pool, table) in enumerate(zip(self.pools, rc.tables)):
            lo = self.first_needed_page(g, n * ps)
            for i in range(n):
                table.append(pool.lookup(chain[i], tokens[i * ps:(i + 1) * ps]) if i >= lo else -1)
        rc.hashes.extend(chain[:n])
        rc.computed = n * ps
        self.slots.records[rc.slot].position = rc.computed
        return rc.computed

    # ------------------------------------------------------------------ growth
    def first_needed_page(self, group: int, next_position: int) -> int:
        """Index of the first page a query at ``next_position`` still reads in this group."""
        w = self.groups[group].window
        if w is None:
            return 0
        return max(0, next_position - w + 1) // self.page_size

    def ensure(self, rc: RequestCache, tokens: int) -> bool:
        """Make the request's tables cover positions [computed, tokens).  False if a pool ran
        out; pages taken so far stay with the request (the caller preempts or releases)."""
        need = (tokens + self.page_size - 1) // self.page_size
        for g, (pool, table) in enumerate(zip(self.pools, rc.tables)):
            lo = self.first_needed_page(g, rc.computed)
            while len(table) < need:
                if len(table) < lo:
                    table.append(-1)             # wholly before the window: never allocated
                    continue
                page = pool.allocate()
                if page is None:
                    return False
                table.append(page)
        return True

    def can_ever_hold(self, tokens: int, step_tokens: int) -> bool:
        """Whether a request of ``tokens`` tokens fits an empty engine (src/engine.cpp:130-133): every group's
        pool must hold what the request holds there at once, all its pages in a group that keeps all keys, and
        in a windowed group the window and one step's tokens (and the page either end may straddle)."""
        ps = self.page_size
        for g in self.groups:
            held = tokens if g.window is None else min(tokens, g.window + step_tokens + 2 * ps)
            if (held + ps - 1) // ps > self.num_pages:
                return False
        return True

    def pages_missing(self, rc: RequestCache, tokens: int) -> int:
        """Most pages any pool would have to hand out for ``ensure(rc, tokens)``."""
        need = (tokens + self.page_size - 1) // self.page_size
        return max((max(0, need - len(t)) for t in rc.tables), default=0)

    def advance(self, rc: RequestCache, tokens: Sequence[int], computed: int) -> None:
        """After a step: ``computed`` tokens are in the cache.  Register newly full pages
        (src/engine.cpp:196-205) and give back pages a window has passed."""
        rc.computed = computed
        self.slots.records[rc.slot].position = computed
        ps = self.page_size
        if self.prefix_caching:
            full = computed // ps
            if self.fault == Fault.REGISTER_UNFINISHED_PAGE:        # (the page's tokens are known, its keys not yet there)
                full = min(min(len(t) for t in rc.tables), (computed + ps - 1) // ps, len(tokens) // ps)
            for i in range(len(rc.hashes), full):
                toks = tokens[i * ps:(i + 1) * ps]
                h = block_hash(rc.hashes[i - 1] if i else 0, toks)
                for pool, table in zip(self.pools, rc.tables):
                    if table[i] >= 0:                               # (a page before the window was never held)
                        pool.register_full(table[i], h, toks)
                rc.hashes.append(h)
        for g, (pool, table) in enumerate(zip(self.pools, rc.tables)):
            if self.groups[g].window is None:
                continue
            lo = min(self.first_needed_page(g, computed), len(table))
            for i in range(lo):
                if table[i] >= 0:
                    if pool.release(table[i]) and self.on_free is not None:
                        self.on_free(g, table[i])
                    table[i] = -1

    # ------------------------------------------------------------------ accounting
    def free_pages(self, group: int = 0) -> int:
        return self.pools[group].available()

    def free_pages_least(self) -> int:
        """Free pages of the pool that has the fewest (all pools full-sized if the model keeps no paged cache)."""
        return min((p.available() for p in self.pools), default=self.num_pages)

    def all_free(self) -> bool:
        return all(p.available() == p.num_pages for p in self.pools) and self.slots.available() == self.slots.num_slots

    @property
    def evictions(self) -> int:
        return sum(p.evictions for p in self.pools)

    def check(self) -> None:
        for p in self.pools:
            p.check()
