"""Host bookkeeping of cache pages: reference counts, a free stack, and a prefix cache of
full pages keyed by a hash chain (the reference's BlockManager, src/block_manager.h:2-9,
src/block_manager.cpp:21-88, with the page size a run-time value instead of 16).
"""

from __future__ import annotations

from collections import OrderedDict
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

_M64 = (1 << 64) - 1


def block_hash(parent: int, tokens: Sequence[int]) -> int:
    """FNV-1a over the parent hash and the page's tokens, then a 64-bit mixer
    (src/block_manager.cpp:8-19).  The parent of a sequence's first page is 0."""
    h = 1469598103934665603 ^ parent
    for t in tokens:
        h ^= t & 0xFFFFFFFF
        h = (h * 1099511628211) & _M64
    h ^= h >> 33
    h = (h * 0xFF51AFD7ED558CCD) & _M64
    h ^= h >> 33
    return h


class PagePool:
    """Pages 0..num_pages-1 of one cache group.

    A page is free (never used or given back without a hash), referenced (count > 0), or
    cached: full, registered under its hash, count 0, waiting in least-recently-released
    order until the space is needed.  ``allocate`` hands out free pages first, low ids
    first, then evicts the oldest cached page.
    """

    def __init__(self, num_pages: int, page_size: int, prefix_caching: bool = True):
        if num_pages < 1 or page_size < 1:
            raise ValueError("a pool needs at least one page of at least one token")
        self.page_size = page_size
        self.prefix_caching = prefix_caching
        self._ref: List[int] = [0] * num_pages
        self._hash_of: List[Optional[int]] = [None] * num_pages
        self._tokens_of: List[Optional[Tuple[int, ...]]] = [None] * num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))   # pop() gives low ids first
        self._evictable: "OrderedDict[int, None]" = OrderedDict()
        self._by_hash: Dict[int, int] = {}
        self.evictions = 0

    @property
    def num_pages(self) -> int:
        return len(self._ref)

    def available(self) -> int:
        """Pages that can be handed out right now (free or cached without a reference)."""
        return len(self._free) + len(self._evictable)

    def refcount(self, page: int) -> int:
        return self._ref[page]

    def allocate(self) -> Optional[int]:
        if self._free:
            page = self._free.pop()
        elif self._evictable:
            page, _ = self._evictable.popitem(last=False)
            self._forget(page)
            self.evictions += 1
        else:
            return None
        self._ref[page] = 1
        return page

    def release(self, page: int) -> bool:
        """Drop one reference.  True if the page is free now: nobody holds it and it is not kept
        as a cached page either, so what it holds is dead."""
        if self._ref[page] <= 0:
            raise RuntimeError(f"release of unreferenced page {page}")
        self._ref[page] -= 1
        if self._ref[page] > 0:
            return False
        if self._hash_of[page] is not None:
            self._evictable[page] = None          # newest at the tail
            return False
        self._free.append(page)
        return True

    def peek(self, hash_: int, tokens: Sequence[int]) -> Optional[int]:
        """The page ``lookup`` would give, without taking it."""
        if not self.prefix_caching:
            return None
        page = self._by_hash.get(hash_)
        if page is None or self._tokens_of[page] != tuple(tokens):
            return None
        return page

    def lookup(self, hash_: int, tokens: Sequence[int]) -> Optional[int]:
        """A cached full page with this hash AND these tokens; takes a reference on a hit."""
        page = self.peek(hash_, tokens)
        if page is None:
            return None
        self._evictable.pop(page, None)
        self._ref[page] += 1
        return page

    def register_full(self, page: int, hash_: int, tokens: Sequence[int]) -> None:
        """First writer wins: an identical page already cached under the hash is kept."""
        if not self.prefix_caching or self._hash_of[page] is not None or hash_ in self._by_hash:
            return
        self._hash_of[page] = hash_
        self._tokens_of[page] = tuple(tokens)
        self._by_hash[hash_] = page

    def _forget(self, page: int) -> None:
        h = self._hash_of[page]
        if h is not None:
            del self._by_hash[h]
            self._hash_of[page] = None
            self._tokens_of[page] = None

    def check(self) -> None:
        """Invariants: every page is in exactly one of free / cached / referenced."""
        free, cached = set(self._free), set(self._evictable)
        if len(free) != len(self._free):
            raise AssertionError("a page is on the free stack twice")
        if free & cached:
            raise AssertionError("a page is both free and cached")
        for page, ref in enumerate(self._ref):
            states = (page in free) + (page in cached) + (ref > 0)
            if states != 1:
                raise AssertionError(f"page {page}: free={page in free} cached={page in cached} ref={ref}")
            if page in cached and self._hash_of[page] is None:
                raise AssertionError(f"cached page {page} has no hash")
        for h, page in self._by_hash.items():
            if self._hash_of[page] != h:
                raise AssertionError("hash index out of step")


@dataclass
class SlotRecord:
    """What a request's slot holds on the host beside the device state of its mixers: how many of its tokens
    are in the cache (the position of its next token) and the key of its random draws."""
    position: int = 0
    seed: int = 0
    stream: int = 0


class StateSlots:
    """Slots 0..n-1 for per-request state of fixed size; lowest free slot first."""

    def __init__(self, num_slots: int):
        self._free = list(range(num_slots - 1, -1, -1))
        self._used = set()
        self.num_slots = num_slots
        self.records: List[SlotRecord] = [SlotRecord() for _ in range(num_slots)]

    def available(self) -> int:
        return len(self._free)

    def allocate(self, seed: int = 0, stream: int = 0) -> Optional[int]:
        if not self._free:
            return None
        s = self._free.pop()
        self._used.add(s)
        self.records[s] = SlotRecord(0, seed, stream)
        return s

    def release(self, slot: int) -> None:
        if slot not in self._used:
            raise RuntimeError(f"release of free slot {slot}")
        self._used.remove(slot)
        self._free.append(slot)
