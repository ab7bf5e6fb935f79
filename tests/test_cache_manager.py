"""The cache manager on the CPU: no page lost, held twice or freed twice, under random
orders of requests; the reference's own block-manager sequence; windowed groups."""

import random

import pytest

from bitwise_amd.cache.manager import CacheManager, GroupSpec
from bitwise_amd.cache.pages import PagePool, StateSlots, block_hash
from plain_llama import block_hash as plain_block_hash


def test_reference_block_manager_sequence():
    """tests/test_main.cpp:171-197, step by step."""
    m = PagePool(4, 16, prefix_caching=True)
    assert m.available() == 4
    a, b = m.allocate(), m.allocate()
    assert a is not None and b is not None and a != b and (a, b) == (0, 1)      # low ids first
    toks, other = list(range(16)), list(range(1, 17))
    h = block_hash(0, toks)
    m.register_full(a, h, toks)
    assert m.lookup(h, other) is None                 # same hash, different tokens: never a hit
    hit = m.lookup(h, toks)
    assert hit == a and m.refcount(a) == 2
    m.release(a)
    m.release(a)                                       # now cached but unreferenced
    assert m.available() == 3
    assert m.lookup(h, toks) == a                      # revived from the evictable list
    m.release(a)
    c, d, e = m.allocate(), m.allocate(), m.allocate()
    assert None not in (c, d, e) and m.evictions == 1  # free pages first, then the cached one
    assert m.lookup(h, toks) is None
    assert m.allocate() is None
    m.check()


def test_block_hash_matches_the_plain_formula_and_chains():
    toks = [5, 17, 3, 0, 255, 2 ** 31 - 1, 7, 7]
    assert block_hash(0, toks) == plain_block_hash(0, toks)
    assert block_hash(123456789, toks) == plain_block_hash(123456789, toks)
    assert block_hash(0, toks) != block_hash(1, toks) and block_hash(0, toks) != block_hash(0, toks[::-1])


def test_double_release_is_an_error():
    m = PagePool(2, 8)
    p = m.allocate()
    m.release(p)
    with pytest.raises(RuntimeError, match="unreferenced"):
        m.release(p)
    s = StateSlots(2)
    x = s.allocate()
    s.release(x)
    with pytest.raises(RuntimeError, match="free slot"):
        s.release(x)


@pytest.mark.parametrize("seed", range(25))
def test_random_orders_lose_nothing(seed):
    """Requests open, grow, share prefixes, get preempted and close in random order; after
    every operation every page is free, cached or referenced exactly once per holder."""
    rng = random.Random(seed)
    ps = rng.choice([8, 16])
    windows = rng.choice([[None], [None], [None, 24], [40]])
    mgr = CacheManager([GroupSpec(w) for w in windows], num_pages=rng.randint(6, 20), page_size=ps, num_slots=5,
                       prefix_caching=rng.random() < 0.7)
    prefix = [rng.randrange(50) for _ in range(3 * ps)]
    live = []
    for _ in range(400):
        op = rng.random()
        if op < 0.25 and len(live) < 5:
            rc = mgr.open()
            assert rc is not None
            toks = (prefix if rng.random() < 0.6 else []) + [rng.randrange(50) for _ in range(rng.randint(1, 30))]
            mgr.admit_prefix(rc, toks)
            live.append((rc, toks))
        elif op < 0.8 and live:
            rc, toks = rng.choice(live)
            n = rng.randint(1, 12)
            target = min(rc.computed + n, len(toks))
            if target == rc.computed:
                toks.append(rng.randrange(50))
                target += 1
            if mgr.ensure(rc, target):
                mgr.advance(rc, toks, target)
            else:                                   # out of pages: recompute preemption of this request
                mgr.release_pages(rc)
                assert rc.computed == 0 and all(not t for t in rc.tables)
        elif live:
            rc, toks = live.pop(rng.randrange(len(live)))
            mgr.close(rc)
        mgr.check()
        held = {}
        for rc, _ in live:
            for g, table in enumerate(rc.tables):
                for page in table:
                    if page >= 0:
                        held[(g, page)] = held.get((g, page), 0) + 1
        for (g, page), count in held.items():
            assert mgr.pools[g].refcount(page) == count          # shared only through the prefix cache
            if not mgr.prefix_caching:
                assert count == 1
        for g, pool in enumerate(mgr.pools):
            referenced = sum(1 for page in range(pool.num_pages) if pool.refcount(page) > 0)
            assert referenced == len([1 for (gg, _) in held if gg == g])
            assert pool.available() == pool.num_pages - referenced
    for rc, _ in live:
        mgr.close(rc)
    assert mgr.all_free()


def test_window_pages_are_given_back_as_the_window_passes():
    mgr = CacheManager([GroupSpec(None), GroupSpec(20)], num_pages=16, page_size=8, num_slots=2)
    rc = mgr.open()
    toks = list(range(100))
    assert mgr.ensure(rc, 30)
    mgr.advance(rc, toks, 30)
    # next query at position 30 reads keys 11..30 in the windowed group: page 0 (keys 0-7) is gone
    assert rc.tables[1][0] == -1 and rc.tables[1][1] >= 0 and all(p >= 0 for p in rc.tables[0])
    assert mgr.free_pages(1) == 16 - 3 and mgr.free_pages(0) == 16 - 4
    for target in range(31, 101):
        assert mgr.ensure(rc, target)
        mgr.advance(rc, toks, target)
        live = [p for p in rc.tables[1] if p >= 0]
        assert len(live) <= 20 // 8 + 2                            # the window plus partial pages at both ends
        first = (target - 20 + 1) // 8 if target >= 20 else 0
        assert all(p == -1 for p in rc.tables[1][:first]) and all(p >= 0 for p in rc.tables[1][first:])
    assert len([p for p in rc.tables[0] if p >= 0]) == 13
    mgr.close(rc)
    assert mgr.all_free()


def test_prefix_reuse_is_decided_group_by_group():
    """A group that keeps all keys and one with a window of 20 keys, pages of 8: a second request with the same
    tokens starts behind as many pages as every group can still serve: all of them in the first group, the pages
    under the window in the second (found again although the first request gave them back when its window had
    passed them).  Once those have been evicted the prefix is not reused in either group."""
    mgr = CacheManager([GroupSpec(None), GroupSpec(20)], num_pages=12, page_size=8, num_slots=3)
    assert mgr.prefix_caching
    toks = [(i * 7 + 3) % 50 for i in range(60)]
    a = mgr.open()
    for upto in (13, 29, 30, 47, 60):
        assert mgr.ensure(a, upto)
        mgr.advance(a, toks, upto)
        mgr.check()
    assert a.tables[1][:5] == [-1] * 5 and all(p >= 0 for p in a.tables[1][5:]) and len(a.hashes) == 7
    b = mgr.open()
    assert mgr.admit_prefix(b, toks) == 56                         # 7 full pages; the last token's page is computed
    assert b.tables[0] == a.tables[0][:7]
    assert b.tables[1][:4] == [-1] * 4 and all(p >= 0 for p in b.tables[1][4:7])     # position 56 reads keys 37..: pages 4, 5, 6
    assert b.tables[1][5:7] == a.tables[1][5:7] and mgr.pools[1].refcount(b.tables[1][4]) == 1     # page 4: a had given it back
    # a shorter prompt with the same start: 3 full pages, the window of position 24 starts in page 0
    c = mgr.open()
    assert mgr.admit_prefix(c, toks[:30]) == 24 and all(p >= 0 for p in c.tables[1]) and c.tables[0] == a.tables[0][:3]
    for rc in (a, b, c):
        mgr.close(rc)
    mgr.check()
    assert mgr.all_free()
    # everything is still cached; now the windowed group's pool is filled by someone else: its cached pages are evicted
    d = mgr.open()
    other = [49 - t for t in toks] + list(range(40))
    assert mgr.ensure(d, 96)
    assert mgr.pools[1].evictions > 0 and mgr.pools[0].evictions > 0
    mgr.close(d)
    e = mgr.open()
    hit = mgr.admit_prefix(e, toks)
    assert hit % 8 == 0 and hit < 56
    lo = mgr.first_needed_page(1, hit)
    assert all(p >= 0 for p in e.tables[0]) and all(p >= 0 for p in e.tables[1][lo:]) and len(e.tables[0]) == len(e.tables[1]) == hit // 8
    mgr.close(e)
    mgr.check()
    assert mgr.all_free()


def test_prefix_reuse_rules():
    mgr = CacheManager([GroupSpec(None)], num_pages=8, page_size=8, num_slots=3)
    toks = list(range(24)) + [99]
    a = mgr.open()
    assert mgr.admit_prefix(a, toks) == 0
    assert mgr.ensure(a, 25)
    mgr.advance(a, toks, 25)
    assert len(a.hashes) == 3                                       # only full pages are registered
    b = mgr.open()
    assert mgr.admit_prefix(b, toks) == 24 and b.tables[0] == a.tables[0][:3]
    c = mgr.open()
    assert mgr.admit_prefix(c, toks[:24]) == 16                    # the page of the last token is computed
    assert mgr.admit_prefix(c, toks[:24]) == 16                    # asking again takes nothing more
    assert mgr.pools[0].refcount(a.tables[0][0]) == 3
    for rc in (a, b, c):
        mgr.close(rc)
    assert mgr.free_pages() == 8
    d = mgr.open()                                                  # cached pages outlive their requests
    assert mgr.admit_prefix(d, toks) == 24
    mgr.close(d)
    off = CacheManager([GroupSpec(None)], 8, 8, 2, prefix_caching=True, has_state=True)
    assert not off.prefix_caching                                   # state outside the pages cannot be reused


def test_two_storages_on_one_model_share_nothing():
    """Caches, state and page size belong to a storage, not to the model: a second storage (another engine, a
    replayer, Model.logits) leaves the first one's tensors and the model's plan alone."""
    from tiny import TINY_A
    from bitwise_amd.config.llama import LlamaConfig
    from bitwise_amd.engine.storage import CacheStorage
    from bitwise_amd.models.assembled import AssembledModel
    from bitwise_amd.models.llama import llama_spec
    from bitwise_amd.runtime import Runtime

    asm = AssembledModel(llama_spec(LlamaConfig.from_dict(TINY_A)), Runtime("float32", None))   # described only: host tensors
    first = CacheStorage(asm, num_pages=4, num_slots=2, page_size=16)
    mine = [(c.k_cache, c.v_cache) for c in first.bindings]
    second = CacheStorage(asm, num_pages=9, num_slots=3, page_size=8)
    assert all(c.k_cache is None and c.v_cache is None and c.state is None for c in asm.calls)
    for c, (k, v) in zip(first.bindings, mine):
        assert c.k_cache is k and c.v_cache is v and k.shape[0] == 4
    assert [c.k_cache.shape for c in second.bindings] == [(9, 2 * 8 * 16)] * 2
    assert first.bindings[0].k_cache.data_ptr() != second.bindings[0].k_cache.data_ptr()
    assert first.page_size == 16 and second.page_size == 8


def test_slot_records_position_and_seed():
    from bitwise_amd.cache.manager import CacheManager, GroupSpec

    m = CacheManager([GroupSpec(None)], 8, 4, 2, prefix_caching=False)
    rc = m.open(seed=77)
    assert (m.record(rc).position, m.record(rc).seed, m.record(rc).stream) == (0, 77, 0)
    assert m.ensure(rc, 9)
    m.advance(rc, list(range(9)), 9)
    assert m.record(rc).position == 9
    m.close(rc)
    again = m.open(seed=5)
    assert (m.record(again).position, m.record(again).seed) == (0, 5)
