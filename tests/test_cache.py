"""The cache manager without a GPU: pages are never lost, held twice or freed twice; groups
with windows give pages back; prefix reuse; state slots.  Vectors marked with a reference
location are the ones the reference's own tests hold."""

import random

import pytest

from atomserve_amd.cache import CacheManager, OutOfPagesError, PageAllocator, blocks_for_tokens, page_hash
from atomserve_amd.cache.manager import RELEASED
from atomserve_amd.engine.batch import slot_of
from atomserve_amd.parts.base import PagedCacheRequest, StateCacheRequest

H1, H2, H3 = (page_hash(b"", [i]) for i in (1, 2, 3))


def test_ceiling_and_slot_vectors():
    # reference tests/test_block_allocator.py:14-16, tests/test_kv_cache.py:18-21
    assert [blocks_for_tokens(n, 16) for n in (0, 1, 15, 16, 17, 32, 33)] == [0, 1, 1, 1, 2, 2, 3]
    assert [slot_of([7, 2, 5], p, 4) for p in (0, 3, 4, 5, 11)] == [28, 31, 8, 9, 23]


def test_allocate_is_all_or_nothing_and_pages_are_distinct():
    a = PageAllocator(8)
    x, y = a.allocate(3), a.allocate(5)
    assert set(x + y) == set(range(8)) and a.num_free == 0
    b = PageAllocator(4)
    b.allocate(3)
    with pytest.raises(OutOfPagesError):
        b.allocate(2)
    assert b.num_free == 1


def test_double_free_and_foreign_pages_are_rejected():
    a = PageAllocator(4)
    pages = a.allocate(2)
    a.free(pages)
    assert a.num_free == 4
    for bad in (pages[:1], [99], [-1]):
        with pytest.raises(ValueError, match="not allocated"):
            a.free(bad)
    p = a.allocate(1)
    with pytest.raises(ValueError, match="not allocated"):
        a.free(p + p)  # twice in one call, held once
    assert a.refcount(p[0]) == 1
    a.check()


def test_hash_chains_on_the_whole_prefix():
    tokens = [5, 6, 7, 8]
    assert page_hash(b"", tokens) == page_hash(b"", list(tokens))
    assert page_hash(H1, tokens) != page_hash(H2, tokens)
    assert page_hash(b"", [1, 2]) != page_hash(b"", [2, 1])


def test_sharing_reviving_and_eviction_order():
    # reference tests/test_block_allocator.py:65-104
    a = PageAllocator(4)
    [p] = a.allocate(1)
    a.register(p, H1)
    a.acquire(a.lookup(H1))
    a.free([p])
    assert a.num_free == 3
    a.free([p])
    assert a.num_free == 4 and a.lookup(H1) == p  # free, still cached
    a.acquire(p)
    assert a.num_free == 3  # revived out of the middle of the queue
    a.check()

    b = PageAllocator(3)
    x, y, z = b.allocate(3)
    for page, h in ((x, H1), (y, H2), (z, H3)):
        b.register(page, h)
    b.free([y])
    b.free([x, z])  # released last page first: z, then x
    assert b.allocate(2) == [y, z]
    assert b.lookup(H2) is None and b.lookup(H3) is None and b.lookup(H1) == x

    c = PageAllocator(2)
    first, second = c.allocate(2)
    c.register(first, H1)
    c.register(second, H1)
    assert c.lookup(H1) == first and c.num_cached == 1


@pytest.mark.parametrize("seed", range(5))
def test_random_orders_lose_no_page(seed):
    """Requests of random lengths arrive, grow, get released and share prefixes in random order;
    after every action each page is either free or held exactly as often as tables name it."""
    rng = random.Random(seed)
    m = CacheManager({0: PagedCacheRequest(2, 16), 1: PagedCacheRequest(2, 16)}, block_size=4, num_blocks=24, max_num_seqs=8)
    assert len(m.paged_groups) == 1  # equal needs share one group
    live = []
    for _ in range(400):
        action = rng.random()
        if action < 0.4 and len(live) < 8:
            tokens = [rng.randrange(3) for _ in range(rng.randrange(1, 30))]
            rc = m.new_request()
            done = m.adopt_cached_prefix(rc, tokens)
            if m.reserve(rc, done, len(tokens) - done):
                m.publish_full_pages(rc, tokens, len(tokens))
                live.append((rc, tokens))
            else:
                m.release(rc)
        elif action < 0.7 and live:
            rc, tokens = rng.choice(live)
            if m.reserve(rc, len(tokens), 3):
                tokens.extend(rng.randrange(3) for _ in range(3))
                m.publish_full_pages(rc, tokens, len(tokens))
        elif live:
            rc, _ = live.pop(rng.randrange(len(live)))
            m.release(rc)
            with pytest.raises(ValueError):
                m.paged_groups[0].allocator.free([10**6])
        m.check()
        alloc = m.paged_groups[0].allocator
        held = {}
        for rc, tokens in live:
            assert len(rc.tables[0]) == blocks_for_tokens(len(tokens), 4)
            for page in rc.tables[0]:
                held[page] = held.get(page, 0) + 1
        for page in range(24):
            assert alloc.refcount(page) == held.get(page, 0)
        assert alloc.num_free == 24 - len(held)
    for rc, _ in live:
        m.release(rc)
    assert m.num_free == 24


def test_groups_by_need_and_a_window_gives_pages_back():
    full, windowed = PagedCacheRequest(2, 16), PagedCacheRequest(2, 16, window=6)
    m = CacheManager({0: full, 1: windowed, 2: full, 3: windowed, 4: PagedCacheRequest(4, 8)}, 4, 16, 4)
    assert [g.cache_ids for g in m.paged_groups] == [[0, 2], [1, 3], [4]]
    assert m.group_of_cache[3] == ("paged", 1, 1)
    assert not m.prefix_reuse_possible  # a windowed group cannot serve an old prefix
    rc = m.new_request()
    assert m.reserve(rc, 0, 13)
    assert [len(t) for t in rc.tables] == [4, 4, 4]
    # next query at position 13 sees keys 8..13 in the windowed group: pages 0 and 1 are behind it
    assert m.release_behind_window(rc, 13) == 2
    assert rc.tables[1][:2] == [RELEASED, RELEASED] and RELEASED not in rc.tables[0]
    assert m.paged_groups[1].allocator.num_free == 14 and m.paged_groups[0].allocator.num_free == 12
    assert m.release_behind_window(rc, 13) == 0  # nothing is given back twice
    assert m.reserve(rc, 13, 7) and len(rc.tables[1]) == 5
    assert m.release_behind_window(rc, 16) == 0  # position 16 still sees key 11, the last of page 2
    assert m.release_behind_window(rc, 17) == 1  # position 17 sees 12..17: page 2 is behind the window
    m.release(rc)
    assert all(g.allocator.num_free == 16 for g in m.paged_groups)
    m.check()


def test_window_release_keeps_every_visible_key():
    m = CacheManager({0: PagedCacheRequest(1, 8, window=5)}, 4, 8, 2)
    rc = m.new_request()
    for computed in range(1, 30):
        assert m.reserve(rc, computed - 1, 1)
        m.release_behind_window(rc, computed)
        first_visible = max(0, computed - 5 + 1)
        for p in range(first_visible, computed):
            assert rc.tables[0][p // 4] != RELEASED, (computed, p)
        assert sum(1 for b in rc.tables[0] if b != RELEASED) <= 3  # a window of 5 touches at most 3 pages of 4
    m.release(rc)
    assert m.num_free == 8


def test_state_slots_beside_the_pages():
    m = CacheManager({0: PagedCacheRequest(1, 8), 1: StateCacheRequest((4, 2))}, 4, 8, max_num_seqs=2)
    assert len(m.state_groups) == 1 and not m.prefix_reuse_possible
    a, b, c = m.new_request(), m.new_request(), m.new_request()
    assert m.reserve(a, 0, 3) and m.reserve(b, 0, 3)
    assert {a.state_slot, b.state_slot} == {0, 1}
    assert not m.reserve(c, 0, 3) and c.tables == [[]] and c.state_slot == -1  # no slot: nothing taken
    assert m.reserve(a, 3, 4) and a.state_slot in (0, 1)  # growing keeps the slot
    m.release(a)
    assert m.reserve(c, 0, 3) and c.state_slot == 0 or c.state_slot == 1
    m.release(b)
    m.release(c)
    assert m.num_free == 8 and m.num_free_slots == 2


def test_prefix_adoption_stops_at_the_first_miss_and_leaves_a_token():
    m = CacheManager({0: PagedCacheRequest(1, 8)}, 4, 16, 4)
    tokens = list(range(40, 52))
    first = m.new_request()
    assert m.adopt_cached_prefix(first, tokens) == 0
    m.reserve(first, 0, 12)
    m.publish_full_pages(first, tokens, 10)  # pages 0 and 1 are full of computed tokens, page 2 is not
    again = m.new_request()
    assert m.adopt_cached_prefix(again, tokens) == 8 and again.tables[0] == first.tables[0][:2]
    exact = m.new_request()
    assert m.adopt_cached_prefix(exact, tokens[:8]) == 4  # at least one token is left to compute
    other = m.new_request()
    assert m.adopt_cached_prefix(other, [40, 41, 42, 99] + tokens[4:]) == 0
    for rc in (first, again, exact, other):
        m.release(rc)
    assert m.num_free == 16 and m.num_cached == 2
    m.check()


def test_reserving_for_a_whole_step_is_all_or_nothing():
    from atomserve_amd.cache.manager import CacheManager
    from atomserve_amd.parts.base import PagedCacheRequest, StateCacheRequest

    m = CacheManager({0: PagedCacheRequest(2, 16), 1: StateCacheRequest((4,))}, block_size=4, num_blocks=6, max_num_seqs=2)
    a, b, c = m.new_request(), m.new_request(), m.new_request()
    assert m.reserve_all([(a, 0, 9), (b, 0, 10)])  # 3 + 3 pages, both slots
    assert m.num_free == 0 and a.state_slot >= 0 and b.state_slot >= 0 and a.state_slot != b.state_slot
    assert m.reserve_all([(a, 9, 3), (b, 10, 2)])  # both fit in the pages they hold
    before = ([list(t) for t in a.tables], [list(t) for t in b.tables])
    assert not m.reserve_all([(a, 12, 1), (b, 12, 0)])  # a needs a fourth page: nobody gets anything
    assert ([list(t) for t in a.tables], [list(t) for t in b.tables]) == before
    m.release(b)
    assert not m.reserve_all([(a, 12, 1), (b, 0, 4), (c, 0, 1)])  # pages would do, slots would not
    assert m.num_free == 3 and b.state_slot < 0 and c.state_slot < 0
    assert m.reserve_all([(a, 12, 1), (b, 0, 4)])
    m.release(a)
    m.release(b)
    assert m.num_free == 6 and m.num_free_slots == 2
    m.check()


def test_pages_of_a_replay_pool():
    from atomserve_amd.engine.replay import pages_for

    assert pages_for(256, 16, 4) == 16 and pages_for(256, 8, 4) == 32 and pages_for(256, 64, 4) == 4
    # pages that do not divide 64: four requests of 64 tokens take two pages of 48 each
    assert pages_for(256, 48, 4) >= 8 and pages_for(256, 128, 4) >= 4
    assert pages_for(0, 16, 4) == 1
