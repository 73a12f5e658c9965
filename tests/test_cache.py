"""The cache manager without a GPU: no page lost, held twice or freed twice,
under random orders of requests; content sharing; windows; slots."""
import random

import pytest

from kipp_amd.cache import CacheManager, KVNeed, OutOfPages, OutOfSlots, PagePool, StateNeed, chain_hash

P = 4  # page size of the pool scenarios


def test_hash_is_chained_and_order_sensitive():
    # /root/reference/src/kipp_kv_pool.c:48-64: FNV-1a over parent bytes then token bytes
    h = 1469598103934665603
    for b in [0] * 8 + [1, 0, 0, 0]:
        h = ((h ^ b) * 1099511628211) & ((1 << 64) - 1)
    assert chain_hash(0, [1]) == h
    assert chain_hash(0, [1, 2]) != chain_hash(0, [2, 1]) and chain_hash(5, [1, 2]) != chain_hash(0, [1, 2])


def test_pool_alloc_release_lru_and_exhaustion():
    pool = PagePool(3, P)
    a, b, c = pool.alloc(), pool.alloc(), pool.alloc()
    assert sorted([a, b, c]) == [0, 1, 2] and pool.alloc() is None and pool.free_count == 0
    pool.release(b)
    pool.release(a)
    assert pool.alloc() == b and pool.alloc() == a       # least recently released first
    pool.release(c)
    with pytest.raises(ValueError):
        pool.release(c)                                   # freed twice
    pool.check()


def test_pool_seal_match_revive_evict():
    pool = PagePool(6, P)
    toks = list(range(100, 100 + 3 * P + 1))             # three full pages and one token
    pages, parent = [], 0
    for i in range(3):
        pg = pool.alloc()
        parent = pool.seal(pg, parent, toks[i * P:(i + 1) * P])
        pages.append(pg)
    with pytest.raises(ValueError):
        pool.seal(pages[0], 0, toks[:P])                  # sealed twice
    spare = pool.alloc()
    with pytest.raises(ValueError):
        pool.seal(spare, 0, toks[:P - 1])                 # only full pages
    pool.release(spare)
    with pytest.raises(ValueError):
        pool.seal(spare, 0, toks[:P])                     # not held
    got, _ = pool.prefix_match(toks)
    assert got == pages                                   # 3 pages + 1 token -> 3
    for pg in got:
        pool.release(pg)
    got, _ = pool.prefix_match(toks[:3 * P])
    assert got == pages[:2]                               # exactly 3 pages -> 2: one token is left to run
    for pg in got:
        pool.release(pg)
    assert pool.prefix_match(toks[:P])[0] == [] and pool.prefix_match([7] + toks[1:])[0] == []
    for pg in pages:
        pool.release(pg)                                  # free, but still indexed: revivable
    assert pool.free_count == 6
    got, _ = pool.prefix_match(toks)
    assert got == pages and pool.stats().reused_pages_total == 8
    for pg in got:
        pool.release(pg)
    # duplicate content keeps one indexed copy: the second page with the same tokens stays private
    dup = pool.alloc()
    assert dup not in pages                               # the never-sealed pages are older on the free list
    pool.seal(dup, 0, toks[:P])
    assert pool.content[dup] is None and pool.prefix_match(toks[:P + 1])[0] == [pages[0]]
    pool.release(pages[0])
    pool.release(dup)
    pool.check()
    # taking a free indexed page for new content evicts it from the index
    pool2 = PagePool(1, P)
    pg = pool2.alloc()
    pool2.seal(pg, 0, [1, 2, 3, 4])
    pool2.release(pg)
    assert pool2.alloc() == pg and pool2.stats().evicted_pages_total == 1
    pool2.release(pg)
    assert pool2.prefix_match([1, 2, 3, 4, 5])[0] == []


def test_pool_collisions_are_verified_by_tokens():
    pool = PagePool(4, P)
    pool.force_hash = 0x1234
    a, b = pool.alloc(), pool.alloc()
    pool.seal(a, 0, [1, 2, 3, 4])
    pool.seal(b, 0, [9, 9, 9, 9])
    assert pool.prefix_match([9, 9, 9, 9, 0])[0] == [b] and pool.prefix_match([1, 2, 3, 4, 0])[0] == [a]
    assert pool.prefix_match([5, 5, 5, 5, 0])[0] == []


def _manager(num_pages=12, window=None, states=False, share=True, max_requests=4):
    needs = [KVNeed(2, 16), KVNeed(2, 16), KVNeed(2, 16, window=window) if window else KVNeed(2, 16)]
    state_needs = [None, StateNeed((3, 5)) if states else None, None]
    return CacheManager(needs, state_needs, page_size=P, num_pages=num_pages, max_requests=max_requests,
                        max_position=64, runtime=None, share_prefixes=share)


def test_groups_are_formed_by_need():
    m = _manager(window=6)
    assert len(m.groups) == 2 and m.groups[0].runs == [0, 1] and m.groups[1].runs == [2]
    assert m.groups[0].bytes_per_token(2) == 2 * 2 * 2 * 16 * 2
    assert not m.share                                   # a window forbids content sharing
    assert _manager().share and not _manager(states=True).share
    assert m.view(2).group == 1 and m.view(1, reads_run=0).writable is False and m.view(0).writable


def test_a_fresh_pool_hands_out_scattered_pages():
    """Every page once, neighbours far apart: sequences of equal length that arrive together do not
    end up at equal distances in memory."""
    from kipp_amd.cache.pool import PagePool, scattered_order
    for n in (1, 2, 5, 64, 1000, 17028):
        order = scattered_order(n)
        assert sorted(order) == list(range(n))
        if n >= 64:
            assert min(abs(a - b) for a, b in zip(order, order[1:])) > n // 4
    pool = PagePool(10, 4)
    assert [pool.alloc() for _ in range(10)] == scattered_order(10) and pool.alloc() is None


def test_reserve_is_all_or_nothing():
    m = _manager(num_pages=5)
    a, b = m.open("a"), m.open("b")
    m.reserve([(a, 9)])                                   # 3 pages
    m.commit(a, list(range(9)))
    before = [list(t) for t in a.tables]
    assert len(before[0]) == 3 and len(set(before[0])) == 3
    with pytest.raises(OutOfPages):
        m.reserve([(a, 3), (b, 9)])                       # a: +0 (12 fits 3 pages), b: 3 > 2 free
    assert m.free_pages() == [2] and a.tables == before and b.tables == [[]]
    m.check()
    with pytest.raises(ValueError):
        m.reserve([(a, 0)])
    with pytest.raises(ValueError):
        m.reserve([(a, 60)])                              # beyond the model's positions
    m.close("a")
    m.close("b")
    assert m.free_pages() == [5]
    m.check()


def test_window_pages_are_given_back_when_passed():
    m = _manager(window=6, share=False)
    r = m.open("w")
    for n in (5, 3, 9, 1, 1, 1):
        m.reserve([(r, n)])
        m.commit(r, [1] * n)
        m.check()
        full, win = r.tables
        assert all(p >= 0 for p in full)
        first_needed = max(0, r.length - 6 + 1)           # the next query sees keys > length - window
        for block, page in enumerate(win):
            assert (page < 0) == ((block + 1) * P <= first_needed)
    assert m.free_pages()[1] > m.free_pages()[0]
    m.close("w")
    assert m.free_pages() == [12, 12]


def test_prefix_adoption_through_the_manager():
    m = _manager()
    toks = list(range(30))
    a = m.open("a", toks)
    assert a.length == 0
    m.reserve([(a, 30)])
    m.commit(a, toks)
    m.close("a")                                          # publishes 7 full pages
    b = m.open("b", toks[:17] + [99, 98])
    assert b.length == 16 and b.adopted == [4] and b.tokens == toks[:16]
    m.reserve([(b, 3)])
    m.commit(b, toks[16:17] + [99, 98])
    c = m.open("c", toks[:8])                             # exactly two pages known: one is adopted
    assert c.length == 4
    m.check()
    m.close("b")
    m.close("c")
    assert m.free_pages() == [12] and m.groups[0].pool.stats().reused_pages_total == 5
    m.check()


def test_truncate_gives_back_the_pages_above_and_never_the_adopted_ones():
    # /root/reference/src/kipp.c:3739-3774: only the private tail is released
    m = _manager()
    toks = list(range(30))
    a = m.open("a")
    m.reserve([(a, 30)])
    m.commit(a, toks)
    assert m.free_pages() == [4]
    m.truncate(a, 9)                                      # into the third page
    assert a.length == 9 and a.tokens == toks[:9] and len([p for p in a.tables[0] if p >= 0]) == 3
    assert m.free_pages() == [9]
    m.check()
    m.reserve([(a, 8)])
    m.commit(a, toks[9:17])
    m.close("a")                                          # publishes four full pages of the new timeline
    b = m.open("b", toks)
    assert b.length == 16
    with pytest.raises(ValueError):
        m.truncate(b, 12)                                 # adopted pages are shared
    with pytest.raises(ValueError):
        m.truncate(b, 17)
    m.truncate(b, 16)
    m.close("b")
    assert m.free_pages() == [12]
    m.check()
    for other in (_manager(window=6, share=False), _manager(states=True)):
        r = other.open("r")
        with pytest.raises(NotImplementedError):
            other.truncate(r, 0)


def test_early_publication_lets_a_neighbour_adopt_pages_of_a_running_request():
    m = _manager()
    toks = list(range(30))
    a = m.open("a", toks, publish_early=True)
    m.reserve([(a, 9)])
    m.commit(a, toks[:9])                                 # two full pages are published at once
    b = m.open("b", toks, publish_early=True)
    assert b.length == 8 and b.tables[0] == a.tables[0][:2]
    with pytest.raises(ValueError):
        m.truncate(a, 7)                                  # published pages can no longer be cut
    m.truncate(a, 8)
    m.reserve([(a, 5), (b, 5)])                           # both compute the fourth page themselves
    m.commit(a, toks[8:13])
    m.commit(b, toks[8:13])
    assert a.published == 3 and b.published == 3 and a.tables[0][2] != b.tables[0][2]
    m.check()
    c = m.open("c", toks)
    assert c.length == 12 and c.tables[0][2] == a.tables[0][2]   # the first of the two copies is the indexed one
    for r in "abc":
        m.close(r)
    assert m.free_pages() == [12]
    m.check()
    d = m.open("d", toks)                                 # published pages outlive their requests
    assert d.length == 12
    m.close("d")


def test_slots():
    m = _manager(states=True, max_requests=2)
    a, b = m.open("a"), m.open("b")
    assert {a.slot, b.slot} == {0, 1}
    with pytest.raises(OutOfSlots):
        m.open("c")
    with pytest.raises(ValueError):
        m.open("a")
    m.close("a")
    assert m.open("c").slot == a.slot
    m.check()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_lose_nothing(seed):
    rng = random.Random(seed)
    window = rng.choice([None, 5, 9])
    m = _manager(num_pages=rng.randint(6, 14), window=window, share=window is None, max_requests=4)
    live = {}
    next_id = 0
    for _ in range(400):
        action = rng.random()
        if action < 0.25 and len(live) < 4:
            prompt = [rng.randrange(3) for _ in range(rng.randint(1, 20))]
            live[next_id] = m.open(next_id, prompt if rng.random() < 0.7 else None)
            next_id += 1
        elif action < 0.85 and live:
            chosen = rng.sample(sorted(live), rng.randint(1, len(live)))
            entries = [(live[i], rng.randint(1, 7)) for i in chosen]
            entries = [(r, n) for r, n in entries if r.length + n <= 64]
            before = m.free_pages()
            try:
                if entries:
                    m.reserve(entries)
                    for r, n in entries:
                        m.commit(r, [rng.randrange(3) for _ in range(n)])
            except OutOfPages:
                assert m.free_pages() == before           # nothing changed
        elif live:
            rid = rng.choice(sorted(live))
            m.close(rid)
            del live[rid]
        m.check()
    for rid in list(live):
        m.close(rid)
    m.check()
    assert m.free_pages() == [g.pool.num_pages for g in m.groups] and len(m.free_slots) == 4


def test_groups_with_page_sizes_and_pool_sizes_of_their_own():
    """Two groups that differ in both: runs that keep every key in pages of 4 tokens, 10 of them, and a run with a
    window of 6 that asks for pages of 2 tokens and gets a pool of 7.  Each group's tables, claims and returns go
    by its own page size; content sharing is off (a page does not hold the same tokens in both)."""
    needs = [KVNeed(2, 16), KVNeed(1, 32, window=6, page_size=2), KVNeed(2, 16)]
    m = CacheManager(needs, [None, None, None], page_size=4, num_pages=[10, 7], max_requests=3, max_position=40, runtime=None)
    full, win = m.groups
    assert (full.page_size, full.pool.num_pages, full.runs) == (4, 10, [0, 2])
    assert (win.page_size, win.pool.num_pages, win.runs) == (2, 7, [1])
    assert not m.share and m.view(1).page_size == 2 and m.view(2).page_size == 4
    # one number for every group: the same tokens in each pool
    same = CacheManager(needs, [None, None, None], page_size=4, num_pages=10, max_requests=3, max_position=40, runtime=None)
    assert [g.pool.num_pages for g in same.groups] == [10, 20]
    r = m.open("r")
    assert [len(row) for row in r.rows] == [10, 20]
    for n in (5, 4, 1, 1, 6):
        m.reserve([(r, n)])
        m.commit(r, [1] * n)
        m.check()
        assert len(r.tables[0]) == -(-r.length // 4) and len(r.tables[1]) == -(-r.length // 2)
        first_needed = max(0, r.length - 6 + 1)
        assert all((page < 0) == ((block + 1) * 2 <= first_needed) for block, page in enumerate(r.tables[1]))
        assert all(page >= 0 for page in r.tables[0])
    # 17 tokens: 5 pages of 4; of the 9 pages of 2 the window keeps those from position 12 on
    assert m.free_pages() == [10 - 5, 7 - 3]
    # what a scheduler must keep free for it up to 40 tokens in steps of at most 4: every block of the first group,
    # and in the windowed one the distance to the most it ever holds, the pages of 6 - 1 + 4 tokens and one more
    assert m.pages_bound(r, 40, 4) == [10 - 5, 6 - 3]
    assert m.pages_bound(None, 40, 4) == [10, 6]
    with pytest.raises(OutOfPages):
        m.reserve([(r, 23)])                       # 40 tokens: 20 pages of 2, 12 of them beyond what it has, 4 free
    assert m.free_pages() == [5, 4]
    m.close("r")
    assert m.free_pages() == [10, 7]
    m.check()
