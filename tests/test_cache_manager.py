"""The cache manager without a GPU: the page pool's order and errors, and the manager's books under
random orders of requests (no page lost, held twice or freed twice), windows, groups and state slots."""
import random

import pytest
import torch

from geneinfer_amd.cache import CacheError, CacheManager, OutOfPages, PagedKvNeed, PageError, PagePool, StateNeed


def test_pool_hands_out_page_0_first_and_the_last_freed_next():          # src/model/kv_cache.cpp:22-56, tests/verify_kvpool.py:24-45
    pool = PagePool(4)
    assert [pool.allocate() for _ in range(3)] == [0, 1, 2]
    pool.release(1)
    pool.release(0)
    assert pool.allocate() == 0 and pool.allocate() == 1 and pool.allocate() == 3
    with pytest.raises(OutOfPages):
        pool.allocate()
    assert pool.free_count == 0


def test_pool_hands_out_many_pages_in_the_order_of_single_ones():
    a, b = PagePool(9), PagePool(9)
    for pool in (a, b):
        held = [pool.allocate() for _ in range(5)]
        for p in (held[1], held[3], held[0]):
            pool.release(p)
    assert a.allocate_many(4) == [b.allocate() for _ in range(4)] and a.free_count == b.free_count == 3
    assert all(a.ref_count(p) == b.ref_count(p) for p in range(9))
    with pytest.raises(OutOfPages):
        a.allocate_many(4)
    assert a.free_count == 3 and a.allocate_many(0) == [] and len(a.allocate_many(3)) == 3 and a.free_count == 0


def test_pool_misuse_raises():
    pool = PagePool(2)
    p = pool.allocate()
    pool.retain(p)
    pool.release(p)
    assert pool.ref_count(p) == 1 and pool.free_count == 1
    pool.release(p)
    with pytest.raises(PageError, match="already free"):
        pool.release(p)
    with pytest.raises(PageError, match="cannot be retained"):
        pool.retain(p)
    with pytest.raises(PageError, match="does not exist"):
        pool.release(5)


FULL = PagedKvNeed(2, 16)
WINDOW = PagedKvNeed(2, 16, window=10)


def manager(needs, reads=None, n_pages=12, page_size=4, max_requests=4, max_positions=64):
    return CacheManager(needs, reads or [None] * len(needs), page_size=page_size, n_pages=n_pages, max_requests=max_requests,
                        max_positions=max_positions, allocate_storage=False)


def test_layers_with_equal_needs_share_a_group():
    m = manager([FULL, WINDOW, FULL, None, StateNeed((3,)), WINDOW], [None, None, None, None, None, 1])
    assert len(m.groups) == 2
    assert m.groups[0].entries == [0, 2] and m.groups[1].entries == [1]       # entry 5 reads entry 1's pages
    assert m._entry_group[5] == m._entry_group[1]
    with pytest.raises(CacheError, match="whose need differs"):
        manager([FULL, WINDOW], [None, 0])


def test_reserve_is_all_or_nothing():
    m = manager([FULL], n_pages=5)
    m.open("a"); m.open("b")
    m.reserve([("a", 9)])                                                      # 3 pages
    m.advance("a", 9)
    before = (m.free_pages(), list(m.groups[0].table_host[m.slot("b")]))
    with pytest.raises(OutOfPages):
        m.reserve([("a", 4), ("b", 5)])                                        # 1 + 2 pages > 2 free
    assert (m.free_pages(), list(m.groups[0].table_host[m.slot("b")])) == before
    m.reserve([("a", 3), ("b", 5)])                                            # 0 + 2 pages
    m.check_consistency()
    assert m.free_pages() == [0]


def test_positions_map_to_pages_and_close_gives_everything_back():
    m = manager([FULL], n_pages=6)
    m.open("a")
    m.reserve([("a", 5)]); m.advance("a", 5)
    m.reserve([("a", 4)]); m.advance("a", 4)
    g = m.groups[0]
    assert g.held_pages(m.slot("a")) == [0, 1, 2] and m.length("a") == 9
    m.open("b")
    m.reserve([("b", 1)]); m.advance("b", 1)
    m.close("a")
    assert m.free_pages() == [5]
    m.open("c")
    m.reserve([("c", 8)])
    assert g.held_pages(m.slot("c")) == [0, 1]                                 # the pages freed last are used again first
    m.check_consistency()


def test_window_pages_are_given_back_as_the_request_moves_on():
    m = manager([WINDOW], n_pages=5, page_size=4)                              # window 10: at most ceil((10 + 3) / 4) + 1 pages live
    m.open("a")
    g, slot = m.groups[0], None
    for step in range(40):
        m.reserve([("a", 1)])
        m.advance("a", 1)
        slot = m.slot("a")
        length = m.length("a")
        live = g.held_pages(slot)
        first_visible = max(0, length - 10 + 1)                                # what the next row still sees
        assert int(g.first_live[slot]) == first_visible // 4
        assert all(p >= 0 for p in live) and len(live) <= 4
        m.check_consistency()
    assert m.length("a") == 40                                                 # longer than the pool (5 pages = 20 positions) could hold whole


def test_a_chunk_keeps_the_pages_its_first_row_sees():
    m = manager([WINDOW], n_pages=8, page_size=4)
    m.open("a")
    m.reserve([("a", 13)]); m.advance("a", 13)                                 # next row at 13 sees 4..13: page 0 is gone
    g, slot = m.groups[0], m.slot("a")
    assert int(g.first_live[slot]) == 1
    m.reserve([("a", 9)])                                                      # rows 13..21; row 13 still needs page 1
    assert int(g.first_live[slot]) == 1 and g.table_host[slot, 1] >= 0
    m.advance("a", 9)                                                          # next row at 22 sees 13..22: pages 0..2 gone
    assert int(g.first_live[slot]) == 3


def test_limits_and_misuse():
    m = manager([FULL], max_requests=2, max_positions=10)
    m.open("a"); m.open("b")
    with pytest.raises(CacheError, match="already open"):
        m.open("a")
    with pytest.raises(CacheError, match="request slots are in use"):
        m.open("c")
    with pytest.raises(CacheError, match="not open"):
        m.length("zzz")
    with pytest.raises(CacheError, match="beyond the limit 10"):
        m.reserve([("a", 11)])
    with pytest.raises(CacheError, match="named twice"):
        m.reserve([("a", 1), ("a", 1)])
    with pytest.raises(CacheError, match="beyond its reserved pages"):
        m.advance("a", 1)
    m.reserve([("a", 10)]); m.advance("a", 10)                                 # the exact last position is allowed
    m.close("a"); m.open("c")
    assert m.slot("c") == 0                                                    # the slot freed last is used again


def test_state_slots_are_zeroed_when_a_request_opens():
    m = CacheManager([StateNeed((2, 3)), FULL], [None, None], page_size=4, n_pages=4, max_requests=2, max_positions=16, device="cpu")
    assert m.state(0).shape == (3, 2, 3)                                       # two request slots and the spare one
    s = m.open("a")
    m.state(0)[s] += 5.0
    m.close("a")
    assert m.open("b") == s and float(m.state(0)[s].abs().sum()) == 0.0
    kv, table, window = m.kv(1)
    assert kv.shape == (5, 2, 2, 4, 16) and table.shape == (3, 4) and window is None      # the pool's pages and request slots, and the spare ones


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_of_requests_keep_the_books(seed):
    rng = random.Random(seed)
    needs = [FULL, WINDOW, FULL] if seed % 2 else [FULL]
    m = manager(needs, n_pages=rng.choice([6, 9, 14]), page_size=rng.choice([1, 3, 4]), max_requests=3, max_positions=40)
    live, counter, refused = {}, 0, 0
    for _ in range(400):
        action = rng.random()
        if action < 0.2 and len(live) < 3:
            counter += 1
            m.open(counter)
            live[counter] = 0
        elif action < 0.3 and live:
            rid = rng.choice(list(live))
            m.close(rid)
            del live[rid]
        elif action < 0.4 and live:                                            # a rewind, where the cache can do one
            rid = rng.choice(list(live))
            to = rng.randint(0, live[rid])
            try:
                m.truncate(rid, to)
                live[rid] = to
            except CacheError as e:
                assert "window" in str(e) and len(needs) == 3 and m.length(rid) == live[rid]
        elif live:
            batch = rng.sample(list(live), rng.randint(1, len(live)))
            adds = [(rid, rng.randint(1, 7)) for rid in batch if live[rid] < 33]
            if not adds:
                continue
            before = m.free_pages()
            try:
                m.reserve(adds)
            except OutOfPages:
                refused += 1
                assert m.free_pages() == before                                # a refused reservation changes nothing
                victim = max(live, key=live.get)
                m.close(victim)
                del live[victim]
                continue
            for rid, n in adds:
                m.advance(rid, n)
                live[rid] += n
                assert m.length(rid) == live[rid]
        m.check_consistency()
    for rid in list(live):
        m.close(rid)
    m.check_consistency()
    assert all(f == g.pool.n_pages for f, g in zip(m.free_pages(), m.groups))
    assert refused > 0                                                         # the pool did run out: the refusals above were exercised


@pytest.mark.parametrize("seed", range(4))
def test_one_position_for_each_is_the_same_as_the_general_path(seed):
    """reserve_one_each / advance_one_each against reserve / advance on a twin manager."""
    rng = random.Random(seed)
    needs = [FULL, WINDOW] if seed % 2 else [FULL]
    a, b = (manager(needs, n_pages=10, page_size=4, max_requests=4, max_positions=40) for _ in range(2))
    live = []
    for step in range(120):
        first = rng.randint(1, 6)
        if len(live) < 4 and rng.random() < 0.2 and min(a.free_pages()) >= 2:
            rid = f"r{step}"
            for m in (a, b):
                m.open(rid)
                m.reserve([(rid, first)]); m.advance(rid, first)
            live.append(rid)
        if live and rng.random() < 0.1:
            rid = live.pop(rng.randrange(len(live)))
            a.close(rid); b.close(rid)
        batch = [r for r in live if rng.random() < 0.8 and a.length(r) < 39]
        if not batch:
            continue
        slots, lengths = [a.slot(r) for r in batch], [a.length(r) for r in batch]
        try:
            a.reserve([(r, 1) for r in batch])
            general_ok = True
        except OutOfPages:
            general_ok = False
        if general_ok:
            b.reserve_one_each(batch, slots, lengths)
            for r in batch:
                a.advance(r, 1)
            b.advance_one_each(batch, slots, lengths)
        else:
            with pytest.raises(OutOfPages):
                b.reserve_one_each(batch, slots, lengths)
            victim = live.pop(0)
            a.close(victim); b.close(victim)
        for ga, gb in zip(a.groups, b.groups):
            assert (ga.table_host == gb.table_host).all() and ga.pool.free_count == gb.pool.free_count
        assert all(a.length(r) == b.length(r) for r in live)
        b.check_consistency()


# ------------------------------------------------------------------------------- prefix sharing
def test_prefix_index_matches_true_prefixes_of_full_pages_only():                 # src/model/prefix_cache.h:1-11
    from geneinfer_amd.cache import PagePool, PrefixIndex
    pool = PagePool(12)
    index = PrefixIndex(pool, page_size=4)
    tokens = list(range(100, 114))                                                # 3 full pages and 2 tokens
    pages = [pool.allocate() for _ in range(4)]
    assert index.insert(tokens, 14, pages) == 3 and len(index) == 3                # the partly filled page is not named
    assert [pool.ref_count(p) for p in pages] == [2, 2, 2, 1]
    assert index.insert(tokens, 14, pages) == 0                                    # known links are followed, not named again
    found = index.match(tokens, 14)
    assert found == pages[:3] and [pool.ref_count(p) for p in pages[:3]] == [3, 3, 3]      # retained for the caller
    for p in found:
        pool.release(p)
    assert index.match(tokens, 11) == pages[:2] and index.match(tokens, 3) == []   # the limit counts whole pages
    for p in pages[:2]:
        pool.release(p)
    other = tokens[:4] + [7, 7, 7, 7] + tokens[8:]                                 # equal first page, then another, then an equal third
    assert index.match(other, 14) == pages[:1]                                     # the third page is no prefix of this
    pool.release(pages[0])
    assert index.match(tokens[4:], 10) == []                                       # the same tokens elsewhere in a prompt do not match
    # another request computed the same first page itself, then went on differently: its copy is not named, its second page is
    own = [pool.allocate() for _ in range(2)]
    assert index.insert(other, 8, own) == 1 and own[0] not in index and own[1] in index
    assert index.match(other, 8) == [pages[0], own[1]]


def test_prefix_index_goes_on_where_a_request_was_inserted_last():
    """A request that grows is inserted again and again; with the place its last walk ended at, the new walk passes only
    the new pages.  If that place has been given back and its page named anew under another chain, the walk starts over."""
    from geneinfer_amd.cache import PagePool, PrefixIndex
    pool = PagePool(12)
    index = PrefixIndex(pool, page_size=2)
    tokens = [1, 1, 2, 2, 3, 3, 4, 4]
    pages = [pool.allocate() for _ in range(4)]
    assert index.insert(tokens, 4, pages) == 2
    place = index.last_walk
    assert place[1] == 2 and place[0].page == pages[1]
    lookups = []
    real = index._children_of
    index._children_of = lambda node: lookups.append(node) or real(node)
    assert index.insert(tokens, 8, pages, after=place) == 2 and len(index) == 4
    assert all(node is not None for node in lookups)                                  # the root was not visited again
    index._children_of = real
    assert index.match(tokens, 8) == pages
    for p in pages * 2:
        pool.release(p)                                                            # the request and the match let go
    assert index.evict(4) == 4 and len(index) == 0
    # the page comes back under other tokens; the stale place is recognised
    other = [pool.allocate() for _ in range(2)]
    assert pages[1] in other
    index.insert([7, 7, 8, 8], 4, other)
    again = [pool.allocate() for _ in range(4)]
    assert index.insert(tokens, 8, again, after=place) == 4
    assert index.match(tokens, 8) == again and index.match([7, 7, 8, 8, 3, 3], 6) == other


def test_prefix_index_gives_back_least_recently_used_leaves_that_nobody_uses():    # src/model/prefix_cache.cpp:60-97
    from geneinfer_amd.cache import PagePool, PrefixIndex
    pool = PagePool(10)
    index = PrefixIndex(pool, page_size=2)
    a = [pool.allocate() for _ in range(3)]
    b = [pool.allocate() for _ in range(2)]
    index.insert([1, 1, 2, 2, 3, 3], 6, a)
    index.insert([9, 9, 8, 8], 4, b)
    assert index.evictable() == 0 and index.evict(5) == 0                          # everything is still used by its request
    for p in a + b:
        pool.release(p)                                                            # the requests end
    assert index.evictable() == 5 and pool.free_count == 5
    held = index.match([1, 1, 2, 2], 4)                                            # a request uses a's first two pages (and touches them)
    assert held == a[:2] and index.evictable() == 3
    assert index.evict(1) == 1 and a[2] not in index and b[1] in index             # a's leaf was used before b's
    assert index.evict(10) == 2 and len(index) == 2 and pool.free_count == 8       # b's leaf, then b's root; the used pages stay
    assert [pool.ref_count(p) for p in held] == [2, 2]
    for p in held:
        pool.release(p)
    index.clear()
    assert pool.free_count == 10 and len(index) == 0


def test_prefix_index_forgets_a_used_leaf_to_reach_an_unused_page_above():
    from geneinfer_amd.cache import PagePool, PrefixIndex
    pool = PagePool(4)
    index = PrefixIndex(pool, page_size=1)
    chain = [pool.allocate() for _ in range(3)]
    index.insert([5, 6, 7], 3, chain)
    pool.release(chain[0]); pool.release(chain[1])                                 # only the last page is still used by someone
    assert index.evictable() == 2
    assert index.evict(2) == 2 and len(index) == 0                                 # the used leaf is forgotten, then the two above go
    assert pool.ref_count(chain[2]) == 1 and pool.free_count == 3


def test_requests_open_on_shared_pages():
    m = manager([FULL], n_pages=8, page_size=4, max_requests=3, max_positions=32)
    assert m.enable_prefix_sharing() and m.prefix is not None
    m.open("a")
    m.reserve([("a", 10)]); m.advance("a", 10)
    tokens = list(range(10))
    assert m.prefix.insert(tokens, 10, m.pages_of("a")) == 2
    shared = m.prefix.match(tokens + [77], 10)
    m.open("b", shared)
    assert m.length("b") == 8 and m.pages_of("b") == m.pages_of("a")[:2]
    m.check_consistency()
    m.reserve([("b", 3)]); m.advance("b", 3)
    assert m.pages_of("b")[2] not in m.pages_of("a")                              # what b writes goes to a page of its own
    m.close("a")
    m.check_consistency()
    assert m.free_pages() == [8 - 3] and m.evictable_pages() == 0                  # a's third page is free, the shared two serve b
    m.close("b")
    assert m.free_pages() == [6] and m.evictable_pages() == 2 and m.evict(5) == 2 and m.free_pages() == [8]
    m.check_consistency()
    with pytest.raises(CacheError, match="already open|shared"):
        m2 = manager([FULL], n_pages=4, page_size=4, max_requests=2, max_positions=16)
        m2.open("x", [0])


def test_requests_open_on_shared_pages_of_every_group():
    """Two groups of pages without a window (other head counts): the index names the first group's pages and keeps the other
    group's beside them; a request that opens on a match holds both, and a page given back is one of each group."""
    other = PagedKvNeed(1, 32)
    m = manager([FULL, other, FULL], n_pages=8, page_size=4, max_requests=3, max_positions=32)
    assert len(m.groups) == 2 and m.enable_prefix_sharing()
    m.groups[1].pool._free.reverse()                                              # (so that the two groups hand out other page numbers)
    m.open("a")
    m.reserve([("a", 10)]); m.advance("a", 10)
    tokens = list(range(10))
    a0, a1 = [g.held_pages(m.slot("a")) for g in m.groups]
    assert a0 != a1
    assert m.index_prefix("a", tokens, 10) == 2
    m.open("b", m.prefix.match(tokens + [77], 10))
    assert m.length("b") == 8 and [g.held_pages(m.slot("b")) for g in m.groups] == [a0[:2], a1[:2]]
    m.check_consistency()
    m.reserve([("b", 3)]); m.advance("b", 3)
    m.close("a")
    m.check_consistency()
    assert m.free_pages() == [5, 5] and m.evictable_pages() == 0
    m.close("b")
    assert m.free_pages() == [6, 6] and m.available_pages() == [8, 8] and m.evictable_pages() == 2
    m.open("c")
    m.reserve([("c", 30)])                                                          # needs all 8 pages of both groups: the index gives its two back
    assert m.free_pages() == [0, 0] and len(m.prefix) == 0
    m.close("c")
    m.check_consistency()
    assert m.free_pages() == [8, 8]


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_shared_prefixes_over_two_groups_keep_the_books_under_random_use(seed):
    """Requests over a small alphabet open on matched pages of two groups, grow, name their pages, are cut back and end, in
    random order, on a pool so small that the index has to give pages back: after every action no page of either group is
    lost, held twice without the index knowing, or counted wrongly, and both groups hold the same number of pages."""
    import random
    rng = random.Random(seed)
    m = manager([FULL, PagedKvNeed(1, 32)], n_pages=14, page_size=2, max_requests=4, max_positions=24)
    assert m.enable_prefix_sharing()
    m.groups[1].pool._free.reverse()
    live, walks = {}, {}
    for turn in range(500):
        roll = rng.random()
        if roll < 0.35 and len(live) < 4:
            tokens = [rng.randrange(2) for _ in range(rng.choice([3, 4, 6, 9, 12]))]
            shared = m.prefix.match(tokens, len(tokens) - 1)
            m.open(turn, shared)
            live[turn], walks[turn] = tokens, None
        elif roll < 0.7 and live:
            r = rng.choice(list(live))
            n = min(rng.randint(1, 4), len(live[r]) - m.length(r))
            if n > 0:
                try:
                    m.reserve([(r, n)])
                except OutOfPages:
                    continue
                m.advance(r, n)
                m.index_prefix(r, live[r], m.length(r), after=walks[r])
                walks[r] = m.prefix.last_walk
        elif roll < 0.8 and live:
            r = rng.choice(list(live))
            if m.length(r) > 0:
                try:
                    m.truncate(r, rng.randrange(m.length(r)))
                except OutOfPages:
                    pass
                walks[r] = None
        elif live:
            r = rng.choice(list(live))
            m.close(r)
            del live[r], walks[r]
        m.check_consistency()
        free = m.free_pages()
        assert free[0] == free[1] and m.available_pages() == [free[0] + m.evictable_pages()] * 2
    for r in list(live):
        m.close(r)
    m.prefix.clear()
    m.check_consistency()
    assert m.free_pages() == [14, 14]


def test_prefix_sharing_needs_pages_without_window_or_state():
    assert not manager([FULL, WINDOW], n_pages=8, page_size=4, max_requests=2, max_positions=32).enable_prefix_sharing()
    assert not manager([WINDOW], n_pages=8, page_size=4, max_requests=2, max_positions=32).enable_prefix_sharing()
    from geneinfer_amd.cache import StateNeed
    assert not manager([FULL, StateNeed((3,), torch.float32)], n_pages=8, page_size=4, max_requests=2, max_positions=32).enable_prefix_sharing()


def test_rewind_gives_pages_back_and_goes_on_from_there():                        # src/model/kv_cache.cpp:100-109
    m = manager([FULL], n_pages=6, page_size=4)
    m.open("a")
    m.reserve([("a", 14)]); m.advance("a", 14)                                    # pages 0..3
    pages = m.pages_of("a")
    m.truncate("a", 14)                                                           # nothing to do
    assert m.pages_of("a") == pages
    m.truncate("a", 6)
    assert m.length("a") == 6 and m.pages_of("a") == pages[:2] and m.free_pages() == [4]
    m.check_consistency()
    m.reserve([("a", 3)]); m.advance("a", 3)                                      # positions 6, 7 in the kept page, 8 in a new one
    assert m.pages_of("a") == pages[:2] + [pages[2]]                              # the page freed last comes back first
    m.truncate("a", 8)                                                            # exactly at a page's edge: the page after it goes
    assert m.pages_of("a") == pages[:2]
    m.truncate("a", 0)
    assert m.length("a") == 0 and m.pages_of("a") == [] and m.free_pages() == [6]
    m.reserve([("a", 1)]); m.advance("a", 1)
    m.check_consistency()
    with pytest.raises(CacheError, match="cannot be cut"):
        m.truncate("a", 2)
    with pytest.raises(CacheError, match="cannot be cut"):
        m.truncate("a", -1)
    with pytest.raises(CacheError, match="not open"):
        m.truncate("b", 0)


def test_rewind_into_a_shared_page_copies_it_first():                             # src/model/kv_cache.cpp:116-141
    m = CacheManager([FULL, FULL], [None, None], page_size=4, n_pages=5, max_requests=3, max_positions=32, dtype=torch.float32)
    assert m.enable_prefix_sharing()
    g = m.groups[0]
    m.open("a")
    m.reserve([("a", 8)]); m.advance("a", 8)
    first, second = m.pages_of("a")
    g.storage[:, second] = torch.arange(g.storage[:, second].numel(), dtype=torch.float32).reshape(g.storage[:, second].shape)
    tokens = list(range(8))
    m.prefix.insert(tokens, 8, m.pages_of("a"))
    m.open("b", m.prefix.match(tokens + [9], 8))                                  # b shares both pages
    m.truncate("b", 6)                                                            # b will write position 6: inside the second page
    mine = m.pages_of("b")
    assert mine[0] == first and mine[1] != second and m.pages_of("a") == [first, second]
    assert torch.equal(g.storage[:, mine[1]], g.storage[:, second])               # every layer, keys and values
    m.check_consistency()
    g.storage[:, mine[1], :, :, 2:] = -1.0                                        # what b writes from position 6 on
    assert (g.storage[:, second] >= 0).all()                                      # a and the index still see their own
    m.truncate("b", 5)                                                            # its own page now: no second copy
    assert m.pages_of("b") == mine
    m.truncate("b", 4)                                                            # at the edge: the copy goes, the shared first page stays
    assert m.pages_of("b") == [first] and m.free_pages() == [3]
    # no page to copy into: refused with nothing changed
    m.open("c")
    m.reserve([("c", 9)]); m.advance("c", 9)                                      # the 3 free pages
    with pytest.raises(OutOfPages):
        m.truncate("b", 2)
    assert m.length("b") == 4 and m.pages_of("b") == [first]
    m.close("c")
    m.truncate("b", 2)                                                            # the first page is shared as well
    assert m.pages_of("b")[0] != first and m.length("b") == 2
    m.check_consistency()
    for r in ("a", "b"):
        m.close(r)
    m.prefix.clear()
    m.check_consistency()
    assert m.free_pages() == [5]


def test_rewind_is_refused_where_the_past_is_gone():
    m = manager([WINDOW], n_pages=6, page_size=4)                                 # window 10
    m.open("a")
    for _ in range(30):
        m.reserve([("a", 1)]); m.advance("a", 1)                                  # the next row sees 21..: pages 0..4 were given back
    assert int(m.groups[0].first_live[m.slot("a")]) == 5
    before = (m.pages_of("a"), m.free_pages())
    with pytest.raises(CacheError, match="window of 10"):
        m.truncate("a", 20)                                                       # would need positions 11..19
    assert (m.pages_of("a"), m.free_pages(), m.length("a")) == (*before, 30)
    m.truncate("a", 29)                                                           # sees 20..28: page 5 on, all held
    assert m.length("a") == 29
    m.truncate("a", 0)                                                            # a fresh start needs nothing
    assert m.free_pages() == [6] and int(m.groups[0].first_live[m.slot("a")]) == 0
    s = manager([FULL, StateNeed((3,))])
    s.open("a")
    s.reserve([("a", 5)]); s.advance("a", 5)
    with pytest.raises(CacheError, match="fixed-size state"):
        s.truncate("a", 2)


def test_prefix_index_counts_hold_under_random_use():
    """Random requests over a small alphabet (so that beginnings repeat) open on matched pages, fill pages, name them, end;
    now and then pages are taken back.  At every point the index's constant-time count equals a recount, every page it
    names has a place under its parent, `evict(k)` gives back min(k, evictable) pages, and at the end nothing is lost."""
    import random
    from geneinfer_amd.cache import PagePool, PrefixIndex
    rng = random.Random(3)
    pool = PagePool(40)
    index = PrefixIndex(pool, page_size=2)
    live = {}                                                                      # request -> (tokens, pages it holds)
    for turn in range(600):
        roll = rng.random()
        if roll < 0.45 and len(live) < 5:
            tokens = [rng.randrange(3) for _ in range(rng.choice([2, 4, 5, 8, 12]))]
            pages = index.match(tokens, len(tokens) - 1)
            need = -(-len(tokens) // 2) - len(pages)
            if need > pool.free_count:
                short, could = need - pool.free_count, recount(index, pool)
                assert index.evict(short) == min(short, could)
            if need > pool.free_count:
                for p in pages:
                    pool.release(p)
                continue
            pages += [pool.allocate() for _ in range(need)]
            index.insert(tokens, len(tokens), pages)
            live[turn] = (tokens, pages)
        elif roll < 0.85 and live:
            _, pages = live.pop(rng.choice(list(live)))
            for p in reversed(pages):
                pool.release(p)
        else:
            k, before, could = rng.randint(1, 6), pool.free_count, recount(index, pool)
            assert index.evict(k) == min(k, could) == pool.free_count - before
        assert index.evictable() == recount(index, pool)
        assert pool.free_count + len(set(p for _, pages in live.values() for p in pages) | set(index.pages())) == pool.n_pages
        for page in index.pages():
            node = index._by_page[page]
            assert index._children_of(node.parent)[node.tokens] is node and pool.ref_count(page) >= 1
    for _, pages in live.values():
        for p in pages:
            pool.release(p)
    assert index.evictable() == len(index)
    named, free = len(index), pool.free_count
    assert index.evict(named // 2) == named // 2 and pool.free_count == free + named // 2
    index.clear()
    assert pool.free_count == pool.n_pages and len(index) == 0


def recount(index, pool):
    return sum(1 for page in index.pages() if pool.ref_count(page) == 1)


def test_the_device_copy_of_the_tables_follows_under_random_use_with_few_columns_sent():
    """Requests open, grow by portions and single positions, are cut back, slide a window and end, with a sync now and
    then (not after every change): after each sync the device's tables equal the host's, and a request that only
    crossed into a new page sent one column, not its row."""
    rng = random.Random(11)
    m = CacheManager([FULL, WINDOW], [None, None], page_size=4, n_pages=60, max_requests=4, max_positions=120, dtype=torch.float32, device="cpu")
    sent = []
    def upload(rows, block):
        sent.append(block.size)
        return torch.from_numpy(rows.copy().reshape(-1)), torch.from_numpy(block.copy().reshape(-1))
    live = []
    for turn in range(500):
        roll = rng.random()
        if roll < 0.15 and len(live) < 4:
            live.append(f"r{turn}")
            m.open(live[-1])
        elif roll < 0.75 and live:
            r = rng.choice(live)
            n = rng.choice([1, 1, 1, 2, 7, 19])
            if m.length(r) + n <= 120 and m.fits([(r, n)]):
                m.reserve([(r, n)]); m.advance(r, n)
        elif roll < 0.85 and live:
            r = rng.choice(live)
            try:
                m.truncate(r, rng.randrange(m.length(r) + 1))
            except CacheError:
                pass                                                              # behind the window: refused
        elif roll < 0.93 and live:
            m.close(live.pop(rng.randrange(len(live))))
        if rng.random() < 0.6:
            m.sync(upload if rng.random() < 0.5 else None)
            for g in m.groups:
                assert (g.table_dev.numpy() == g.table_host).all(), turn
    m.check_consistency()
    # one request alone, position by position: a new page sends the row's number and one entry (with a window, also
    # the entries between the page given back and the new one), never the row of 30 entries
    for r in live:
        m.close(r)
    m.sync(upload)
    m.open("solo")
    m.reserve([("solo", 50)]); m.advance("solo", 50)
    m.sync(upload)
    del sent[:]
    for _ in range(8):
        m.reserve([("solo", 1)]); m.advance("solo", 1)
        m.sync(upload)
    assert sent and max(sent) <= 5 and sent.count(1) >= len(sent) // 2, sent
    for g in m.groups:
        assert (g.table_dev.numpy() == g.table_host).all()


def test_the_spare_slot_has_a_page_of_its_own_outside_the_pool():
    """Behind the request slots: one more row of every table and state tensor, whose first entry names a page behind the pool's
    pages; no request gets that slot or that page, whatever is opened, grown and closed."""
    m = CacheManager([FULL, WINDOW, StateNeed((3,), torch.float32)], [None, None, None], page_size=4, n_pages=6, max_requests=2, max_positions=24,
                     dtype=torch.float32, device="cpu")
    assert m.spare_slot == 2
    for g in m.groups:
        assert g.table_host.shape[0] == 3 and g.table_host[2].tolist() == [6] + [-1] * 5 and g.table_dev[2].tolist() == [6] + [-1] * 5
        assert g.storage.shape[1] == 7 and g.pool.n_pages == 6
    assert m.states[2].shape == (3, 3)
    for turn in range(3):
        for r in ("a", "b"):
            assert m.open(r) in (0, 1)
        with pytest.raises(CacheError):
            m.open("c")
        m.reserve([("a", 12), ("b", 12)]); m.advance("a", 12); m.advance("b", 12)
        m.sync()
        for g in m.groups:
            assert 6 not in g.table_host[:2] and g.table_host[2].tolist() == [6] + [-1] * 5 and (g.table_dev.numpy() == g.table_host).all()
        m.check_consistency()
        m.close("a"); m.close("b")
    assert m.free_pages() == [6, 6]


def test_batch_sizes_of_captured_decode_steps():
    from geneinfer_amd.engine.runner import captured_batch_size
    sizes = [captured_batch_size(n, 4096) for n in range(1, 400)]
    assert sizes[:8] == list(range(1, 9)) and sizes == sorted(sizes)
    assert all(n <= s <= max(n + 15, n) and s - n < max(1, n // 4) + 1 for n, s in zip(range(1, 400), sizes))
    assert all(captured_batch_size(s, 4096) == s for s in sizes)                       # a size of the list serves itself
    assert len(set(sizes[:64])) == 24 and len(set(sizes)) < 60
    assert captured_batch_size(9, 9) == 9 and captured_batch_size(9, 10) == 10         # never beyond the rows a step may hold
