"""The cache manager: the behaviours the reference's tests fix (tests/test_block_manager.py:11-127
there), groups of pages with different needs, state slots, and that under random orders of
requests no page is lost, held twice or freed twice."""

import random

import pytest

from paged_llm_amd.cache import NO_PAGE, CacheManager, GroupSpec

FULL = [GroupSpec("full")]


def mgr(num_pages, block_size=4, groups=FULL, **kw):
    return CacheManager(groups, num_pages, block_size, **kw)


def test_allocate_and_free_round_trip():
    m = mgr(8)
    assert m.allocate("a", 0, 10)
    table = m.block_table("a", "full")
    assert len(table) == 3 and m.num_free_pages() == 5
    assert m.slot_mapping("a", "full", 0, 10) == [b * 4 + o for b in table for o in range(4)][:10]
    m.free("a")
    assert m.num_free_pages() == 8 and not m.holds("a")
    m.check_invariants()


def test_exhaustion_changes_nothing():
    m = mgr(2)
    assert m.allocate("a", 0, 8)
    assert not m.allocate("b", 0, 3)
    assert not m.holds("b") and m.num_free_pages() == 0
    m.check_invariants()


def test_decoding_fills_the_partial_page_then_takes_a_new_one():
    m = mgr(4)
    assert m.allocate("a", 0, 5)
    assert m.allocate("a", 5, 1) and len(m.block_table("a", "full")) == 2
    assert m.allocate("a", 8, 1) and len(m.block_table("a", "full")) == 3


def test_prefix_hit_shares_pages():
    m = mgr(16)
    a = list(range(10))
    m.allocate("a", 0, 10)
    m.note_computed("a", a, 0, 10)
    assert m.num_cached_pages() == 2
    b = list(range(8)) + [99, 98, 97]
    hits, n = m.find_cached_prefix(b)
    assert n == 8 and hits["full"] == m.block_table("a", "full")[:2]
    assert m.allocate("b", n, len(b) - n, hits)
    assert m.block_table("b", "full")[:2] == m.block_table("a", "full")[:2] and len(m.block_table("b", "full")) == 3
    shared = m.block_table("a", "full")[0]
    assert m.pools["full"].refs[shared] == 2
    m.free("a")
    assert m.pools["full"].refs[shared] == 1
    m.free("b")
    assert m.num_free_pages() == 16
    assert m.find_cached_prefix(list(range(9)))[1] == 8          # still findable while free
    assert m.num_cache_queries == 2 and m.num_cache_hits == 2
    m.check_invariants()


def test_prefix_hit_never_covers_the_whole_prompt():
    m = mgr(8)
    m.allocate("a", 0, 8)
    m.note_computed("a", list(range(8)), 0, 8)
    assert m.find_cached_prefix(list(range(8)))[1] == 4           # the last page is computed again: logits are needed


def test_cached_free_pages_about_to_be_revived_do_not_count_as_available():
    m = mgr(3)
    m.allocate("a", 0, 8)
    m.note_computed("a", list(range(8)), 0, 8)
    m.free("a")
    b = list(range(8)) + [1, 2, 3, 4, 5]
    hits, n = m.find_cached_prefix(b)
    assert n == 8
    assert not m.allocate("b", n, len(b) - n, hits)               # 2 revived + 2 new = 4 > 3
    assert m.num_free_pages() == 3 and not m.holds("b")
    m.check_invariants()


def test_oldest_cached_page_is_evicted_first():
    m = mgr(3)
    for rid, toks in (("a", list(range(4))), ("b", list(range(10, 14)))):
        m.allocate(rid, 0, 4)
        m.note_computed(rid, toks, 0, 4)
        m.free(rid)
    assert m.num_cached_pages() == 2
    m.allocate("c", 0, 8)                                          # takes the untouched page, then a's (older)
    assert m.find_cached_prefix(list(range(4)) + [7])[1] == 0
    assert m.find_cached_prefix(list(range(10, 14)) + [7])[1] == 4


def test_fork_and_copy_on_write():
    m = mgr(8)
    m.allocate("parent", 0, 6)
    m.fork("parent", "child")
    pt = list(m.block_table("parent", "full"))
    assert m.block_table("child", "full") == pt and m.pools["full"].refs[pt[1]] == 2
    assert m.allocate("child", 6, 1)                              # writes into the shared partial page
    ct = m.block_table("child", "full")
    assert ct[0] == pt[0] and ct[1] != pt[1]
    copies = m.take_pending_copies()
    assert [(c.src, c.dst) for c in copies["full"]] == [(pt[1], ct[1])]
    assert m.pools["full"].refs[pt[1]] == 1
    assert m.allocate("parent", 6, 1) and m.take_pending_copies() == {}
    m.check_invariants()


def test_copy_on_write_without_a_free_page_changes_nothing():
    m = mgr(2)
    m.allocate("parent", 0, 6)
    m.fork("parent", "child")
    assert not m.allocate("child", 6, 1)
    assert m.block_table("child", "full") == m.block_table("parent", "full") and m.take_pending_copies() == {}
    m.check_invariants()


def test_double_free_is_detected():
    m = mgr(2)
    m.allocate("a", 0, 4)
    page = m.block_table("a", "full")[0]
    m.free("a")
    with pytest.raises(AssertionError):
        m.pools["full"].drop(page)
    m.free("a")                                                   # freeing an unknown request is a no-op


def test_prefix_caching_off_forgets_freed_pages():
    m = mgr(4, enable_prefix_caching=False)
    m.allocate("a", 0, 8)
    m.note_computed("a", list(range(8)), 0, 8)
    m.free("a")
    assert m.num_cached_pages() == 0 and m.find_cached_prefix(list(range(9)))[1] == 0


def test_digest_depends_on_the_whole_prefix():
    m = mgr(8)
    m.allocate("a", 0, 8)
    m.note_computed("a", [1, 2, 3, 4, 5, 6, 7, 8], 0, 8)
    assert m.find_cached_prefix([9, 9, 9, 9, 5, 6, 7, 8, 0])[1] == 0      # same second page, other first page
    assert m.find_cached_prefix([1, 2, 3, 4, 5, 6, 7, 8, 0])[1] == 8


# ------------------------------------------------------------------ groups with different needs
def test_groups_have_pages_of_their_own():
    groups = [GroupSpec("full"), GroupSpec("win", "window", 6)]
    m = mgr({"full": 8, "win": 4}, groups=groups)
    assert m.allocate("a", 0, 10)
    assert len(m.block_table("a", "full")) == 3 and len(m.block_table("a", "win")) == 3
    assert m.num_free_pages("full") == 5 and m.num_free_pages("win") == 1
    assert not m.prefix_caching
    # the next portion starts at 10: keys before 10 - 6 + 1 = 5 are out of every window: page 0 comes back
    assert m.allocate("a", 10, 4)
    assert m.block_table("a", "win")[0] == NO_PAGE and m.block_table("a", "win")[1] != NO_PAGE
    assert m.num_free_pages("win") == 1 and len(m.block_table("a", "win")) == 4
    assert NO_PAGE not in m.block_table("a", "full")
    m.check_invariants()
    m.free("a")
    assert m.num_free_pages("full") == 8 and m.num_free_pages("win") == 4


def test_window_group_decodes_forever_in_a_small_pool():
    m = mgr(3, groups=[GroupSpec("win", "window", 5)])
    at = 0
    assert m.allocate("a", at, 3)
    at = 3
    for _ in range(200):
        assert m.allocate("a", at, 1), at
        at += 1
        live = [p for p in m.block_table("a", "win") if p != NO_PAGE]
        assert len(live) <= 3
        first_key = at - 1 - 5 + 1
        assert all(p != NO_PAGE for p in m.block_table("a", "win")[max(0, first_key) // 4:])
    m.check_invariants()


def test_smallest_group_decides_all_or_nothing():
    m = mgr({"full": 8, "win": 1}, groups=[GroupSpec("full"), GroupSpec("win", "window", 100)])
    assert not m.allocate("a", 0, 5)                               # 2 pages needed in "win", 1 there
    assert m.num_free_pages("full") == 8 and not m.holds("a")


# ------------------------------------------------------------------ state slots
def test_state_slots_come_and_go_with_the_pages():
    m = mgr(8, num_state_slots=2)
    assert m.allocate("a", 0, 3) and m.allocate("b", 0, 3)
    assert {m.state_slot("a"), m.state_slot("b")} == {0, 1}
    assert not m.allocate("c", 0, 3) and not m.holds("c") and m.num_free_pages() == 6
    m.free("a")
    assert m.allocate("c", 0, 3) and m.state_slot("c") is not None
    m.check_invariants()
    no_state = mgr(8)
    no_state.allocate("a", 0, 3)
    assert no_state.state_slot("a") is None


def test_state_only_model_has_no_pages():
    m = CacheManager([], 1, 16, num_state_slots=1)
    assert m.allocate("a", 0, 1000) and m.state_slot("a") == 0
    assert not m.allocate("b", 0, 1)
    m.free("a")
    assert m.allocate("b", 0, 1)


# ------------------------------------------------------------------ random orders
@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("groups", [FULL, [GroupSpec("full"), GroupSpec("win", "window", 9)]], ids=["one", "two"])
def test_random_orders_lose_nothing(seed, groups):
    rng = random.Random(seed)
    bs = 4
    m = CacheManager(groups, 24, bs, enable_prefix_caching=True, num_state_slots=5)
    live: dict = {}        # id -> [tokens, computed]
    next_id = 0
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and len(live) < 8:
            base = rng.choice([[1] * 8, [2] * 12, []])                 # shared prefixes now and then
            toks = base + [rng.randrange(50) for _ in range(rng.randrange(1, 20))]
            hits, n = m.find_cached_prefix(toks)
            first = min(len(toks) - n, rng.randrange(1, 12))
            if m.allocate(next_id, n, first, hits):
                m.note_computed(next_id, toks, n, n + first)
                live[next_id] = [toks, n + first]
            next_id += 1
        elif action < 0.75 and live:
            rid = rng.choice(list(live))
            toks, done = live[rid]
            if done == len(toks):
                toks.append(rng.randrange(50))                          # a decoded token
            n = min(len(toks) - done, rng.randrange(1, 7))
            if m.allocate(rid, done, n):
                m.note_computed(rid, toks, done, done + n)
                live[rid][1] = done + n
        elif action < 0.85 and live and len(live) < 8:
            parent = rng.choice(list(live))
            try:
                m.fork(parent, next_id)
                live[next_id] = [list(live[parent][0]), live[parent][1]]
            except RuntimeError:
                pass
            next_id += 1
        elif live:
            rid = rng.choice(list(live))
            m.free(rid)
            del live[rid]
        m.take_pending_copies()
        m.check_invariants()
        for rid, (toks, done) in live.items():
            for g in m.groups.values():
                table = m.block_table(rid, g.name)
                assert len(table) >= (done + bs - 1) // bs
                first_key = max(0, done - g.window + 1) if g.kind == "window" else 0
                assert all(p != NO_PAGE for p in table[first_key // bs:])
    for rid in list(live):
        m.free(rid)
    m.check_invariants()
    assert all(m.num_free_pages(g) == 24 for g in m.groups) and m.slots.num_free == 5


@pytest.mark.parametrize("seed", range(4))
def test_digests_made_ahead_index_the_same_pages(seed):
    """Two managers in lockstep under random orders of requests with shared prefixes, forks and decoded tokens; one
    has the digests of a request's full pages made ahead (at random moments, for random lengths of what it holds):
    after every action both index the same pages under the same digests."""
    rng = random.Random(seed)
    bs = 4
    a, b = (CacheManager(FULL, 32, bs, enable_prefix_caching=True) for _ in range(2))
    live: dict = {}
    next_id = made = 0
    for _ in range(500):
        action = rng.random()
        if action < 0.3 and len(live) < 8:
            base = rng.choice([[1] * 8, [2] * 12, [3] * 17, []])
            toks = base + [rng.randrange(50) for _ in range(rng.randrange(1, 30))]
            (hits, n), (hits_b, n_b) = a.find_cached_prefix(toks), b.find_cached_prefix(toks)
            assert (hits, n) == (hits_b, n_b)
            first = min(len(toks) - n, rng.randrange(1, 24))
            ok = a.allocate(next_id, n, first, hits)
            assert ok == b.allocate(next_id, n, first, hits_b)
            if ok:
                if rng.random() < 0.7:
                    a.digests_ahead(next_id, toks, rng.randrange(0, len(toks) + 1))
                    made += 1
                a.note_computed(next_id, toks, n, n + first)
                b.note_computed(next_id, toks, n, n + first)
                live[next_id] = [toks, n + first]
            next_id += 1
        elif action < 0.75 and live:
            rid = rng.choice(list(live))
            toks, done = live[rid]
            if done == len(toks):
                toks.append(rng.randrange(50))
            n = min(len(toks) - done, rng.randrange(1, 9))
            ok = a.allocate(rid, done, n)
            assert ok == b.allocate(rid, done, n)
            if ok:
                if rng.random() < 0.5:
                    a.digests_ahead(rid, toks, done + n)
                    made += 1
                a.note_computed(rid, toks, done, done + n)
                b.note_computed(rid, toks, done, done + n)
                live[rid][1] = done + n
        elif action < 0.85 and live and len(live) < 8:
            parent = rng.choice(list(live))
            a.fork(parent, next_id)
            b.fork(parent, next_id)
            live[next_id] = [list(live[parent][0]), live[parent][1]]
            next_id += 1
        elif live:
            rid = rng.choice(list(live))
            a.free(rid)
            b.free(rid)
            del live[rid]
        assert a.take_pending_copies() == b.take_pending_copies()
        a.check_invariants()
        for g in a.pools:
            assert a.pools[g].digest == b.pools[g].digest and a.pools[g].by_digest == b.pools[g].by_digest
    assert made > 50 and any(p.by_digest for p in a.pools.values())


def test_no_prefix_reuse_for_models_with_state_slots():
    """A state of fixed size exists only as of the last token run: a request that entered behind a cached
    prefix would start from a state that never saw those tokens.  With state slots in use the prefix index
    is off, whatever the option says."""
    m = CacheManager([GroupSpec("full")], 16, 4, True, num_state_slots=4)
    assert not m.prefix_caching
    tokens = list(range(100, 120))
    assert m.allocate("a", 0, len(tokens))
    m.note_computed("a", tokens, 0, len(tokens))
    m.free("a")
    hits, cached = m.find_cached_prefix(tokens + [1, 2])
    assert cached == 0 and hits == {"full": []} and m.num_cached_pages() == 0
    m.check_invariants()
    # the same without state slots finds the prefix again
    plain = CacheManager([GroupSpec("full")], 16, 4, True)
    assert plain.allocate("a", 0, len(tokens))
    plain.note_computed("a", tokens, 0, len(tokens))
    plain.free("a")
    assert plain.find_cached_prefix(tokens + [1, 2])[1] == 20


def test_a_fork_hands_the_parents_state_to_the_child():
    m = CacheManager([GroupSpec("full")], 16, 4, False, num_state_slots=3)
    assert m.allocate("parent", 0, 6)
    m.fork("parent", "child")
    copies = m.take_pending_state_copies()
    assert [(c.src, c.dst) for c in copies] == [(m.state_slot("parent"), m.state_slot("child"))]
    assert m.state_slot("parent") != m.state_slot("child") and m.take_pending_state_copies() == []
    m.check_invariants()
