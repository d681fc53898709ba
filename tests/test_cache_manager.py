"""The cache manager without a model: no page or slot lost, held twice or freed twice.

Vectors from the reference's tests/unit/kv/test_block_manager.py (page size 4, 16 pages,
watermark 0) and tests/unit/kv/test_hashing_and_policies.py.
"""

from __future__ import annotations

import random

import pytest

from dli_amd.cache import (
    RELEASED, CacheManager, CopyOp, GroupSpec, OldestFirst, ReusedLast, NoFreePagesError, NoFreeSlotError,
    ROOT_PARENT, SequenceError, StateSlots, chain_hashes, page_hash,
)


def mk(num_pages=16, page_size=4, **kw):
    kw.setdefault("watermark", 0.0)
    return CacheManager(num_pages=num_pages, page_size=page_size, **kw)


# ------------------------------------------------------------------ allocation and addressing

def test_prompt_takes_ceil_pages_and_slots_follow_the_table():
    m = mk()
    a = m.allocate("a", list(range(9)))
    assert len(a.block_table) == 3 and m.num_available_pages == 13 and a.num_cached_tokens == 0
    t = a.block_table
    assert m.slot_mapping("a", 2, 8) == [t[0] * 4 + 2, t[0] * 4 + 3, t[1] * 4, t[1] * 4 + 1, t[1] * 4 + 2, t[1] * 4 + 3]
    with pytest.raises(ValueError):
        m.slot_mapping("a", 0, 10)
    m.check_invariants()


def test_appends_take_a_page_at_boundaries_only():
    m = mk()
    m.allocate("a", [1, 2, 3])
    assert len(m.block_table("a")) == 1
    m.append_slots("a", [4])
    assert len(m.block_table("a")) == 1
    m.append_slots("a", [5])
    assert len(m.block_table("a")) == 2
    m.append_slots("a", [6, 7, 8, 9])
    assert len(m.block_table("a")) == 3 and m.num_tokens("a") == 9
    m.check_invariants()


def test_errors_leave_the_state_unchanged():
    m = mk(num_pages=4)
    m.allocate("a", list(range(10)))
    with pytest.raises(NoFreePagesError):
        m.allocate("b", list(range(8)))
    with pytest.raises(SequenceError):
        m.allocate("a", [1])
    with pytest.raises(ValueError):
        m.allocate("c", [])
    m.append_slots("a", [0, 0])  # fills page 3
    m.append_slots("a", [0, 0, 0, 0])  # takes the last page
    with pytest.raises(NoFreePagesError):
        m.append_slots("a", [0])
    assert m.num_tokens("a") == 16 and not m.has_sequence("b")
    with pytest.raises(SequenceError):
        m.free("zzz")
    m.free("a")
    with pytest.raises(SequenceError):
        m.free("a")  # freed twice
    m.check_invariants()
    assert m.stats().free_pages == 4


def test_watermark_holds_pages_back_at_admission_only():
    m = CacheManager(num_pages=10, page_size=4, watermark=0.2)
    assert not m.can_allocate(list(range(36)))  # 9 pages would leave 1 < 2
    assert m.can_allocate(list(range(32)))
    m.allocate("a", list(range(32)))
    m.append_slots("a", list(range(8)))  # appends may use the reserve
    assert m.num_available_pages == 0
    m.check_invariants()


# ------------------------------------------------------------------ content reuse

def test_pages_are_reusable_only_after_they_are_computed():
    m = mk()
    p = list(range(10))
    m.allocate("a", p)
    assert m.allocate("b", p).num_cached_tokens == 0  # allocated, not computed: no hit
    m.mark_computed("a", 10)
    assert m.allocate("c", p).num_cached_tokens == 8
    m.check_invariants()


def test_last_token_page_is_never_served_from_the_index():
    m = mk()
    p = list(range(8))  # exactly two pages
    m.allocate("a", p)
    m.mark_computed("a", 8)
    assert m.allocate("b", p).num_cached_tokens == 4
    q = p[:5] + [99] + p[6:] + [1, 2]
    assert m.allocate("c", q).num_cached_tokens == 4  # differs inside page 2
    m.check_invariants()


def test_namespaces_do_not_share():
    m = mk()
    p = list(range(9))
    m.allocate("a", p, namespace=b"x")
    m.mark_computed("a", 9)
    assert m.allocate("b", p, namespace=b"y").num_cached_tokens == 0
    assert m.allocate("c", p, namespace=b"x").num_cached_tokens == 8


def test_decoded_tokens_complete_pages_that_become_reusable():
    m = mk()
    m.allocate("a", [1, 2, 3])
    m.mark_computed("a", 3)
    for t in range(4, 10):
        m.append_slots("a", [t])
        m.mark_computed("a", m.num_tokens("a"))
    assert m.allocate("b", list(range(1, 10)) + [0]).num_cached_tokens == 8
    m.check_invariants()


def test_duplicate_prompts_admitted_together_keep_private_pages():
    m = mk()
    p = list(range(9))
    m.allocate("a", p)
    m.allocate("b", p)
    m.mark_computed("a", 9)
    m.mark_computed("b", 9)
    assert m.stats().duplicate_registrations == 2
    m.free("a")
    m.free("b")
    m.check_invariants()
    assert m.num_available_pages == 16


def test_leaves_are_reclaimed_first_and_revived_pages_are_safe():
    m = mk(num_pages=4)
    p = list(range(13))  # 4 pages, 3 of them full
    m.allocate("a", p)
    m.mark_computed("a", 13)
    m.free("a")
    assert m.stats().cached_idle_pages == 3 and m.stats().free_pages == 1
    m.allocate("b", [50, 51, 52, 53, 54])  # 2 pages: the free one and the deepest cached leaf
    assert m.stats().evictions == 1
    m.free("b")
    assert m.allocate("c", p[:9]).num_cached_tokens == 8  # the two-page prefix survived
    m.check_invariants()
    with pytest.raises(NoFreePagesError):  # the revived pages cannot be reclaimed for someone else
        m.allocate("d", [7] * 9)
    m.free("c")
    m.reset_prefix_cache()
    m.check_invariants()
    assert m.stats().free_pages == 4


def test_fork_shares_pages_and_copies_on_write():
    m = mk()
    m.allocate("a", list(range(6)))
    m.mark_computed("a", 6)
    m.fork("a", "b")
    shared = m.block_table("a")[-1]
    ops = m.append_slots("b", [7])
    assert ops == [CopyOp(src=shared, dst=m.block_table("b")[-1], group=0)]
    assert m.block_table("a")[-1] == shared and m.block_table("b")[0] == m.block_table("a")[0]
    assert m.append_slots("a", [8]) == []  # a is the only holder now
    assert m.stats().cow_copies == 1
    m.check_invariants()
    m2 = mk()
    m2.allocate("a", list(range(8)))
    m2.fork("a", "b")
    assert m2.append_slots("b", [1]) == []  # fork at a page boundary: nothing to copy
    m2.check_invariants()


def test_without_content_reuse_nothing_is_kept():
    m = mk(enable_prefix_caching=False)
    p = list(range(9))
    m.allocate("a", p)
    m.mark_computed("a", 9)
    m.free("a")
    assert m.stats().cached_idle_pages == 0 and m.allocate("b", p).num_cached_tokens == 0


# ------------------------------------------------------------------ identities and policies

def test_page_identities():
    a, b = chain_hashes(b"m", [1, 2, 3, 4, 5, 6], 3), chain_hashes(b"m", [9, 9, 9, 4, 5, 6], 3)
    assert len(a) == len(b) == 2 and a[1] != b[1]
    assert len(chain_hashes(b"m", list(range(7)), 3)) == 2  # the partial tail has no identity
    assert page_hash(b"ab", ROOT_PARENT, [1, 2, 3]) != page_hash(b"a", ROOT_PARENT, [1, 2, 3])
    assert page_hash(b"", ROOT_PARENT, [2 ** 40]) != page_hash(b"", ROOT_PARENT, [0])
    import hashlib
    import struct
    want = hashlib.sha256(struct.pack("<I", 1) + b"m" + bytes(32) + struct.pack("<3q", 1, 2, 3)).digest()
    assert a[0] == want


def test_reclaim_orders():
    p = OldestFirst()
    for page in (1, 2, 3):
        p.offer(page)
    p.withdraw(1)
    p.offer(1)
    assert [p.take() for _ in range(3)] == [2, 3, 1]
    with pytest.raises(LookupError):
        p.take()
    # a page that a later request found again outlives one-off pages however recent ...
    r = ReusedLast()
    for page in (1, 2, 3):
        r.cached(page, 0)
        r.offer(page)
    r.found(1)
    r.withdraw(1)          # revived by the request that found it
    r.offer(1)             # and released again
    r.cached(4, 0)
    r.offer(4)
    assert len(r) == 4 and [r.take() for _ in range(4)] == [2, 3, 4, 1]
    with pytest.raises(LookupError):
        r.take()
    # ... but only as long as it keeps being found: one stay without a match and it is ordinary again
    r.offer(1)
    r.offer(5)
    assert [r.take(), r.take()] == [1, 5]
    # in a manager: the prefix two requests shared survives pressure that the one-off prompt does not
    for order, kept in (("reuse", True), ("lru", False)):
        m = CacheManager(num_pages=8, page_size=4, max_seqs=4, eviction_policy=order, watermark=0.0)
        popular, one_off = list(range(8)), list(range(100, 108))
        for rid, prompt in (("a", popular + [50]), ("b", popular + [51]), ("c", one_off + [52])):
            m.allocate(rid, prompt)
            m.mark_computed(rid, 9)
            m.free(rid)
        m.allocate("big", list(range(200, 224)))   # 6 of 8 pages: two of the four idle pages must go
        m.free("big")
        assert (m.allocate("again", popular + [1]).num_cached_tokens == 8) == kept, order
        m.check_invariants()
    with pytest.raises(ValueError):
        CacheManager(num_pages=8, page_size=4, max_seqs=4, eviction_policy="newest")


# ------------------------------------------------------------------ groups, windows, state slots

def test_window_group_gives_pages_back_while_the_request_runs():
    m = CacheManager([GroupSpec(), GroupSpec("window", 6)], num_pages=[32, 8], page_size=4, watermark=0.0)
    m.allocate("a", list(range(10)))
    assert len(m.block_table("a", 0)) == 3 and len(m.block_table("a", 1)) == 3
    m.mark_computed("a", 10)
    # next query at position 10 sees keys 5..10: page 0 (keys 0..3) is passed
    assert m.block_table("a", 1)[0] == RELEASED and m.block_table("a", 1)[1] != RELEASED
    assert m.block_table("a", 0)[0] != RELEASED
    used_before = m.pools[1].num_pages - m.pools[1].num_available
    for t in range(40):  # far more tokens than the 8 window pages could hold
        m.append_slots("a", [t])
        m.mark_computed("a", m.num_tokens("a"))
        m.check_invariants()
    assert m.pools[1].num_pages - m.pools[1].num_available <= used_before + 1
    assert m.stats().window_pages_released >= 10
    with pytest.raises(ValueError):
        m.slot_mapping("a", 0, 1, group=1)
    m.free("a")
    m.check_invariants()
    assert all(p.num_available == p.num_pages for p in m.pools)


def test_two_full_groups_serve_a_prompt_as_far_as_both_hold_it():
    m = CacheManager([GroupSpec(), GroupSpec()], num_pages=[16, 5], page_size=4, watermark=0.0)
    assert m.prefix_caching
    a = list(range(17))                       # four full pages and the page of the last token
    m.allocate("a", a)
    m.mark_computed("a", 17)
    m.free("a")
    got = m.allocate("b", a + [99])
    assert got.num_cached_tokens == 16
    assert all(len(t) == 5 for t in got.block_tables)
    m.free("b")
    # the small group loses pages of the run to another prompt (leaves first): the run ends there in both
    m.allocate("c", [50, 51, 52, 53, 54, 55, 56, 57, 58])        # three pages of the second group's five
    m.check_invariants()
    assert sum(1 for h in chain_hashes(b"", a[:16], 4) if h in m.pools[1].by_identity) == 2
    assert sum(1 for h in chain_hashes(b"", a[:16], 4) if h in m.pools[0].by_identity) == 4
    m.free("c")
    got = m.allocate("d", a)
    assert got.num_cached_tokens == 8
    assert got.block_tables[0][:2] != got.block_tables[0][2:4] and len(got.block_tables[1]) == 5
    m.check_invariants()


def test_a_window_group_serves_the_pages_that_the_first_computed_token_still_reaches():
    ps, window = 4, 6
    m = CacheManager([GroupSpec(), GroupSpec("window", window)], num_pages=[32, 12], page_size=ps, watermark=0.0)
    a = list(range(30))
    m.allocate("a", a)
    for upto in (7, 19, 30):                  # in portions: pages are entered before the window passes them
        m.mark_computed("a", upto)
        m.check_invariants()
    held = m.block_table("a", 1)
    assert held[:6] == (RELEASED,) * 6        # next query at 30 sees keys 25..: pages 0..5 are passed
    m.free("a")
    # 22 tokens in common, then others: five full pages match; a query at 20 sees keys 15..20: from page 3 on
    b = a[:22] + [77, 78, 79]
    got = m.allocate("b", b)
    assert got.num_cached_tokens == 20
    full, win = got.block_tables
    assert RELEASED not in full and len(full) == len(win) == 7
    assert win[:3] == (RELEASED,) * 3 and RELEASED not in win[3:]
    assert m.slot_mapping("b", 15, 25, group=1)
    with pytest.raises(ValueError):
        m.slot_mapping("b", 11, 12, group=1)
    m.check_invariants()
    m.mark_computed("b", 25)
    m.check_invariants()
    # the window group has lost a page that such a run needs: the run is cut back to where both can serve it
    m.free("b")
    h = chain_hashes(b"", a[:20], ps)
    pool = m.pools[1]
    victim = pool.by_identity[h[4]]
    while victim in pool.cached:              # reclaim idle pages until that one has gone
        pool.free.append(pool._evict(pool.order.take()))
    m.check_invariants()
    got = m.allocate("c", b)
    assert got.num_cached_tokens < 20
    first = max(0, got.num_cached_tokens - window + 1) // ps
    assert got.block_tables[1][:first] == (RELEASED,) * first and RELEASED not in got.block_tables[1][first:]
    m.check_invariants()


def test_state_slots_are_taken_and_given_back():
    m = mk(max_seqs=2)
    a = m.allocate("a", [1]).state_slot
    b = m.allocate("b", [1]).state_slot
    assert {a, b} == {0, 1} and not m.can_allocate([1])
    with pytest.raises(NoFreeSlotError):
        m.allocate("c", [1])
    m.free("a")
    assert m.allocate("c", [1]).state_slot == a
    m.check_invariants()
    s = StateSlots(1)
    slot = s.take()
    s.give_back(slot)
    with pytest.raises(AssertionError):
        s.give_back(slot)


# ------------------------------------------------------------------ random orders

@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("policy", ["lru", "reuse"])
def test_random_orders_of_requests_keep_every_invariant(seed, policy):
    rng = random.Random(seed)
    page_size = rng.choice([1, 2, 4, 8])
    groups = [GroupSpec()] if seed % 2 == 0 else [GroupSpec(), GroupSpec("window", rng.choice([3, 8, 17]))]
    m = CacheManager(groups, num_pages=rng.randrange(6, 40), page_size=page_size, max_seqs=5,
                     eviction_policy=policy, watermark=rng.choice([0.0, 0.1]))
    shadow: dict = {}   # request -> tokens, as the manager should know them
    stems = [[rng.randrange(5) for _ in range(rng.randrange(1, 30))] for _ in range(4)]
    n_id = 0
    for _ in range(600):
        op = rng.random()
        try:
            if op < 0.3:
                toks = list(rng.choice(stems)) + [rng.randrange(5) for _ in range(rng.randrange(0, 6))]
                alloc = m.allocate(n_id, toks)
                assert alloc.num_cached_tokens % page_size == 0 and alloc.num_cached_tokens < len(toks)
                shadow[n_id] = toks
                n_id += 1
            elif op < 0.55 and shadow:
                rid = rng.choice(list(shadow))
                new = [rng.randrange(5) for _ in range(rng.randrange(1, 5))]
                m.append_slots(rid, new)
                shadow[rid] = shadow[rid] + new
            elif op < 0.8 and shadow:
                rid = rng.choice(list(shadow))
                lo = m.num_computed_tokens(rid)
                m.mark_computed(rid, rng.randrange(lo, len(shadow[rid]) + 1))
            elif op < 0.88 and shadow:
                rid = rng.choice(list(shadow))
                m.fork(rid, n_id)
                shadow[n_id] = list(shadow[rid])
                n_id += 1
            elif shadow:
                rid = rng.choice(list(shadow))
                m.free(rid)
                del shadow[rid]
        except (NoFreePagesError, NoFreeSlotError):
            pass  # refused: the state must be unchanged, which the invariants below check
        m.check_invariants()
        for rid, toks in shadow.items():
            assert m.num_tokens(rid) == len(toks)
        st = m.stats()
        assert st.free_pages + st.cached_idle_pages + st.used_pages == st.num_pages
    for rid in list(shadow):
        m.free(rid)
    m.reset_prefix_cache()
    m.check_invariants()
    assert m.stats().free_pages == m.stats().num_pages, "pages were lost"
    assert m.slots.num_free == 5, "state slots were lost"


@pytest.mark.parametrize("groups,pages", [
    ([GroupSpec()], [24]),
    ([GroupSpec(), GroupSpec()], [24, 17]),
    ([GroupSpec(), GroupSpec("window", 6)], [24, 14]),
    ([GroupSpec("window", 9), GroupSpec(), GroupSpec("window", 3)], [20, 24, 12]),
])
def test_shadow_cache_never_serves_wrong_or_unwritten_content(groups, pages):
    """A shadow of the device memory of every group: slot -> (token prefix that was written there).
    A hit must point at pages whose shadow equals the new prompt's prefix, in every group, for
    every key that the request's first computed token and the ones after it read there (all
    of them, or those inside the window); and a write must never land in a page that another
    request holds. Steps compute in portions of any length, as an engine's would."""
    rng = random.Random(7 + len(groups))
    ps = 4
    m = CacheManager(groups, num_pages=pages, page_size=ps, watermark=0.0)
    assert m.prefix_caching
    written: list[dict[int, tuple]] = [{} for _ in groups]
    live: dict = {}
    hits = 0
    stems = [[rng.randrange(3) for _ in range(22)] for _ in range(3)]
    for step in range(1200):
        if rng.random() < 0.4 or not live:
            toks = (rng.choice(stems)[:rng.randrange(0, 22)] + [rng.randrange(3) for _ in range(rng.randrange(1, 12))])[:28]
            try:
                alloc = m.allocate(step, toks)
            except (NoFreePagesError, NoFreeSlotError):
                if live:
                    rid = rng.choice(list(live))
                    m.free(rid)
                    del live[rid]
                continue
            cached = alloc.num_cached_tokens
            hits += cached > 0
            for g, spec in enumerate(groups):
                first_read = max(0, cached - spec.window + 1) if spec.kind == "window" else 0
                for p in range(first_read, cached):
                    slot = m.slot_mapping(step, p, p + 1, group=g)[0]
                    assert written[g].get(slot) == tuple(toks[:p + 1]), "a hit serves wrong or unwritten content"
            live[step] = toks
        else:
            rid = rng.choice(list(live))
            toks = live[rid]
            lo = m.num_computed_tokens(rid)
            hi = rng.randrange(lo, len(toks) + 1)
            for g, spec in enumerate(groups):
                for p in range(lo, hi):  # the step function writes these slots
                    slot = m.slot_mapping(rid, p, p + 1, group=g)[0]
                    page = slot // ps
                    holders = sum(1 for other in live if page in m.block_table(other, g))
                    assert holders == 1, "a write lands in a page that another request holds"
                    written[g][slot] = tuple(toks[:p + 1])
                if spec.kind == "window" and hi > lo:   # and every key that the portion's queries read is in place
                    for p in range(max(0, lo - spec.window + 1), lo):
                        slot = m.slot_mapping(rid, p, p + 1, group=g)[0]
                        assert written[g].get(slot) == tuple(toks[:p + 1])
            m.mark_computed(rid, hi)
            if hi == len(toks) and rng.random() < 0.5:
                m.free(rid)
                del live[rid]
        m.check_invariants()
    assert hits > 40


def test_reserving_ahead_takes_pages_now_and_appends_use_them():
    m = CacheManager(num_pages=8, page_size=4, max_seqs=4, watermark=0.0)
    m.allocate("a", [1, 2, 3, 4, 5])           # 2 pages
    m.mark_computed("a", 4)
    m.reserve_ahead("a", 7)                     # room for 12 tokens: 3 pages
    assert len(m.block_table("a")) == 3 and m.num_tokens("a") == 5
    m.check_invariants()
    before = m.stats().free_pages
    table = m.block_table("a")
    for t in range(6):
        assert m.append_slots("a", [t]) == []
    assert m.block_table("a") == table and m.stats().free_pages == before, "appends took pages they had"
    m.check_invariants()
    assert m.append_slots("a", [9, 9]) == []    # 13 tokens: a 4th page
    assert len(m.block_table("a")) == 4
    m.check_invariants()
    # nothing changes when the pool cannot serve the reservation
    m.allocate("b", list(range(13)))            # 4 pages: the pool is full
    with pytest.raises(NoFreePagesError):
        m.reserve_ahead("a", 8)
    assert len(m.block_table("a")) == 4
    m.check_invariants()
    m.free("b")
    m.reserve_ahead("a", 8)                     # 21 tokens: 6 pages
    assert len(m.block_table("a")) == 6
    # a fork shares what is written, not what is reserved ahead
    m.fork("a", "c")
    assert len(m.block_table("c")) == 4
    m.check_invariants()
    ops = m.append_slots("a", [7])              # position 13 lies in a page that the fork shares
    assert len(ops) == 1 and ops[0].src == m.block_table("c")[3] and ops[0].dst == m.block_table("a")[3]
    m.check_invariants()
    m.free("a")
    m.free("c")
    m.reset_prefix_cache()
    m.check_invariants()
    assert m.stats().free_pages == 8


def test_a_confined_manager_refuses_other_threads():
    """The owner-thread check of the reference's block manager (src/dli/kv/block_manager.py:447-449):
    changes from a thread that does not own the manager fail at once and change nothing; reading
    is allowed; adopt() hands the manager over."""
    import threading

    from dli_amd.cache import WrongThreadError

    m = CacheManager(num_pages=8, page_size=4, confine_to_thread=True)
    m.allocate("a", [1, 2, 3, 4, 5])
    seen = {}

    def elsewhere():
        for name, call in (("allocate", lambda: m.allocate("b", [1, 2, 3])), ("append", lambda: m.append_slots("a", [6])),
                           ("free", lambda: m.free("a")), ("fork", lambda: m.fork("a", "c")),
                           ("computed", lambda: m.mark_computed("a", 5)), ("reset", m.reset_prefix_cache)):
            try:
                call()
                seen[name] = "went through"
            except WrongThreadError as e:
                seen[name] = str(e)
        seen["read"] = (m.block_table("a"), m.num_tokens("a"))

    t = threading.Thread(target=elsewhere)
    t.start()
    t.join()
    assert all("belongs to thread" in seen[k] for k in ("allocate", "append", "free", "fork", "computed", "reset")), seen
    assert seen["read"] == (m.block_table("a"), 5)
    m.check_invariants()
    assert m.sequences() == ["a"]

    def adopted():
        m.adopt()
        m.append_slots("a", [6])
        seen["adopted"] = m.num_tokens("a")

    t = threading.Thread(target=adopted)
    t.start()
    t.join()
    assert seen["adopted"] == 6
    with pytest.raises(WrongThreadError):
        m.free("a")          # the first thread gave it away
    m.adopt()
    m.free("a")
    # not confined: any thread may call
    free_for_all = CacheManager(num_pages=4, page_size=4)
    t = threading.Thread(target=lambda: free_for_all.allocate("x", [1]))
    t.start()
    t.join()
    assert free_for_all.sequences() == ["x"]


def test_messages_of_unknown_requests_and_of_the_policy_that_is_not_built():
    """A request id's error prints as its message, not as a quoted repr (it is a KeyError for
    callers that catch that); and the reference's second eviction policy, which is not built, is
    refused by name with the nearest one named, instead of silently selecting another order."""
    from dli_amd.cache.manager import SequenceError
    from dli_amd.cache.reclaim import make_order

    assert str(SequenceError("unknown sequence 'x'")) == "unknown sequence 'x'"
    m = CacheManager(num_pages=4, page_size=4)
    with pytest.raises(SequenceError, match="^unknown sequence 'nobody'$"):
        m.num_tokens("nobody")
    with pytest.raises(KeyError):
        m.free("nobody")
    assert make_order("lru").name == "lru" and make_order("reuse").name == "reuse"
    with pytest.raises(ValueError, match="'reuse' is the nearest"):
        make_order("cost")
    with pytest.raises(ValueError, match="'reuse' is the nearest"):
        CacheManager(num_pages=4, page_size=4, eviction_policy="cost")
    with pytest.raises(ValueError, match="unknown eviction policy"):
        make_order("random")
