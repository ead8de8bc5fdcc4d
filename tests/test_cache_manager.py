"""The cache manager: pages and slots under every order of requests.

No page is lost, held twice or given back twice; groups keep pages of their own; a windowed
group gives back the pages its window has passed; exhaustion changes nothing.
"""
import random

import pytest
from hypothesis import given, settings, strategies as st

from gesso_amd.cache import RELEASED, CacheLayout, CacheManager, PagePool, SlotPool
from gesso_amd.errors import InvalidPlan, OutOfPages, OutOfSlots, ResourceLimit
from gesso_amd.parts.base import PagedKV, SlotState

FULL = PagedKV(2, 16, None)
WIN = PagedKV(2, 16, 20)
CONV = SlotState((("history", (8, 2), "float32"),))


def lfm2_like():
    # conv, attn, conv, attn
    return CacheLayout.plan([CONV, FULL, CONV, FULL], [None] * 4)


def test_pool_basics():
    p = PagePool(3)
    a = p.take(2)
    assert a == [0, 1] and p.n_free == 1
    with pytest.raises(OutOfPages):
        p.take(2)
    assert p.n_free == 1                     # nothing was taken
    p.give_back([0])
    with pytest.raises(InvalidPlan):
        p.give_back([0])                     # given back twice
    with pytest.raises(InvalidPlan):
        p.give_back([2])                     # never handed out
    assert p.take(1) == [0]                  # the page that came back is used again first
    p.check()
    with pytest.raises(OutOfSlots):
        SlotPool(0).take(1)


def test_layout_groups_by_need():
    lay = CacheLayout.plan([CONV, FULL, WIN, FULL, None, WIN, CONV], [None, None, None, None, 1, None, None])
    assert [g.members for g in lay.paged] == [(1, 3), (2, 5)]
    assert [g.need.window for g in lay.paged] == [None, 20]
    assert [m.call for m in lay.slots] == [0, 6]
    assert lay.source_of_call[4] == 1 and lay.source_of_call[3] == 3
    with pytest.raises(InvalidPlan):
        CacheLayout.plan(["what"], [None])


def test_pages_grow_at_page_edges():
    m = CacheManager(lfm2_like(), page_size=4, num_pages=10, num_slots=2, max_length=64)
    m.admit("a")
    assert m.fresh_slots == [0]
    m.reserve("a", 5)                        # 5 rows at page size 4: two pages (test/test_kv_manager.jl:128-166)
    assert m.get("a").tables == [[0, 1]]
    m.commit("a", 5)
    assert m.pages_needed("a", 3) == [0] and m.pages_needed("a", 4) == [1]
    m.reserve("a", 3)
    m.commit("a", 3)
    m.reserve("a", 1)
    assert m.get("a").tables == [[0, 1, 2]]
    m.commit("a", 1)
    assert m.get("a").length == 9
    m.check()
    m.release("a")
    assert m.stats()["pages_free"] == [10] and m.stats()["slots_free"] == 2
    with pytest.raises(InvalidPlan):
        m.release("a")


def test_exhaustion_changes_nothing():
    m = CacheManager(lfm2_like(), page_size=4, num_pages=3, num_slots=1, max_length=64)
    m.admit("a")
    with pytest.raises(OutOfSlots):
        m.admit("b")
    m.reserve("a", 8)
    with pytest.raises(OutOfPages) as e:
        m.reserve("a", 13 - 8 + 8)           # would need 6 pages in all
    assert e.value.detail["free"] == 1
    assert m.get("a").tables == [[0, 1]] and m.pools[0].n_free == 1
    with pytest.raises(ResourceLimit):
        m.reserve("a", 100)                  # beyond the context, whatever the pool holds
    m.check()


def test_reserve_many_is_one_decision():
    m = CacheManager(lfm2_like(), page_size=4, num_pages=4, num_slots=3, max_length=64)
    for r in "abc":
        m.admit(r)
    with pytest.raises(OutOfPages):
        m.reserve_many([("a", 8), ("b", 8), ("c", 1)])
    assert all(m.get(r).tables == [[]] for r in "abc") and m.pools[0].n_free == 4
    m.reserve_many([("a", 8), ("b", 7)])
    assert m.pools[0].n_free == 0
    m.check()


def test_window_group_gives_pages_back_and_full_group_keeps_them():
    lay = CacheLayout.plan([FULL, WIN], [None, None])
    m = CacheManager(lay, page_size=8, num_pages=[16, 5], num_slots=1, max_length=128)
    m.admit("a")
    assert m.get("a").slot is None           # nobody keeps fixed-size state here
    m.reserve("a", 30)
    m.commit("a", 30)
    # the next query is at 30 and reads keys 11..30: page 0 (keys 0..7) has been passed
    assert m.get("a").tables[1] == [RELEASED, 1, 2, 3] and m.get("a").tables[0] == [0, 1, 2, 3]
    for _ in range(60):
        m.reserve("a", 1)
        m.commit("a", 1)
        m.check()
    t = m.get("a").tables
    assert len(t[0]) == 12 and RELEASED not in t[0]
    held = [p for p in t[1] if p != RELEASED]
    assert len(held) <= 4 and len(t[1]) == 12     # the window of 20 never needs more than 4 pages of 8
    assert m.pools[1].n_free >= 1
    m.release("a")
    assert m.stats()["pages_free"] == [16, 5]


def test_a_window_group_can_run_on_fewer_pages_than_the_sequence_needs():
    lay = CacheLayout.plan([WIN], [None])
    m = CacheManager(lay, page_size=4, num_pages=7, num_slots=0, max_length=1000)
    m.admit("a")
    for _ in range(500):                      # 500 tokens through 7 pages of 4
        m.reserve("a", 1)
        m.commit("a", 1)
    m.check()


def test_commit_beyond_reserved_is_refused():
    m = CacheManager(lfm2_like(), page_size=4, num_pages=4, num_slots=1, max_length=64)
    m.admit("a")
    m.reserve("a", 4)
    with pytest.raises(InvalidPlan):
        m.commit("a", 5)


def test_slot_is_fresh_on_every_admission():
    m = CacheManager(lfm2_like(), page_size=4, num_pages=4, num_slots=1, max_length=64)
    m.admit("a")
    m.fresh_slots.clear()                    # the engine has zeroed it
    m.release("a")
    m.admit("b")
    assert m.get("b").slot == 0 and m.fresh_slots == [0]    # the same slot, to be zeroed again
    m.release("b")
    assert m.fresh_slots == []


@settings(max_examples=60, deadline=None)
@given(st.integers(0, 2 ** 31), st.integers(2, 9), st.integers(6, 40), st.integers(1, 5))
def test_random_orders_of_requests(seed, page_size, num_pages, num_slots):
    rng = random.Random(seed)
    lay = CacheLayout.plan([CONV, FULL, PagedKV(1, 32, 11), FULL], [None, None, None, None])
    m = CacheManager(lay, page_size=page_size, num_pages=[num_pages, max(2, num_pages // 2)], num_slots=num_slots,
                     max_length=200)
    live, n = {}, 0
    for _ in range(300):
        op = rng.random()
        if op < 0.25:
            try:
                m.admit(n)
                live[n] = 0
            except OutOfSlots:
                assert len(live) == num_slots
            n += 1
        elif op < 0.85 and live:
            rid = rng.choice(list(live))
            k = rng.choice((1, 1, 1, 2, 5, 13))
            before = (m.stats()["pages_free"], [list(t) for t in m.get(rid).tables])
            try:
                m.reserve(rid, k)
                m.commit(rid, k)
                live[rid] += k
            except (OutOfPages, ResourceLimit):
                assert (m.stats()["pages_free"], m.get(rid).tables) == before
        elif live:
            rid = rng.choice(list(live))
            m.release(rid)
            del live[rid]
        m.check()
        for rid, length in live.items():
            rc = m.get(rid)
            assert rc.length == length
            assert all(len(t) >= -(-length // page_size) for t in rc.tables)
    for rid in list(live):
        m.release(rid)
    m.check()
    assert m.stats()["pages_free"] == [num_pages, max(2, num_pages // 2)] and m.stats()["slots_free"] == num_slots


def test_keys_and_values_of_different_widths_get_pools_of_their_own():
    """A mixer may keep values wider or narrower than its keys, or none at all (one cached row per token): its layers
    form a group apart from layers with equal widths, and the storage gives the group a key pool and a value pool of
    the widths asked for, addressed by the same page ids."""
    import torch
    from gesso_amd.cache.storage import CacheStorage
    wide = PagedKV(2, 16, None, value_dim=40)
    latent = PagedKV(1, 24, None, value_dim=0)
    lay = CacheLayout.plan([FULL, wide, CONV, latent, wide, FULL], [None] * 6)
    assert [g.need for g in lay.paged] == [FULL, wide, latent] and [g.members for g in lay.paged] == [(0, 5), (1, 4), (3,)]
    st_ = CacheStorage(lay, page_size=4, num_pages=[5, 6, 7], num_slots=2, dtype=torch.float32, device="cpu")
    assert st_.keys[0].shape == (2, 6, 2, 4, 16) and st_.values[0].shape == (2, 6, 2, 4, 16)
    assert st_.keys[1].shape == (2, 7, 2, 4, 16) and st_.values[1].shape == (2, 7, 2, 4, 40)
    assert st_.keys[2].shape == (1, 8, 1, 4, 24) and st_.values[2].shape == (1, 8, 1, 4, 0)
    tables = [torch.zeros(1, 2, dtype=torch.int32)] * 3
    v = st_.view(4, tables)
    assert v.k.shape == (7, 2, 4, 16) and v.v.shape == (7, 2, 4, 40) and v.write
    assert v.k.data_ptr() == st_.keys[1][1].data_ptr()
    assert st_.view(3, tables).v.numel() == 0
    assert st_.bytes() == 4 * sum(t.numel() for t in st_.keys + st_.values) + 4 * sum(
        t.numel() for d in st_.state.values() for t in d.values())
