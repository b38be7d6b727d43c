import random

import pytest
import torch

from jax_llm_examples_amd.cache import CacheManager, OutOfPages, OutOfSlots, PagePool, SlotPool
from jax_llm_examples_amd.parts.base import CacheNeed, first_needed_position


def test_page_pool_all_or_nothing_and_lifo():
    p = PagePool(5)
    a = p.alloc(3)
    with pytest.raises(OutOfPages):
        p.alloc(3)
    assert p.num_free == 2  # nothing was taken
    p.release([a[1]])
    assert p.alloc(1) == [a[1]]  # the page given back last is used again first
    with pytest.raises(AssertionError, match="twice"):
        p.release([a[0], a[0]])
    p.check()


def test_slot_pool():
    s = SlotPool(2)
    a, b = s.alloc(), s.alloc()
    with pytest.raises(OutOfSlots):
        s.alloc()
    s.release(a)
    assert s.alloc() == a
    with pytest.raises(AssertionError):
        s.release(b), s.release(b)


def _needs():
    return {0: CacheNeed(kv=(2, 8), retention=("chunk", 20)), 1: CacheNeed(kv=(2, 8), retention=("all",)),
            2: CacheNeed(kv=(2, 8), retention=("chunk", 20)), 3: CacheNeed(kv=(2, 8), retention=("window", 9)),
            4: CacheNeed(kv=None, state_shape=(3, 4), state_dtype=torch.float32)}


def _manager(pages=12, ps=8, reqs=3):
    return CacheManager(_needs(), page_size=ps, num_pages=pages, max_requests=reqs, dtype=torch.float32, device="cpu")


def test_groups_by_need_and_state_slots():
    m = _manager()
    assert [(g.retention, g.cache_ids) for g in m.groups] == [(("chunk", 20), [0, 2]), (("all",), [1]),
                                                               (("window", 9), [3])]
    assert m.state[4].shape == (3, 3, 4) and 4 not in m.group_of
    assert m.groups[0].tensors[0].shape == (12, 2, 2, 8, 8)
    e = m.add_request("a")
    m.state[4][e.slot] += 1
    m.free("a")
    assert m.add_request("b").slot == e.slot and float(m.state[4][e.slot].abs().sum()) == 0  # slot reused, cleared


def _visible(retention, q):
    return set(range(first_needed_position(retention, q), q + 1))


def test_release_never_frees_a_page_a_later_query_reads_and_frees_all_others():
    """Brute force against the mask's definition, with steps of changing size."""
    rng = random.Random(1)
    ps = 8
    m = _manager(pages=40, ps=ps)
    m.add_request("a")
    n = 0
    while n < 150:
        k = rng.choice([1, 1, 2, 3, 7, 19, 30])
        m.reserve("a", k)
        for g in m.groups:  # during the step every query of the portion finds its keys
            for q in range(n, n + k):
                for kp in _visible(g.retention, q):
                    assert m.table("a", g.index)[kp // ps] >= 0
        m.commit("a")
        n += k
        for g in m.groups:
            later = set()
            for q in range(n, n + 200):
                later |= {kp // ps for kp in _visible(g.retention, q) if kp < n}
            table = m.table("a", g.index)
            held = {j for j, p in enumerate(table) if p >= 0}
            assert later <= held, "a page some later query reads was given back"
            assert held == later | ({(n - 1) // ps} if g.retention[0] != "all" and not later else set()) or held == later | {(n - 1) // ps} or held == later
            # nothing older than what can be read is kept
            assert all(j >= first_needed_position(g.retention, n) // ps for j in held)
        m.check()
    m.free("a")
    assert all(g.pool.num_free == 40 for g in m.groups)


def test_random_orders_no_page_lost_held_twice_or_freed_twice():
    rng = random.Random(7)
    m = _manager(pages=24, ps=8, reqs=4)
    live, n_ok, n_full = {}, 0, 0
    for it in range(600):
        r = rng.random()
        if r < 0.25 and len(live) < 4:
            rid = f"q{it}"
            m.add_request(rid)
            live[rid] = 0
        elif r < 0.85 and live:
            rid = rng.choice(list(live))
            k = rng.choice([1, 1, 1, 2, 5, 17, 40])
            before = m.num_free_pages()
            try:
                m.reserve(rid, k)
            except OutOfPages:
                n_full += 1
                assert m.num_free_pages() == before  # nothing was taken
            else:
                n_ok += 1
                if rng.random() < 0.1:
                    m.cancel(rid)
                else:
                    m.commit(rid)
                    live[rid] += k
                assert m.num_tokens(rid) == live[rid]
        elif live:
            rid = rng.choice(list(live))
            m.free(rid)
            del live[rid]
        m.check()
    assert n_ok > 50 and n_full > 5
    for rid in list(live):
        m.free(rid)
    m.check()
    assert all(g.pool.num_free == 24 for g in m.groups) and m.slots.num_free == 4
    with pytest.raises(KeyError):
        m.free("q0")


def test_cancel_gives_back_only_the_reservation():
    m = _manager()
    m.add_request("a")
    m.reserve("a", 10)
    m.commit("a")
    free = m.num_free_pages()
    m.reserve("a", 30)
    assert m.num_free_pages() != free
    m.cancel("a")
    assert m.num_free_pages() == free and m.num_tokens("a") == 10
    m.reserve("a", 3)
    m.commit("a")
    m.check()


def test_pages_needed_matches_what_reserve_takes():
    m = _manager(pages=30)
    m.add_request("a")
    for k in (5, 3, 1, 20, 8, 1):
        need = m.pages_needed("a", k)
        before = m.num_free_pages()
        m.reserve("a", k)
        assert [b - a for a, b in zip(m.num_free_pages(), before)] == need
        m.commit("a")
    assert m.pages_needed_new(17) == [3, 3, 3]
