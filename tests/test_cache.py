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


def test_each_group_is_sized_by_what_its_retention_rule_can_hold():
    """A group that lets go of old tokens needs a chunk plus a step's portion per request, whatever the
    context length; sized for the whole context it would take most of the memory for nothing."""
    from jax_llm_examples_amd.cache import pool_sizes, tokens_held_at_most

    # three chunked runs per run that keeps everything, as in the large configuration
    needs = {i: CacheNeed(kv=(8, 128), retention=("all",) if i % 4 == 3 else ("chunk", 8192)) for i in range(8)}
    kw = dict(page_size=16, itemsize=2, max_requests=4, max_step_tokens=2048)
    assert tokens_held_at_most(("chunk", 8192), 2048, None) == 10240
    assert tokens_held_at_most(("window", 100), 7, 60) == 60 and tokens_held_at_most(("all",), 7, None) is None
    sizes = pool_sizes(needs, cache_tokens=4 * 32768, **kw)
    chunked, full = sizes[0], sizes[1]  # groups in order of their first run
    assert full == 4 * 32768 // 16
    assert chunked == 4 * (10240 // 16 + 1) and chunked < full // 3
    # the same memory holds many more tokens of context than with equal pools
    page = 2 * 8 * 128 * 16 * 2
    equal_pools_bytes = 8 * page * full
    budget = equal_pools_bytes // 2
    by_memory = pool_sizes(needs, memory_bytes=budget, **kw)
    assert by_memory[0] == chunked and by_memory[1] * 16 > 32768 * 4
    used = 6 * page * by_memory[0] + 2 * page * by_memory[1]
    assert used <= budget < used + 2 * page  # the largest that fits
    with pytest.raises(ValueError, match="one page"):
        pool_sizes(needs, memory_bytes=100, **kw)
    # a manager built with these sizes: a request of 32,768 tokens fits, fed in portions
    small = {0: CacheNeed(kv=(1, 8), retention=("chunk", 64)), 1: CacheNeed(kv=(1, 8), retention=("all",))}
    sz = pool_sizes(small, page_size=8, itemsize=4, max_requests=2, max_step_tokens=24, cache_tokens=2 * 1000)
    assert sz == {0: 2 * (88 // 8 + 1), 1: 250}
    m = CacheManager(small, page_size=8, num_pages=sz, max_requests=2, dtype=torch.float32, device="cpu")
    for rid in ("a", "b"):
        m.add_request(rid)
    for step in range(41):
        for rid in ("a", "b"):
            m.reserve(rid, 24)  # never out of pages in the small pool
        for rid in ("a", "b"):
            m.commit(rid)
        m.check()
    assert m.num_tokens("a") == 984 and m.groups[0].pool.handed_out > m.groups[0].pool.num_pages


def test_further_per_token_tensors_get_pages_of_their_own_shapes():
    needs = {0: CacheNeed(kv=(2, 8), retention=("all",)),
             1: CacheNeed(paged=(("k", (2, 24)), ("v", (2, 8))), retention=("all",)),
             2: CacheNeed(paged=(("latent", (10,)),), retention=("window", 5)),
             3: CacheNeed(paged=(("k", (2, 24)), ("v", (2, 8))), retention=("all",))}
    m = CacheManager(needs, page_size=4, num_pages={0: 6, 1: 5, 2: 3}, max_requests=2, dtype=torch.bfloat16,
                     device="cpu", poison=True)
    assert [g.cache_ids for g in m.groups] == [[0], [1, 3], [2]]
    assert m.groups[1].pages[3]["k"].shape == (5, 4, 2, 24) and m.groups[1].pages[1]["v"].shape == (5, 4, 2, 8)
    assert m.groups[2].pages[2]["latent"].shape == (3, 4, 10) and not m.groups[2].tensors
    assert m.groups[1].bytes_per_token() == 2 * (48 + 16) * 2 and m.groups[2].bytes_per_token() == 20
    assert m.bytes_per_token() == 2 * 2 * 8 * 2 + 256 + 20
    m.add_request("a")
    m.reserve("a", 9)
    page = m.table("a", 2)[0]
    m.groups[2].pages[2]["latent"][page] = 1.0
    m.commit("a")  # the window has passed the first page: given back and poisoned
    assert m.table("a", 2)[0] == -1 and bool(m.groups[2].pages[2]["latent"][page].isnan().all())
    m.free("a")
    m.check()
