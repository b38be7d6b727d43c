import random

import torch

from jax_llm_examples_amd.cache import CacheManager
from jax_llm_examples_amd.engine.scheduler import FINISHED, Request, Scheduler, SchedulerConfig
from jax_llm_examples_amd.parts.base import CacheNeed
from jax_llm_examples_amd.sampling import SamplingParams


def _cache(pages, reqs=8, ps=4):
    needs = {0: CacheNeed(kv=(1, 8), retention=("all",)), 1: CacheNeed(kv=(1, 8), retention=("chunk", 12))}
    return CacheManager(needs, page_size=ps, num_pages=pages, max_requests=reqs, dtype=torch.float32, device="cpu")


def _drive(s, cache, on_plan=None, max_steps=10000):
    """Stands in for the model: reserves and commits what the plan says, 'samples' a counter."""
    done, tok = [], 1000
    for _ in range(max_steps):
        if not s.has_work():
            break
        plan = s.schedule()
        done += plan.dropped
        if on_plan:
            on_plan(plan)
        for seg in plan.segments:
            rid = seg.request.id
            if not cache.has_request(rid):
                cache.add_request(rid)
            assert seg.start == cache.num_tokens(rid)
            cache.reserve(rid, seg.count)  # must never raise: the scheduler has checked
        for seg in plan.segments:
            cache.commit(seg.request.id)
        sampled = []
        for seg in plan.segments:
            if seg.samples:
                tok += 1
                sampled.append(tok)
        done += s.update(plan, sampled)
        cache.check()
    return done


def test_budget_fifo_portions_and_every_token_once():
    cache = _cache(pages=200)
    s = Scheduler(SchedulerConfig(max_num_batched_tokens=16, decode_batch_size=3), cache)
    reqs = [Request(i, list(range(n)), SamplingParams(max_decode_length=5)) for i, n in enumerate([40, 7, 23, 5, 30])]
    for r in reqs:
        s.add(r)
    seen = {r.id: [] for r in reqs}
    first_step = {}

    def on_plan(plan):
        assert plan.num_tokens <= 16
        assert len(s.running) <= 3
        for seg in plan.segments:
            seen[seg.request.id].append((seg.start, seg.count))
            first_step.setdefault(seg.request.id, s.stats["steps"])
        # decode tokens are never starved by prompts: every running request in decode phase is in the plan
        in_plan = {seg.request.id for seg in plan.segments}
        for r in s.running:
            if r.num_pending == 1 and r.output:
                assert r.id in in_plan

    done = _drive(s, cache, on_plan)
    assert sorted(r.id for r in done) == [0, 1, 2, 3, 4] and all(r.state == FINISHED for r in reqs)
    assert all(len(r.output) == 5 and r.finish_reason == "length" for r in reqs)
    for r in reqs:  # every token of prompt + output (but the last sampled) computed exactly once, in order
        pos = 0
        for a, n in seen[r.id]:
            assert a == pos
            pos += n
        assert pos == len(r.prompt) + 4
    assert [first_step[i] for i in range(5)] == sorted(first_step[i] for i in range(5))  # first come first served
    assert any(n not in (1, len(r.prompt)) for r in reqs for _, n in seen[r.id])  # prompts were cut
    assert cache.num_live() == 0 and all(f == 200 for f in cache.num_free_pages())


def test_eos_ends_a_request():
    cache = _cache(pages=50)
    s = Scheduler(SchedulerConfig(32, 4), cache)
    r = Request("a", [1, 2, 3], SamplingParams(max_decode_length=50, eos_tokens=(1003,)))
    r2 = Request("b", [1, 2, 3], SamplingParams(max_decode_length=4, eos_tokens=(1003,), ignore_eos=True))
    s.add(r)
    _drive(s, cache)
    assert r.output == [1001, 1002, 1003] and r.finish_reason == "eos"
    s.add(r2)
    _drive(s, cache)
    assert len(r2.output) == 4 and r2.finish_reason == "length"


def test_pages_run_out_the_request_admitted_last_is_preempted_and_computed_again():
    cache = _cache(pages=12, ps=4)  # 48 tokens per group
    s = Scheduler(SchedulerConfig(max_num_batched_tokens=64, decode_batch_size=4), cache)
    a = Request("a", list(range(20)), SamplingParams(max_decode_length=16))
    b = Request("b", list(range(18)), SamplingParams(max_decode_length=16))
    s.add(a), s.add(b)
    events = []

    def on_plan(plan):
        for r in plan.preempted:
            events.append((r.id, len(r.output)))

    done = _drive(s, cache, on_plan)
    assert events and all(rid == "b" for rid, _ in events)  # the one admitted last gives way
    assert b.preemptions >= 1 and a.preemptions == 0
    assert [r.id for r in done] == ["a", "b"]
    assert len(a.output) == 16 and len(b.output) == 16  # what b had generated was kept
    assert b.output == sorted(b.output)
    assert all(f == 12 for f in cache.num_free_pages())


def test_a_request_that_can_never_fit_ends_with_out_of_pages():
    cache = _cache(pages=4, ps=4)  # 16 tokens
    s = Scheduler(SchedulerConfig(64, 4), cache)
    big = Request("big", list(range(30)), SamplingParams(max_decode_length=4))
    grow = Request("grow", list(range(10)), SamplingParams(max_decode_length=40))
    ok = Request("ok", list(range(6)), SamplingParams(max_decode_length=3))
    s.add(big), s.add(grow), s.add(ok)
    done = _drive(s, cache)
    assert big.finish_reason == "out_of_pages" and big.output == []
    assert grow.finish_reason == "out_of_pages" and 0 < len(grow.output) < 40  # grew until the pool was full
    assert ok.finish_reason == "length" and len(ok.output) == 3
    assert {r.id for r in done} == {"big", "grow", "ok"}
    assert all(f == 4 for f in cache.num_free_pages()) and cache.num_live() == 0


def test_random_loads_always_finish_and_free_everything():
    rng = random.Random(3)
    for trial in range(10):
        cache = _cache(pages=rng.randint(10, 40), reqs=5)
        s = Scheduler(SchedulerConfig(rng.choice([8, 16, 33]), rng.randint(1, 5), keep_free_pages=rng.choice([0, 1])),
                      cache)
        reqs = [Request(i, list(range(rng.randint(1, 30))), SamplingParams(max_decode_length=rng.randint(1, 20)))
                for i in range(12)]
        for r in reqs:
            s.add(r)
        done = _drive(s, cache)
        assert len(done) == 12 and not s.has_work()
        assert all(r.finish_reason in ("length", "out_of_pages") for r in reqs)
        assert cache.num_live() == 0 and all(g.pool.num_held == 0 for g in cache.groups)


def test_a_request_ends_at_the_context_limit():
    cache = _cache(pages=200)
    s = Scheduler(SchedulerConfig(max_num_batched_tokens=16, decode_batch_size=3, max_seq_len=30), cache)
    reqs = [Request(0, list(range(25)), SamplingParams(max_decode_length=50)),
            Request(1, list(range(30)), SamplingParams(max_decode_length=50)),
            Request(2, list(range(5)), SamplingParams(max_decode_length=4))]
    for r in reqs:
        s.add(r)
    import pytest
    with pytest.raises(ValueError, match="longer than max_seq_len"):
        s.add(Request(3, list(range(31))))
    _drive(s, cache)
    assert [(len(r.prompt) + len(r.output), r.finish_reason) for r in reqs] == [(30, "length"), (31, "length"),
                                                                                (9, "length")]
    assert max(r.num_computed for r in reqs) <= 30  # no token was ever given a position beyond the limit
    assert cache.num_live() == 0


def test_bench_refuses_more_than_one_gpu():
    """The engine runs on one GPU: ``bench.py --gpus 2`` prints one line that says so and exits with 2."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert p.returncode == 2
    lines = [ln for ln in p.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]
    env = dict(os.environ, WORLD_SIZE="2")
    p = subprocess.run([sys.executable, os.path.join(root, "bench.py")], capture_output=True, text=True, timeout=120,
                       env=env)
    assert p.returncode == 2
