"""A request id that lives twice (ended and started again, by the caller or by a preemption) and
the recorded decode steps: a recording keeps block tables on the device from step to step and
rewrites a row only when the request in it, this life of it, or its tables changed.  The second
life of an id gets other pages than the first while its counts of table changes may be the same,
so what tells a row's content is the cache manager's stamp, which names the life.

The reference re-initialises a decode slot whenever a request takes it
(``serving/serving_jax/serving_loop.py:611-633``)."""
import random

import numpy as np
import pytest
import torch

import traces
from jax_llm_examples_amd import Engine, SamplingParams, load_model
from jax_llm_examples_amd.cache import CacheManager
from jax_llm_examples_amd.engine.batch import StepEntry, StepLayout, fill_step
from jax_llm_examples_amd.engine.replay import make_runner
from jax_llm_examples_amd.parts.base import CacheNeed
from plain_llama4 import PlainModel
from tiny_configs import TINY


def _manager(groups=1, pages=12, ps=8):
    needs = {0: CacheNeed(kv=(1, 8), retention=("all",))}
    if groups > 1:
        needs[1] = CacheNeed(kv=(1, 8), retention=("chunk", 16))
    return CacheManager(needs, page_size=ps, num_pages=pages, max_requests=4, dtype=torch.float32, device="cpu")


def _life(m, rid, prompt, decoded):
    if not m.has_request(rid):
        m.add_request(rid)
    m.reserve(rid, prompt)
    m.commit(rid)
    for _ in range(decoded):
        m.reserve(rid, 1)
        m.commit(rid)


def test_two_lives_of_one_id_with_equal_histories_have_different_stamps():
    m = _manager()
    _life(m, "a", 20, 3)
    _life(m, "b", 5, 0)
    first, table = m.table_stamp("a"), list(m.table("a", 0))
    m.free("a")
    m.reserve("b", 8)  # "b" takes one of the pages that "a" held
    m.commit("b")
    _life(m, "a", 20, 3)
    assert m.requests["a"].versions == list(first[1:])  # the same count of table changes ...
    assert m.table("a", 0) != table  # ... over other pages
    assert m.table_stamp("a") != first
    # and within one life the stamp changes exactly when a table does
    before, t0 = m.table_stamp("a"), list(m.table("a", 0))
    m.reserve("a", 1)
    m.commit("a")
    assert (m.table_stamp("a") == before) == (m.table("a", 0) == t0)


@pytest.mark.parametrize("groups", [1, 2])
def test_a_kept_block_table_follows_the_live_one_through_ends_restarts_and_preemptions(groups):
    """What a recorded step does on the host, without a GPU: one buffer kept from step to step, rows rewritten
    only on a changed stamp; after every step each row equals the live table of the request in it."""
    rng = random.Random(groups)
    m = _manager(groups, pages=40, ps=4)
    R, width = 3, 16
    layout = StepLayout(R, R, R, [width] * groups)
    mirror = np.zeros(layout.size, np.int32)
    stamps = [None] * R
    live = []
    reused = 0
    for step in range(600):
        while len(live) < R:
            rid = rng.choice("abcd")
            if rid in live:
                continue
            _life(m, rid, rng.choice([5, 9, 9, 9, 13]), 0)
            live.append(rid)
        rng.shuffle(live) if rng.random() < 0.1 else None
        entries = [StepEntry(rid, [1], (0,)) for rid in live]
        for rid in live:
            m.reserve(rid, 1)
        before = list(stamps)
        fill_step(layout, mirror, m, entries, vocab_size=8, stamps=stamps)
        for i, rid in enumerate(live):
            for g in m.groups:
                row = layout.view(mirror, f"block_table{g.index}")[i * width: (i + 1) * width].tolist()
                table = m.table(rid, g.index)
                assert row == table + [-1] * (width - len(table)), (step, rid, g.index)
            reused += before[i] == stamps[i]
        for rid in live:
            m.commit(rid)
        for rid in list(live):
            if m.num_tokens(rid) >= 40 or rng.random() < 0.08:  # ends (or is preempted: the same to the cache)
                m.free(rid)
                live.remove(rid)
    assert reused > 200  # most rows were kept as they were: the test did exercise the stamps


# ----------------------------------------------------------------------------------------------- on the GPU
def _rows(runner, entries):
    return runner.step([StepEntry(*e) for e in entries]).float().cpu().clone()


def _id_reuse_trace(runner, a1, b, a2):
    """"a" decodes beside "b" and ends; "b" takes its pages; a new "a" of the same length arrives and decodes
    beside "b" again.  Returns the logits of both lives of "a" and of "b", by position."""
    out = {"a1": {}, "a2": {}, "b": {}}

    def run(entries, names):
        logits = _rows(runner, entries)
        o = 0
        for (rid, toks, want), name in zip(entries, names):
            start = runner.cache.num_tokens(rid) - len(toks)
            for w in want:
                out[name][start + w] = logits[o]
                o += 1

    n1, nb = len(a1) - 6, 5
    run([("a", a1[:n1], [n1 - 1]), ("b", b[:nb], [nb - 1])], ["a1", "b"])
    pb = nb
    for i in range(n1, len(a1)):  # steps of two single tokens: recorded when they come the second time
        run([("a", [a1[i]], [0]), ("b", [b[pb]], [0])], ["a1", "b"])
        pb += 1
    runner.finish("a")
    grow = 2 * runner.cache.page_size
    run([("b", b[pb: pb + grow], [grow - 1])], ["b"])  # "b" takes pages that "a" gave back
    pb += grow
    n2 = len(a2) - 6
    run([("a", a2[:n2], [n2 - 1])], ["a2"])
    for i in range(n2, len(a2)):
        run([("a", [a2[i]], [0]), ("b", [b[pb]], [0])], ["a2", "b"])
        pb += 1
    runner.finish("a")
    runner.finish("b")
    return out, pb


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_an_id_that_lives_twice_reads_its_own_pages(model_dirs, model_dirs_bf16, name, dtype):
    folder = (model_dirs if dtype == "float32" else model_dirs_bf16)[name]
    plain = PlainModel(folder)
    V = plain.cfg["vocab_size"]
    g = torch.Generator().manual_seed(21)
    a1, a2 = (torch.randint(0, V, (26,), generator=g).tolist() for _ in range(2))
    b = torch.randint(0, V, (64,), generator=g).tolist()
    got = {}
    for graphs in (False, True):
        runner = make_runner(folder, dtype, 128, "cuda:0", poison=True, decode_graphs=graphs)
        got[graphs], used = _id_reuse_trace(runner, a1, b, a2)
        if graphs:
            assert runner.graphs.replays >= 8
        runner.cache.check()
    for key in got[True]:
        for pos in got[True][key]:
            assert torch.equal(got[True][key][pos], got[False][key][pos]), (key, pos)
    tol = 2e-5 if dtype == "float32" else 3e-2
    for key, toks in (("a1", a1), ("a2", a2), ("b", b[:used])):
        ref = plain.logits(toks).float()
        for pos, row in got[True][key].items():
            assert torch.isfinite(row).all(), (key, pos)
            assert float((row - ref[pos]).abs().max() / ref.abs().max()) < tol, (key, pos)


ONE_GROUP = dict(TINY["A"], no_rope_layers=[1, 1, 1, 1], attention_chunk_size=4096, seed=71)  # every layer keeps all


@pytest.mark.gpu
def test_preempted_requests_come_back_under_their_ids_with_recorded_steps(tmp_path):
    """One retention group, so that a second life's count of table changes can equal the first's; a pool so
    small that requests are preempted again and again while the others' steps of single tokens are replays."""
    from jax_llm_examples_amd.config import get_architecture
    from jax_llm_examples_amd.weights import write_random_model
    top = {k: v for k, v in ONE_GROUP.items() if k != "seed"}
    arch = get_architecture(top["architectures"][0])
    folder = write_random_model(arch, arch.parse_config(top), str(tmp_path / "G"), ONE_GROUP["seed"], torch.float32,
                                architecture=top["architectures"][0])
    g = torch.Generator().manual_seed(9)
    prompts = [torch.randint(0, 512, (n,), generator=g).tolist() for n in (30, 28, 25, 31, 18, 27)]
    outs = {}
    for graphs in (False, True):
        eng = Engine(load_model(folder, "float32", "cuda:0"), poison=True, cache_tokens=144, decode_batch_size=3,
                     max_num_batched_tokens=64, decode_graphs=graphs)
        assert len(eng.cache.groups) == 1
        outs[graphs] = eng.generate(prompts, SamplingParams(max_decode_length=40))
        assert eng.scheduler.stats["preemptions"] >= 3
        if graphs:
            assert eng.runner.graphs.replays > 30
        eng.cache.check()
    assert outs[True] == outs[False]
    plain = PlainModel(folder)
    for p, out in zip(prompts, outs[True]):
        seq = list(p)
        for tok in out:
            assert tok == int(plain.logits(seq)[-1].argmax())
            seq.append(tok)


@pytest.mark.gpu
def test_logits_held_by_a_caller_outlive_the_recording_they_came_from(model_dirs):
    """More (requests, context bound) pairs than recordings are kept: the oldest recording goes while the
    caller still holds logits that lay in its buffer."""
    from jax_llm_examples_amd.engine.decode_graph import DecodeGraphs
    folder = model_dirs["A"]
    runner = make_runner(folder, "float32", 4096, "cuda:0", max_requests=24, decode_graphs=True)
    g = torch.Generator().manual_seed(2)
    rids = [f"q{i}" for i in range(DecodeGraphs.MAX_RECORDINGS + 4)]
    for rid in rids:
        runner.step([StepEntry(rid, torch.randint(0, 512, (9,), generator=g).tolist(), [])])
    held = []
    for n in range(1, len(rids) + 1):  # steps of 1, 2, 3, ... requests: each count a recording of its own
        entries = [StepEntry(rid, [int(torch.randint(0, 512, (1,), generator=g))], [0]) for rid in rids[:n]]
        for _ in range(DecodeGraphs.RECORD_AFTER + 1):
            logits = runner.step(entries)
        held.append((logits, logits.clone()))
    assert runner.graphs.captures == len(rids) and len(runner.graphs.recordings) == DecodeGraphs.MAX_RECORDINGS
    torch.cuda.synchronize()
    for kept, copy in held:
        assert torch.equal(kept, copy)
