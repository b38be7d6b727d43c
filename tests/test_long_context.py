"""A long sequence that crosses the real boundaries: attention chunks of 8192 (rotary layers),
the temperature's steps at multiples of 8192 (NoPE layers), llama3 frequency scaling with
factor 16 over an original length of 8192, and hundreds of pages per request.  Tiny widths, so
that the plain implementation can hold the whole score matrix (it runs on the GPU here, being
plain PyTorch).  The prompt is fed in portions of 2,048 tokens, then token by token."""
import pytest
import torch

import traces
from jax_llm_examples_amd.config import get_architecture
from jax_llm_examples_amd.engine.replay import make_runner
from jax_llm_examples_amd.weights import write_random_model
from plain_llama4 import PlainModel

pytestmark = pytest.mark.gpu

CONFIG = {
    "architectures": ["Llama4ForCausalLM"],
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 32,
    "interleave_moe_layer_step": 1, "num_local_experts": 4, "num_experts_per_tok": 1, "intermediate_size": 64,
    "intermediate_size_mlp": 64, "vocab_size": 300, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 16.0, "low_freq_factor": 1.0, "high_freq_factor": 1.0,
                     "original_max_position_embeddings": 8192},
    "no_rope_layers": [1, 0], "attention_chunk_size": 8192, "use_qk_norm": True, "attn_temperature_tuning": True,
    "floor_scale": 8192, "attn_scale": 0.1, "rms_norm_eps": 1e-5, "tie_word_embeddings": False,
}
T = 16500


def _plain_on_gpu(folder, toks, forced, dtype):
    """The plain model on the GPU (plain PyTorch all the same).  In float64 it is the yardstick of the float32
    engine: everything exact but the rotation angles, which the reference forms in float32."""
    import plain_llama4
    plain = PlainModel(folder, dtype)
    plain.w = {k: v.cuda() for k, v in plain.w.items()}
    prev = torch.get_default_device()
    torch.set_default_device("cuda")
    plain_llama4.ANGLES_IN_FLOAT32 = True
    try:
        forced = {li: ids.cuda() for li, ids in forced.items()} if forced else None
        return plain.logits(toks, forced=forced).float().cpu()
    finally:
        plain_llama4.ANGLES_IN_FLOAT32 = False
        torch.set_default_device(prev)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sixteen_thousand_tokens(tmp_path, dtype):
    arch = get_architecture("Llama4ForCausalLM")
    folder = write_random_model(arch, arch.parse_config(CONFIG), str(tmp_path / "m"), seed=3,
                                dtype=torch.float32 if dtype == "float32" else torch.bfloat16)
    toks = torch.randint(0, 300, (T,), generator=torch.Generator().manual_seed(1)).tolist()
    steps, o = [], 0
    while o < T - 40:
        n = min(2048, T - 40 - o)
        steps.append({"step": len(steps), "entries": [{"id": "a", "tokens": toks[o:o + n], "want": list(range(n))}],
                      "end": []})
        o += n
    for i in range(o, T):
        steps.append({"step": len(steps), "entries": [{"id": "a", "tokens": toks[i:i + 1], "want": [0]}],
                      "end": ["a"] if i == T - 1 else []})
    runner = make_runner(folder, dtype, T + 64, "cuda:0", poison=True)
    got, routes = traces.run_trace(runner, steps, record_routing=True)
    got = got["a"]
    assert all(g.pool.num_held == 0 for g in runner.cache.groups)
    # (float32 against the plain model in float64: nothing of the engine's arithmetic is shared)
    ref = _plain_on_gpu(folder, toks, routes["a"] if dtype == "bfloat16" else None,
                        torch.float64 if dtype == "float32" else torch.float32)
    assert torch.isfinite(got).all()
    err = (got - ref).abs().max(dim=-1).values / ref.abs().max()
    tol = 5e-5 if dtype == "float32" else 2e-2
    bad = (err > tol).nonzero().squeeze(-1).tolist()
    assert not bad, f"first wrong position {bad[0]} (of {len(bad)}), error {float(err[bad[0]]):.3g}"
    # the boundaries matter: a model that ignored the chunk or the temperature step would differ there
    for p in (8191, 8192, 16383, 16384, T - 1):
        assert err[p] <= tol


def test_serving_widths_float32_mixed_batches_across_the_chunk_boundaries(wide_model_dir_f32):
    """The layer sizes that serving runs at, in float32, with three requests of up to 16,500 tokens: prompts
    fed in portions of 2,048 tokens while other requests decode in the same steps; positions 8191 / 8192 and
    16383 / 16384 (the chunk's edge on the rotary layer, the temperature's step on the other) are crossed
    inside a portion by some requests and by single tokens by others; the page pools are so small that pages a
    chunk has released are taken by another request; freed pages are poisoned.  Against the plain model in
    float64."""
    folder = wide_model_dir_f32
    V = 20008
    g = torch.Generator().manual_seed(21)
    lengths = {"a": 16500, "b": 8300, "c": 16420}
    toks = {r: torch.randint(0, V, (n,), generator=g).tolist() for r, n in lengths.items()}
    # per request: its cuts.  a: portions (8192 inside one), then single tokens across 16384.
    # b: starts when a is at 4048; portions to 8150, single tokens across 8192.
    # c: portions to 8180, single tokens across 8192, portions again with 16384 inside one.
    def cuts(total, plan):
        out, o = [], 0
        for kind, upto in plan:
            upto = min(upto, total)
            while o < upto:
                n = 1 if kind == "single" else min(2048, upto - o)
                out.append((o, n))
                o += n
        assert o == total
        return out
    plans = {"a": cuts(16500, [("portion", 2000), ("portion", 16340), ("single", 16500)]),
             "b": cuts(8300, [("portion", 8150), ("single", 8300)]),
             "c": cuts(16420, [("portion", 8180), ("single", 8200), ("portion", 16420)])}
    start_step = {"a": 0, "b": 2, "c": 3}
    steps, at, budget = [], {r: 0 for r in plans}, 2048 + 64
    want_rows = {r: set() for r in plans}
    while any(at[r] < len(plans[r]) for r in plans):
        entries, end, left = [], [], budget
        order = sorted(plans, key=lambda r: plans[r][at[r]][1] if at[r] < len(plans[r]) else 0)  # single tokens first
        for r in order:
            if at[r] >= len(plans[r]) or len(steps) < start_step[r]:
                continue
            o, n = plans[r][at[r]]
            if n > left:
                continue
            left -= n
            want = list(range(n)) if n == 1 else sorted(
                {i for i in range(n) if (o + i) % 97 == 0 or any(abs(o + i - b) <= 2 for b in (8191, 16383))} | {n - 1})
            entries.append({"id": r, "tokens": toks[r][o:o + n], "want": want})
            want_rows[r].update(o + i for i in want)
            at[r] += 1
            if at[r] == len(plans[r]):
                end.append(r)
        steps.append({"step": len(steps), "entries": entries, "end": end})
    assert any(len(s["entries"]) >= 2 and {len(e["tokens"]) for e in s["entries"]} >= {1, 2048} for s in steps)
    from jax_llm_examples_amd.cache import CacheManager, pool_sizes
    from jax_llm_examples_amd.engine import ModelRunner, get_ops, load_model
    model = load_model(folder, "float32", "cuda:0")
    needs = model.cache_needs()
    # the group that keeps everything gets what the three requests hold at most; the chunked one only what its
    # rule can hold (a chunk and a portion each): there the pages that one request gives back go to another
    sizes = pool_sizes(needs, page_size=16, itemsize=4, max_requests=3, max_step_tokens=2048,
                       cache_tokens=sum(lengths.values()) + 3 * 64)
    cache = CacheManager(needs, page_size=16, num_pages=sizes, max_requests=3, dtype=torch.float32, device="cuda:0",
                         poison=True)
    runner = ModelRunner(model, cache, get_ops("cuda:0"))
    rows = {r: {} for r in plans}
    pos = {r: 0 for r in plans}
    from jax_llm_examples_amd.engine import StepEntry
    for s in steps:
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]]).float().cpu()
        o = 0
        for e in s["entries"]:
            for w in e["want"]:
                rows[e["id"]][pos[e["id"]] + w] = logits[o]
                o += 1
            pos[e["id"]] += len(e["tokens"])
        for rid in s["end"]:
            runner.finish(rid)
    cache.check()
    assert all(g_.pool.num_held == 0 for g_ in cache.groups)
    chunked = [g_ for g_ in cache.groups if g_.retention[0] == "chunk"][0]
    assert chunked.pool.handed_out > chunked.pool.num_pages  # released pages were used again
    assert runner.graphs is not None and runner.graphs.replays > 0  # steps of single tokens alone were replays
    for r in plans:
        ref = _plain_on_gpu(folder, toks[r], None, torch.float64)
        idx = sorted(rows[r])
        assert {8191, 8192}.issubset(idx) and (lengths[r] < 16385 or {16383, 16384}.issubset(idx))
        got = torch.stack([rows[r][i] for i in idx])
        assert torch.isfinite(got).all(), f"{r}: non-finite logits (a page that was given back?)"
        err = (got - ref[idx]).abs().max(dim=-1).values / ref.abs().max()
        bad = (err > 5e-5).nonzero().squeeze(-1).tolist()
        assert not bad, f"{r}: first wrong position {idx[bad[0]]} (of {len(bad)}), error {float(err[bad[0]]):.3g}"
