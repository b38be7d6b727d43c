"""The engine against the plain implementation, for every way of cutting and batching:
each request alone and whole; most of it in one step and the last 32 tokens one by one;
portions of changing size down to two tokens; and mixed, up to four live requests with
portions of some beside single tokens of others and so few pages that they are used again
(the pool is poisoned with NaN, so a stale or foreign page shows).

On the CPU the engine runs with the plain PyTorch ops (this checks cache, batch and step
logic); on the GPU with the HIP kernels, in float32 and bfloat16.  In bfloat16 the plain
implementation is given the engine's expert choices: a near-tie in the router may fall
the other way under rounding, which is no fault; that such flips happen only at near-ties
is checked separately."""
import pytest
import torch

import traces
from jax_llm_examples_amd.engine.replay import make_runner
from plain_llama4 import PlainModel
from tiny_configs import FAST, TINY, write_tiny

LENGTHS = {"A": [1, 80, 33, 47, 64, 9], "B": [120, 2, 49, 96, 31, 77], "C": [61, 40, 5, 83], "D": [37, 70, 3, 55, 64, 21],
           "F": [300, 40, 170, 33], "W": [700, 33, 260, 48], "M": [2100, 33, 260, 48]}
MODES = {"whole": traces.whole, "tail": traces.tail, "portions": traces.portions, "mixed": traces.mixed}
TOL = {"float32": 2e-5, "bfloat16": 1.5e-2}  # of the largest logit of the request


def _vocab(name):
    c = {**TINY, **FAST}[name]
    return c.get("text_config", c)["vocab_size"]


def _check(name, folder, dtype, device, mode, reference_ops, plain_device="cpu", record=True,
           plain_dtype=torch.float32, lengths=None, max_requests=8, page_size=16):
    """``record``: watch every step for the experts it chose (a watched step is never the replay of a recorded
    graph); without it, steps of single tokens go through the recorded decode graphs."""
    if lengths is None:
        lengths = LENGTHS[name] + (LENGTHS[name][::-1] + LENGTHS[name] if mode == "mixed" else [])
    reqs = traces.random_requests(_vocab(name), lengths, seed=5)
    steps = MODES[mode](reqs) if isinstance(mode, str) else mode(reqs)
    runner = make_runner(folder, dtype, traces.max_live_tokens(steps), device, reference_ops=reference_ops,
                         poison=True, max_requests=max_requests, page_size=page_size)
    if record:
        got, routes = traces.run_trace(runner, steps, record_routing=True)
    else:
        got, routes = traces.run_trace(runner, steps), {}
        assert runner.graphs is not None and runner.graphs.replays > 0 and runner.graphs.captures > 0
    if mode == "mixed" or not isinstance(mode, str):  # so few pages that they were used again
        assert all(g.pool.handed_out > g.pool.num_pages for g in runner.cache.groups)
    runner.cache.check()
    assert runner.cache.num_live() == 0 and all(g.pool.num_held == 0 for g in runner.cache.groups)
    import plain_llama4
    plain = PlainModel(folder, plain_dtype)
    plain_llama4.ANGLES_IN_FLOAT32 = plain_dtype == torch.float64  # (the yardstick of a float32 run: see there)
    one_by_one = plain_llama4.TOKENS_ONE_BY_ONE
    if plain_device != "cpu":
        plain_llama4.TOKENS_ONE_BY_ONE = 48  # (on the GPU a loop over tokens costs a launch per step: by expert sooner)
    if plain_device != "cpu":  # (plain PyTorch all the same; the wide configuration would take minutes on the CPU)
        plain.w = {k: v.to(plain_device) for k, v in plain.w.items()}
    worst = 0.0
    for rid, toks in reqs.items():
        forced = routes.get(rid) if dtype == "bfloat16" else None
        info = {}
        if plain_device != "cpu":
            prev = torch.get_default_device()
            torch.set_default_device(plain_device)
            try:
                forced = {li: ids.to(plain_device) for li, ids in forced.items()} if forced else forced
                ref = plain.logits(toks, forced=forced, info=info).float().cpu()
                info = {li: (idx.cpu(), sc.cpu()) for li, (idx, sc) in info.items()}
            finally:
                torch.set_default_device(prev)
        else:
            ref = plain.logits(toks, forced=forced, info=info).float()
        assert got[rid].shape == ref.shape
        assert torch.isfinite(got[rid]).all(), f"{rid}: non-finite logits (a page that was given back?)"
        err = (got[rid] - ref).abs().max(dim=-1).values / ref.abs().max()
        bad = (err > TOL[dtype]).nonzero().squeeze(-1).tolist()
        assert not bad, f"{name} {dtype} {mode} {rid}: first wrong position {bad[0]} of {len(toks)}, error {err[bad[0]]:.3g}"
        worst = max(worst, float(err.max()))
        if dtype == "float32" and rid in routes:  # float32: the same experts, always
            for li, (idx, _) in info.items():
                assert torch.equal(routes[rid][li].long(), idx), f"{rid} layer {li}: expert choice differs"
    plain_llama4.ANGLES_IN_FLOAT32 = False
    plain_llama4.TOKENS_ONE_BY_ONE = one_by_one
    return worst


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("name", list(TINY))
def test_cpu_plain_ops_float32(model_dirs, name, mode):
    _check(name, model_dirs[name], "float32", "cpu", mode, reference_ops=True)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("name", list(TINY))
def test_gpu_float32(model_dirs, name, mode):
    _check(name, model_dirs[name], "float32", "cuda:0", mode, reference_ops=False)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["tail", "mixed"])
@pytest.mark.parametrize("name", list(TINY))
def test_gpu_float32_with_recorded_decode_steps(model_dirs, name, mode):
    """The same comparison with the steps of single tokens replayed from recorded HIP graphs."""
    _check(name, model_dirs[name], "float32", "cuda:0", mode, reference_ops=False, record=False)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "F"])
def test_recorded_decode_steps_equal_unrecorded_ones_bit_for_bit(model_dirs, model_dirs_bf16, tmp_path, name, dtype):
    """Replays and launch-by-launch steps run the same kernels with the same arguments.  Between the replays lie
    the trace's other steps (portions of prompts, launch by launch) and a synchronisation after every step."""
    if name == "F":
        folder = write_tiny("F", str(tmp_path / "F"), torch.bfloat16)
    else:
        folder = (model_dirs if dtype == "float32" else model_dirs_bf16)[name]
    lengths = LENGTHS[name]
    reqs = traces.random_requests(_vocab(name), lengths + lengths[::-1], seed=8)
    for mode in ("tail", "mixed"):
        steps = MODES[mode](reqs)
        out = {}
        for graphs in (False, True):
            runner = make_runner(folder, dtype, traces.max_live_tokens(steps), "cuda:0", poison=True,
                                 decode_graphs=graphs)
            out[graphs] = traces.run_trace(runner, steps)
            if graphs:
                assert runner.graphs.replays > 20 and 0 < runner.graphs.captures < runner.graphs.replays
            else:
                assert runner.graphs is None
        for rid in reqs:
            assert torch.equal(out[True][rid], out[False][rid]), (mode, rid)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("name", list(TINY))
def test_gpu_bfloat16(model_dirs_bf16, name, mode):
    _check(name, model_dirs_bf16[name], "bfloat16", "cuda:0", mode, reference_ops=False)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", list(MODES))
def test_gpu_bfloat16_sizes_of_the_fast_kernels(tmp_path_factory, mode, monkeypatch):
    """The tiny configurations are too small for the kernels that serving sizes get (keys shared between the
    query heads of a kv head, expert matrices in the streaming layout, the weight-streaming grouped product
    in prefill): this one is not."""
    folder = write_tiny("F", str(tmp_path_factory.mktemp("models_fast") / "F"), torch.bfloat16)
    runner = make_runner(folder, "bfloat16", 1024, "cuda:0")
    moe = [b.feed_forward for b in runner.model.blocks]
    assert all(ff.tiled for ff in moe), "the expert matrices of this configuration fit the streaming layout"
    from jax_llm_examples_amd.ops.hip import HipOps
    calls = {"stream": 0}
    inner = HipOps.gemm_stream

    def counted(self, *a, **kw):
        calls["stream"] += 1
        return inner(self, *a, **kw)

    monkeypatch.setattr(HipOps, "gemm_stream", counted)
    _check("F", folder, "bfloat16", "cuda:0", mode, reference_ops=False)
    if mode in ("whole", "tail"):  # the other modes cut the prompts into portions too short for it
        assert calls["stream"] > 0, "no step went through the weight-streaming grouped product"


@pytest.fixture(scope="module")
def wide_model_dir(tmp_path_factory):
    return write_tiny("W", str(tmp_path_factory.mktemp("models_wide") / "W"), torch.bfloat16)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", list(MODES))
def test_gpu_bfloat16_serving_widths(wide_model_dir, mode):
    """Two layers (one rotary, one without) at the widths the benchmark runs: the kernel variants that only these
    sizes reach (rows of 5120, 40 heads on 8, experts 8192 wide) against the plain implementation."""
    _check("W", wide_model_dir, "bfloat16", "cuda:0", mode, reference_ops=False, plain_device="cuda:0")


@pytest.fixture(scope="module")
def many_experts_model_dir(tmp_path_factory):
    return write_tiny("M", str(tmp_path_factory.mktemp("models_many_experts") / "M"), torch.bfloat16)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", list(MODES))
def test_gpu_bfloat16_many_experts_on_alternate_layers(many_experts_model_dir, mode):
    """The larger model's shapes (``llama4/llama4_jax/configs.py:57-93``): a dense layer 16,384 wide, then a layer
    of 128 experts (129 groups with the shared expert riding in their launches) at serving widths.  A prompt of
    2,100 tokens gives every expert about 16 rows, some none; steps of a few tokens leave most experts empty."""
    runner = make_runner(many_experts_model_dir, "bfloat16", 64, "cuda:0")
    kinds = [type(b.feed_forward).__name__ for b in runner.model.blocks]
    assert kinds == ["DenseSwiGLU", "MoESigmoidShared"] and runner.model.blocks[1].feed_forward.tiled
    del runner
    _check("M", many_experts_model_dir, "bfloat16", "cuda:0", mode, reference_ops=False, plain_device="cuda:0")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sixty_four_live_requests_with_many_experts(many_experts_model_dir, many_experts_model_dir_f32, dtype):
    """64 live requests over 128 experts and a dense layer: steps of 64 single tokens (recorded in float32, where
    the yardstick is the plain model in float64) beside portions of up to 300 tokens."""
    folder = many_experts_model_dir if dtype == "bfloat16" else many_experts_model_dir_f32
    g = torch.Generator().manual_seed(13)
    lengths = torch.randint(60, 200, (64,), generator=g).tolist()
    lengths[5] = 1100
    mode = lambda reqs: traces.mixed(reqs, seed=4, max_live=64, decode_tail=16, max_portion=300)
    _check("M", folder, dtype, "cuda:0", mode, reference_ops=False, plain_device="cuda:0",
           record=dtype == "bfloat16", plain_dtype=torch.float64 if dtype == "float32" else torch.float32,
           lengths=lengths, max_requests=64)


@pytest.mark.gpu
def test_gpu_float32_many_experts_mixed(many_experts_model_dir_f32):
    _check("M", many_experts_model_dir_f32, "float32", "cuda:0", "mixed", reference_ops=False, plain_device="cuda:0",
           plain_dtype=torch.float64, lengths=[700, 33, 260, 48, 48, 260, 33, 700])


@pytest.mark.gpu
@pytest.mark.parametrize("page_size", [32, 64])
@pytest.mark.parametrize("name,dtype,mode", [("W", "bfloat16", "mixed"), ("W", "bfloat16", "portions"), ("A", "bfloat16", "mixed"),
                                             ("C", "bfloat16", "mixed"), ("B", "float32", "mixed"), ("D", "float32", "portions")])
def test_gpu_pages_of_other_sizes(model_dirs, model_dirs_bf16, wide_model_dir, name, dtype, mode, page_size):
    """Pages of 32 and 64 tokens: block tables half and a quarter as wide, chunks and windows that end inside a page,
    the kernels' walks through pages that hold more than one of their tiles."""
    folder = wide_model_dir if name == "W" else (model_dirs_bf16 if dtype == "bfloat16" else model_dirs)[name]
    _check(name, folder, dtype, "cuda:0", mode, reference_ops=False, plain_device="cuda:0" if name == "W" else "cpu",
           page_size=page_size)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sixty_four_live_requests_at_serving_widths(wide_model_dir, wide_model_dir_f32, dtype):
    """What the benchmark's batches look like: 64 requests live at once, eight of them past 2,000 tokens, so
    that the decode steps' key ranges are more than the GPU takes in one go; steps of 64 single tokens (64 rows
    through the weight-streaming products, the output head and the library's dense projections), portions of
    up to 300 tokens beside them, pages used again.  In float32 the steps of single tokens are replays of
    recorded graphs and the yardstick is the plain model in float64; in bfloat16 the plain model is given the
    engine's expert choices (a watched step runs launch by launch, through the same kernels)."""
    folder = wide_model_dir if dtype == "bfloat16" else wide_model_dir_f32
    g = torch.Generator().manual_seed(12)
    lengths = torch.randint(100, 300, (64,), generator=g).tolist()
    for i in range(0, 64, 8):
        lengths[i] = 2050 + 19 * i
    mode = lambda reqs: traces.mixed(reqs, seed=3, max_live=64, decode_tail=20, max_portion=300)
    _check("W", folder, dtype, "cuda:0", mode, reference_ops=False, plain_device="cuda:0",
           record=dtype == "bfloat16", plain_dtype=torch.float64 if dtype == "float32" else torch.float32,
           lengths=lengths, max_requests=64)


@pytest.mark.gpu
def test_gpu_float32_serving_widths(wide_model_dir_f32):
    """The plain model runs in float64 here: run in float32 on the GPU it would go through the same library
    products as the engine's dense projections, and a reduced-precision mode of the library at inner sizes of
    5120 to 16384 would pass unseen."""
    _check("W", wide_model_dir_f32, "float32", "cuda:0", "mixed", reference_ops=False, plain_device="cuda:0",
           plain_dtype=torch.float64)


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(TINY))
def test_gpu_bfloat16_expert_choices_differ_only_at_near_ties(model_dirs_bf16, name):
    folder = model_dirs_bf16[name]
    reqs = traces.random_requests(_vocab(name), LENGTHS[name], seed=5)
    steps = traces.portions(reqs)
    runner = make_runner(folder, "bfloat16", traces.max_live_tokens(steps), "cuda:0")
    _, routes = traces.run_trace(runner, steps, record_routing=True)
    plain = PlainModel(folder)
    total = flips = 0
    for rid, toks in reqs.items():
        info = {}
        plain.logits(toks, forced=routes[rid], info=info)  # same inputs to every router as the engine's run
        for li, (_, scores) in info.items():
            k = routes[rid][li].shape[1]
            top = torch.sort(scores, dim=-1, descending=True)
            want = top.indices[:, :k]
            got = routes[rid][li].long()
            diff = (got != want).any(-1)
            total += diff.numel()
            flips += int(diff.sum())
            if diff.any():
                # where the choice differs, the scores of the two candidates are close
                margin = (torch.gather(scores, 1, want) - torch.gather(scores, 1, got)).abs().max(-1).values
                assert (margin[diff] < 0.05 * scores.std()).all(), f"{rid} layer {li}: a clear choice went wrong"
    assert flips <= 0.05 * total
