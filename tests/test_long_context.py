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
    plain = PlainModel(folder)
    plain.w = {k: v.cuda() for k, v in plain.w.items()}
    prev = torch.get_default_device()
    torch.set_default_device("cuda")
    try:
        forced = {li: ids.cuda() for li, ids in routes["a"].items()} if dtype == "bfloat16" else None
        ref = plain.logits(toks, forced=forced).cpu()
    finally:
        torch.set_default_device(prev)
    assert torch.isfinite(got).all()
    err = (got - ref).abs().max(dim=-1).values / ref.abs().max()
    tol = 5e-5 if dtype == "float32" else 2e-2
    bad = (err > tol).nonzero().squeeze(-1).tolist()
    assert not bad, f"first wrong position {bad[0]} (of {len(bad)}), error {float(err[bad[0]]):.3g}"
    # the boundaries matter: a model that ignored the chunk or the temperature step would differ there
    for p in (8191, 8192, 16383, 16384, T - 1):
        assert err[p] <= tol
