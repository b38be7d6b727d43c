"""Configurations drawn at random (fixed seeds): head sizes in steps of 16 up to 256, any number of heads and groups,
widths and vocabularies that are no power of two, one to seventeen experts with one or two per token, dense layers
between them, chunks that are no multiple of the page size, three page sizes, with and without frequency scaling,
q/k norm and temperature.  Each runs a mixed trace (portions beside single tokens, pages used again) in float32 and
bfloat16 against the plain implementation: the kernels take every size the configuration allows."""
import random

import pytest
import torch

import traces
from jax_llm_examples_amd.config import get_architecture
from jax_llm_examples_amd.engine.replay import make_runner
from jax_llm_examples_amd.weights import write_random_model
from plain_llama4 import PlainModel

pytestmark = pytest.mark.gpu
TOL = {"float32": 2e-5, "bfloat16": 1.5e-2}  # of the largest logit of the request


def draw(seed: int):
    rng = random.Random(seed)
    hk = rng.choice([1, 2, 3, 4])
    layers = rng.randint(1, 4)
    experts = rng.choice([1, 2, 3, 4, 8, 17])
    scaling = rng.choice([None, {"rope_type": "llama3", "factor": rng.choice([2.0, 8.0]), "low_freq_factor": 1.0,
                                 "high_freq_factor": rng.choice([1.0, 4.0]),
                                 "original_max_position_embeddings": rng.choice([16, 64])}])
    top = {
        "architectures": ["Llama4ForCausalLM"], "num_hidden_layers": layers,
        "hidden_size": rng.choice([56, 64, 72, 100, 128, 136, 192, 256, 264, 320]),
        "num_attention_heads": hk * rng.choice([1, 2, 3, 5, 8]), "num_key_value_heads": hk,
        "head_dim": rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 144, 160, 192, 256]),
        "interleave_moe_layer_step": rng.choice([1, 2]), "num_local_experts": experts,
        "num_experts_per_tok": rng.choice([1, 1, 2]) if experts > 1 else 1,
        "intermediate_size": rng.choice([24, 32, 40, 64, 96, 128, 256]),
        "intermediate_size_mlp": rng.choice([32, 48, 64, 128]), "vocab_size": rng.choice([97, 257, 300, 512, 1001]),
        "rope_theta": rng.choice([50.0, 10000.0, 500000.0]), "rope_scaling": scaling,
        "no_rope_layers": [rng.choice([0, 1, 1]) for _ in range(layers)],
        "attention_chunk_size": rng.choice([5, 16, 24, 32, 50, 64, 100]), "use_qk_norm": rng.choice([True, False]),
        "attn_temperature_tuning": rng.choice([True, False]), "floor_scale": rng.choice([4, 16, 8192]),
        "attn_scale": 0.1, "rms_norm_eps": rng.choice([1e-5, 1e-6, 1e-3]), "tie_word_embeddings": False,
    }
    lengths = [rng.choice([1, 2, 17, 33, 64, 65, 97, 130]) for _ in range(rng.randint(2, 5))]
    return top, rng.choice([16, 16, 32, 64]), lengths


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", list(range(24)))
def test_random_configuration(tmp_path, seed, dtype):
    top, page_size, lengths = draw(seed)
    arch = get_architecture(top["architectures"][0])
    folder = write_random_model(arch, arch.parse_config(top), str(tmp_path / "m"), seed,
                                torch.float32 if dtype == "float32" else torch.bfloat16)
    reqs = traces.random_requests(top["vocab_size"], lengths, seed=seed)
    steps = traces.mixed(reqs, seed=seed)
    runner = make_runner(folder, dtype, traces.max_live_tokens(steps), "cuda:0", page_size=page_size, poison=True)
    got, routes = traces.run_trace(runner, steps, record_routing=True)
    runner.cache.check()
    assert runner.cache.num_live() == 0
    plain = PlainModel(folder)
    for rid, toks in reqs.items():
        ref = plain.logits(toks, forced=routes.get(rid) if dtype == "bfloat16" else None)
        assert torch.isfinite(got[rid]).all(), f"{top}: {rid}: non-finite logits"
        err = (got[rid] - ref).abs().max(dim=-1).values / ref.abs().max()
        bad = (err > TOL[dtype]).nonzero().squeeze(-1).tolist()
        assert not bad, f"{top}, page size {page_size}: {rid}: first wrong position {bad[0]}, error {err[bad[0]]:.3g}"
