"""config.json contents of the published Llama 4 sizes, for benchmarks with random
weights.  The sizes are those of the reference's constants
(``llama4/llama4_jax/configs.py:19-93``: 48 layers, width 5120, 40/8 heads of 128,
16 or 128 experts of width 8192, dense width 16384, vocabulary 202048, chunk 8192,
NoPE every 4th layer); frequency scaling, temperature tuning and qk norm are set
as the benchmark configurations state them."""
from __future__ import annotations

import copy

_COMMON = {
    "hidden_size": 5120, "num_attention_heads": 40, "num_key_value_heads": 8, "head_dim": 128,
    "intermediate_size": 8192, "intermediate_size_mlp": 16384, "vocab_size": 202048, "rms_norm_eps": 1e-5,
    "num_experts_per_tok": 1, "rope_theta": 500000.0, "attention_chunk_size": 8192, "use_qk_norm": True,
    "attn_temperature_tuning": True, "floor_scale": 8192, "attn_scale": 0.1, "tie_word_embeddings": False,
    "torch_dtype": "bfloat16",
}

PRESETS = {
    "llama4-scout": {
        "architectures": ["Llama4ForCausalLM"], **_COMMON, "num_hidden_layers": 48, "num_local_experts": 16,
        "interleave_moe_layer_step": 1,
        "rope_scaling": {"rope_type": "llama3", "factor": 16.0, "low_freq_factor": 1.0, "high_freq_factor": 1.0,
                         "original_max_position_embeddings": 8192},
    },
    "llama4-maverick": {
        "architectures": ["Llama4ForCausalLM"], **_COMMON, "num_hidden_layers": 48, "num_local_experts": 128,
        "interleave_moe_layer_step": 2, "rope_scaling": None,
    },
}


def preset(name: str, num_layers: int | None = None) -> dict:
    """A copy of the named config.json, optionally cut to its first ``num_layers`` layers."""
    if name not in PRESETS:
        raise KeyError(f"unknown preset {name!r}; known: {', '.join(sorted(PRESETS))}")
    c = copy.deepcopy(PRESETS[name])
    if num_layers is not None:
        c["num_hidden_layers"] = int(num_layers)
    L = c["num_hidden_layers"]
    c["no_rope_layers"] = [0 if (i + 1) % 4 == 0 else 1 for i in range(L)]
    return c
