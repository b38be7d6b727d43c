"""Two tiny Llama 4 configurations that differ in every size and option."""
import torch

TINY = {
    # all layers with experts, qk norm, temperature tuning, no frequency scaling, layer 3 NoPE
    "A": {
        "architectures": ["Llama4ForCausalLM"],
        "seed": 11,
        "num_hidden_layers": 4, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
        "head_dim": 16, "interleave_moe_layer_step": 1, "num_local_experts": 4, "num_experts_per_tok": 1,
        "intermediate_size": 128, "intermediate_size_mlp": 256, "vocab_size": 512, "rope_theta": 10000.0,
        "rope_scaling": None, "no_rope_layers": [1, 1, 1, 0], "attention_chunk_size": 32, "use_qk_norm": True,
        "attn_temperature_tuning": True, "floor_scale": 16, "attn_scale": 0.1, "rms_norm_eps": 1e-5,
        "tie_word_embeddings": False,
    },
    # experts on every 2nd layer, dense elsewhere, no qk norm, no temperature, llama3 scaling, multimodal naming
    "B": {
        "architectures": ["Llama4ForConditionalGeneration"],
        "seed": 23,
        "text_config": {
            "num_hidden_layers": 6, "hidden_size": 96, "num_attention_heads": 6, "num_key_value_heads": 3,
            "head_dim": 32, "interleave_moe_layer_step": 2, "num_local_experts": 8, "num_experts_per_tok": 1,
            "intermediate_size": 64, "intermediate_size_mlp": 192, "vocab_size": 1000, "rope_theta": 500000.0,
            "rope_scaling": {"rope_type": "llama3", "factor": 4.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                             "original_max_position_embeddings": 64},
            "no_rope_layers": [1, 1, 0, 1, 1, 0], "attention_chunk_size": 48, "use_qk_norm": False,
            "attn_temperature_tuning": False, "rms_norm_eps": 1e-6, "tie_word_embeddings": False,
        },
    },
    # odd sizes: width and vocabulary that are no power of two, 5 heads in one group, head size 48,
    # two experts per token, a chunk that is no multiple of the page size
    "C": {
        "architectures": ["Llama4ForCausalLM"],
        "seed": 37,
        "num_hidden_layers": 3, "hidden_size": 80, "num_attention_heads": 5, "num_key_value_heads": 1,
        "head_dim": 48, "interleave_moe_layer_step": 1, "moe_layers": [0, 2], "num_local_experts": 3,
        "num_experts_per_tok": 2, "intermediate_size": 40, "intermediate_size_mlp": 56, "vocab_size": 311,
        "rope_theta": 1000.0, "rope_scaling": None, "no_rope_layers": [1, 0, 1], "attention_chunk_size": 20,
        "use_qk_norm": True, "attn_temperature_tuning": True, "floor_scale": 7, "attn_scale": 0.25,
        "rms_norm_eps": 1e-4, "tie_word_embeddings": False,
    },
    # sizes that fit no fast path: a width that is no multiple of 4 or 8, expert width with 4 left over, a
    # vocabulary that is prime, every head its own kv head, a chunk shorter than a page, NoPE first, dense first
    "D": {
        "architectures": ["Llama4ForCausalLM"],
        "seed": 41,
        "num_hidden_layers": 2, "hidden_size": 54, "num_attention_heads": 3, "num_key_value_heads": 3,
        "head_dim": 16, "interleave_moe_layer_step": 2, "num_local_experts": 2, "num_experts_per_tok": 1,
        "intermediate_size": 20, "intermediate_size_mlp": 28, "vocab_size": 257, "rope_theta": 50.0,
        "rope_scaling": {"rope_type": "llama3", "factor": 2.0, "low_freq_factor": 1.0, "high_freq_factor": 2.0,
                         "original_max_position_embeddings": 16},
        "no_rope_layers": [0, 1], "attention_chunk_size": 7, "use_qk_norm": False,
        "attn_temperature_tuning": True, "floor_scale": 5, "attn_scale": 0.3, "rms_norm_eps": 1e-3,
        "tie_word_embeddings": False,
    },
}

# Small, but with the sizes that the fast kernels need (GPU tests only): head size 128 with five query heads per
# kv head (prefill attention shares keys between them), widths that are multiples of 256 (the expert matrices go
# into the streaming layout and prefill goes through the weight-streaming grouped product)
FAST = {
    "F": {
        "architectures": ["Llama4ForCausalLM"],
        "seed": 53,
        "num_hidden_layers": 2, "hidden_size": 256, "num_attention_heads": 10, "num_key_value_heads": 2,
        "head_dim": 128, "interleave_moe_layer_step": 1, "num_local_experts": 4, "num_experts_per_tok": 1,
        "intermediate_size": 256, "intermediate_size_mlp": 512, "vocab_size": 600, "rope_theta": 10000.0,
        "rope_scaling": None, "no_rope_layers": [1, 0], "attention_chunk_size": 96, "use_qk_norm": True,
        "attn_temperature_tuning": True, "floor_scale": 64, "attn_scale": 0.1, "rms_norm_eps": 1e-5,
        "tie_word_embeddings": False,
    },
}

# The widths that serving runs at (Llama 4 Scout's: width 5120, 40 query heads on 8 kv heads of 128, experts 8192
# wide, chunk 8192 and its frequency scaling), with few layers, few experts and a short vocabulary that is no
# power of two: about 3 GB in bfloat16 (GPU tests only)
FAST["W"] = {
    "architectures": ["Llama4ForCausalLM"],
    "seed": 67,
    "num_hidden_layers": 2, "hidden_size": 5120, "num_attention_heads": 40, "num_key_value_heads": 8,
    "head_dim": 128, "interleave_moe_layer_step": 1, "num_local_experts": 4, "num_experts_per_tok": 1,
    "intermediate_size": 8192, "intermediate_size_mlp": 16384, "vocab_size": 20008, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 16.0, "low_freq_factor": 1.0, "high_freq_factor": 1.0,
                     "original_max_position_embeddings": 8192},
    "no_rope_layers": [1, 0], "attention_chunk_size": 8192, "use_qk_norm": True, "attn_temperature_tuning": True,
    "floor_scale": 8192, "attn_scale": 0.1, "rms_norm_eps": 1e-5, "tie_word_embeddings": False,
}

# The shapes of the larger Llama 4 (``llama4/llama4_jax/configs.py:57-93``: experts on every second layer, 128 of
# them, dense layers 16,384 wide between, no frequency scaling) at serving widths, with the experts' width cut (not
# their number) so that the plain model stays cheap: about 1.8 GB in bfloat16 (GPU tests only)
FAST["M"] = {
    "architectures": ["Llama4ForCausalLM"],
    "seed": 79,
    "num_hidden_layers": 2, "hidden_size": 5120, "num_attention_heads": 40, "num_key_value_heads": 8,
    "head_dim": 128, "interleave_moe_layer_step": 2, "num_local_experts": 128, "num_experts_per_tok": 1,
    "intermediate_size": 256, "intermediate_size_mlp": 16384, "vocab_size": 20008, "rope_theta": 500000.0,
    "rope_scaling": None, "no_rope_layers": [1, 0], "attention_chunk_size": 8192, "use_qk_norm": True,
    "attn_temperature_tuning": True, "floor_scale": 8192, "attn_scale": 0.1, "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False,
}


def tiny_config_json(name: str) -> dict:
    c = {k: v for k, v in {**TINY, **FAST}[name].items() if k != "seed"}
    return c


def write_tiny(name: str, out_dir: str, dtype=torch.float32) -> str:
    from jax_llm_examples_amd.config import get_architecture
    from jax_llm_examples_amd.weights import write_random_model

    top = tiny_config_json(name)
    arch = get_architecture(top["architectures"][0])
    cfg = arch.parse_config(top)
    return write_random_model(arch, cfg, out_dir, {**TINY, **FAST}[name]["seed"], dtype,
                              architecture=top["architectures"][0])
