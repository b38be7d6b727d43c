import copy
import json

import pytest

from jax_llm_examples_amd.config import (ConfigError, Llama4TextConfig, UnknownArchitectureError, get_architecture,
                                         known_architectures, load_config)
from jax_llm_examples_amd.config.presets import preset
from tiny_configs import TINY, tiny_config_json


def test_registry_names_and_unknown():
    assert {"Llama4ForCausalLM", "Llama4ForConditionalGeneration"} <= set(known_architectures())
    assert get_architecture("Llama4ForCausalLM") is get_architecture("Llama4ForConditionalGeneration")
    with pytest.raises(UnknownArchitectureError, match="known: .*Llama4ForCausalLM"):
        get_architecture("GPT2LMHeadModel")


@pytest.mark.parametrize("name", list(TINY))
def test_parse_and_round_trip(name, tmp_path):
    top = tiny_config_json(name)
    arch = get_architecture(top["architectures"][0])
    cfg = arch.parse_config(top)
    text = top.get("text_config", top)
    assert cfg.hidden_size == text["hidden_size"] and cfg.head_dim == text["head_dim"]
    assert cfg.rms_norm_eps == text["rms_norm_eps"] and cfg.attention_chunk_size == text["attention_chunk_size"]
    again = arch.parse_config(json.loads(json.dumps(arch.config_to_dict(cfg, top["architectures"][0]))))
    assert again == cfg
    (tmp_path / "config.json").write_text(json.dumps(top))
    arch2, cfg2 = load_config(tmp_path)
    assert arch2 is arch and cfg2 == cfg


def test_model_type_stands_in_for_a_missing_architectures_entry():
    from jax_llm_examples_amd.config.registry import architecture_name
    from tiny_configs import tiny_config_json

    top = {k: v for k, v in tiny_config_json("A").items() if k != "architectures"}
    top["model_type"] = "llama4_text"
    assert get_architecture(architecture_name(top)) is get_architecture("Llama4ForCausalLM")
    with pytest.raises(UnknownArchitectureError, match="neither"):
        architecture_name({"hidden_size": 8})


def test_text_config_is_used_when_present():
    top = tiny_config_json("B")
    assert "text_config" in top
    cfg = Llama4TextConfig.from_dict(top)
    assert cfg.num_hidden_layers == 6 and cfg.moe_layers == (1, 3, 5) and cfg.no_rope_layers == (1, 1, 0, 1, 1, 0)
    assert cfg.rope_scaling.factor == 4.0 and cfg.rope_scaling.original_max_position_embeddings == 64


def test_defaults_follow_the_reference():
    top = copy.deepcopy(tiny_config_json("A"))
    del top["no_rope_layers"], top["head_dim"], top["attn_temperature_tuning"]
    top["num_hidden_layers"] = 9
    cfg = Llama4TextConfig.from_dict(top)
    assert cfg.no_rope_layers == (1, 1, 1, 0, 1, 1, 1, 0, 1)  # every 4th layer is NoPE
    assert cfg.head_dim == 64 // 4 and cfg.attn_temperature_tuning is False
    top["interleave_moe_layer_step"] = 3
    assert Llama4TextConfig.from_dict(top).moe_layers == (2, 5, 8)


def test_errors_name_the_key():
    top = tiny_config_json("A")
    for key in ("hidden_size", "num_local_experts", "rms_norm_eps"):
        bad = {k: v for k, v in top.items() if k != key}
        with pytest.raises(ConfigError, match=key):
            Llama4TextConfig.from_dict(bad)
    with pytest.raises(ConfigError, match="num_key_value_heads"):
        Llama4TextConfig.from_dict({**top, "num_key_value_heads": 3})
    with pytest.raises(ConfigError, match="no_rope_layers"):
        Llama4TextConfig.from_dict({**top, "no_rope_layers": [1, 0]})
    with pytest.raises(ConfigError, match="num_experts_per_tok"):
        Llama4TextConfig.from_dict({**top, "num_experts_per_tok": 9})
    with pytest.raises(ConfigError, match="rope_type"):
        Llama4TextConfig.from_dict({**top, "rope_scaling": {"rope_type": "yarn", "factor": 2}})
    with pytest.raises(ConfigError, match="tie_word_embeddings"):
        Llama4TextConfig.from_dict({**top, "tie_word_embeddings": True})


def test_plan_chooses_parts_layer_by_layer():
    cfg = Llama4TextConfig.from_dict(tiny_config_json("B"))
    plan = cfg.plan()
    assert len(plan.layers) == 6 and [e.layer for e in plan.order] == list(range(6))
    kinds = [(l.mixer.position.kind, l.mixer.retention, l.feed_forward.kind) for l in plan.layers]
    assert kinds[0] == ("rope_interleaved", ("chunk", 48), "dense_swiglu")
    assert kinds[1] == ("rope_interleaved", ("chunk", 48), "moe_sigmoid_shared")
    assert kinds[2] == ("none", ("all",), "dense_swiglu")
    assert kinds[5] == ("none", ("all",), "moe_sigmoid_shared")
    assert plan.layers[0].feed_forward.intermediate_size == 192 and plan.layers[1].feed_forward.intermediate_size == 64
    a = Llama4TextConfig.from_dict(tiny_config_json("A")).plan()
    assert a.layers[0].mixer.qk_norm.eps == 1e-5 and a.layers[3].mixer.qk_norm is None
    assert a.layers[3].mixer.query_scale.floor_scale == 16 and a.layers[0].mixer.query_scale is None


def test_scout_preset_matches_the_benchmark_configuration():
    cfg = Llama4TextConfig.from_dict(preset("llama4-scout"))
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads,
            cfg.head_dim) == (48, 5120, 40, 8, 128)
    assert (cfg.num_local_experts, cfg.intermediate_size, cfg.intermediate_size_mlp, cfg.vocab_size) == \
        (16, 8192, 16384, 202048)
    assert cfg.rope_scaling.factor == 16 and sum(cfg.no_rope_layers) == 36 and len(cfg.moe_layers) == 48
    assert len(Llama4TextConfig.from_dict(preset("llama4-maverick", 8)).moe_layers) == 4


def test_floor_scale_is_written_as_the_integer_it_is():
    """Checkpoints store a whole number there, and strict readers of config.json refuse ``8192.0``."""
    top = tiny_config_json("A")
    cfg = Llama4TextConfig.from_dict(top)
    out = cfg.to_dict()
    assert isinstance(out["floor_scale"], int) and out["floor_scale"] == 16
    top["floor_scale"] = 2.5
    assert Llama4TextConfig.from_dict(top).to_dict()["floor_scale"] == 2.5
