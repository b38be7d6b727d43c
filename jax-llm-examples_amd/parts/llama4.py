"""The Llama 4 text decoder as an architecture: its configuration, its plan and
the names and layouts of its checkpoint tensors.

Checkpoint names and shapes as the reference's converter asserts them
(``llama4/llama4_jax/chkpt_utils.py:80-209``): linear weights are ``[out, in]``;
``experts.gate_up_proj`` is ``[E, D, 2F]`` with the gate in the first half of
the last axis and up in the second (``chkpt_utils.py:198-205``);
``experts.down_proj`` is ``[E, F, D]``.  The multimodal checkpoint prefixes
every text tensor with ``language_model.`` (``scripts/convert_weights.py:41``);
its vision tensors are ignored.
"""
from __future__ import annotations

from typing import Any, Mapping

from ..config.llama4 import Llama4TextConfig
from ..config.registry import register_architecture
from ..config.specs import ModelPlan
from ..weights.bindings import TensorBinding


class Llama4Architecture:
    # config.json's "architectures" entries, and its "model_type" values for folders that carry only those
    names = ("Llama4ForConditionalGeneration", "Llama4ForCausalLM", "llama4", "llama4_text")
    optional_prefixes = ("language_model.",)
    ignored_prefixes = ("vision_model.", "multi_modal_projector.")

    def parse_config(self, top: Mapping[str, Any]) -> Llama4TextConfig:
        return Llama4TextConfig.from_dict(top)

    def plan(self, cfg: Llama4TextConfig) -> ModelPlan:
        return cfg.plan()

    def config_to_dict(self, cfg: Llama4TextConfig, architecture: str | None = None) -> dict:
        return cfg.to_dict(architecture or "Llama4ForCausalLM")

    def checkpoint_prefix(self, architecture: str | None) -> str:
        return "language_model." if architecture == "Llama4ForConditionalGeneration" else ""

    def bindings(self, cfg: Llama4TextConfig, plan: ModelPlan) -> list[TensorBinding]:
        D, V = cfg.hidden_size, cfg.vocab_size
        hq, hk, dh = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
        F, Fm, E = cfg.intermediate_size, cfg.intermediate_size_mlp, cfg.num_local_experts
        ones = ("ones",)
        out = [TensorBinding("model.embed_tokens.weight", (V, D), "embed.weight")]
        moe = set(cfg.moe_layers)
        for i in range(cfg.num_hidden_layers):
            p, t = f"model.layers.{i}.", f"layers.{i}."
            out += [
                TensorBinding(p + "input_layernorm.weight", (D,), t + "mixer_norm.weight", init=ones),
                TensorBinding(p + "self_attn.q_proj.weight", (hq * dh, D), t + "mixer.wqkv", rows=(0, hq * dh)),
                TensorBinding(p + "self_attn.k_proj.weight", (hk * dh, D), t + "mixer.wqkv",
                              rows=(hq * dh, (hq + hk) * dh)),
                TensorBinding(p + "self_attn.v_proj.weight", (hk * dh, D), t + "mixer.wqkv",
                              rows=((hq + hk) * dh, (hq + 2 * hk) * dh)),
                TensorBinding(p + "self_attn.o_proj.weight", (D, hq * dh), t + "mixer.wo"),
                TensorBinding(p + "post_attention_layernorm.weight", (D,), t + "feed_forward_norm.weight", init=ones),
            ]
            ff, tf = p + "feed_forward.", t + "feed_forward."
            if i in moe:
                out += [
                    TensorBinding(ff + "router.weight", (E, D), tf + "router", float32=True),
                    # stored [E, in, out]; held [E, out, in]
                    TensorBinding(ff + "experts.gate_up_proj", (E, D, 2 * F), tf + "w_gate_up", transpose=(1, 2)),
                    TensorBinding(ff + "experts.down_proj", (E, F, D), tf + "w_down", transpose=(1, 2)),
                    TensorBinding(ff + "shared_expert.gate_proj.weight", (F, D), tf + "shared_gate_up", rows=(0, F)),
                    TensorBinding(ff + "shared_expert.up_proj.weight", (F, D), tf + "shared_gate_up", rows=(F, 2 * F)),
                    TensorBinding(ff + "shared_expert.down_proj.weight", (D, F), tf + "shared_down"),
                ]
            else:
                out += [
                    TensorBinding(ff + "gate_proj.weight", (Fm, D), tf + "w_gate_up", rows=(0, Fm)),
                    TensorBinding(ff + "up_proj.weight", (Fm, D), tf + "w_gate_up", rows=(Fm, 2 * Fm)),
                    TensorBinding(ff + "down_proj.weight", (D, Fm), tf + "w_down"),
                ]
        out += [
            TensorBinding("model.norm.weight", (D,), "final_norm.weight", init=ones),
            TensorBinding("lm_head.weight", (V, D), "lm_head.weight"),
        ]
        return out


LLAMA4 = register_architecture(Llama4Architecture())
