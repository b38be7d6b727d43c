"""Typed configuration of the Llama 4 text decoder, read from ``config.json``.

Key names are those of the checkpoint's ``text_config`` as the reference reads
them (``llama4/llama4_jax/model.py:199-226``): ``hidden_size``,
``intermediate_size_mlp``, ``intermediate_size``, ``num_attention_heads``,
``num_key_value_heads``, ``num_hidden_layers``, ``head_dim``, ``vocab_size``,
``rms_norm_eps``, ``use_qk_norm``, ``attention_chunk_size``,
``interleave_moe_layer_step``, ``num_experts_per_tok``, ``num_local_experts``,
``rope_theta``.  The reference fixes the NoPE interval (4, ``model.py:203``)
and the llama3 frequency scaling constants (``model.py:159-163``) in code and
has no attention temperature; here ``no_rope_layers``, ``rope_scaling``,
``attn_temperature_tuning``, ``floor_scale`` and ``attn_scale`` come from
``config.json`` as well.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Mapping, Optional

from .specs import LayerSpec, ModelPlan, default_order, part


def _number(v):
    """A whole number stays an integer (checkpoints store ``floor_scale`` as one)."""
    f = float(v)
    return int(f) if f.is_integer() else f


class ConfigError(ValueError):
    """A config.json that cannot describe a model: names the key at fault."""


@dataclasses.dataclass(frozen=True)
class RopeScaling:
    """llama3-style frequency scaling (``model.py:654-672``)."""

    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int
    rope_type: str = "llama3"


_REQUIRED = (
    "hidden_size",
    "intermediate_size",
    "num_attention_heads",
    "num_key_value_heads",
    "num_hidden_layers",
    "vocab_size",
    "rms_norm_eps",
    "num_local_experts",
    "num_experts_per_tok",
    "interleave_moe_layer_step",
    "rope_theta",
)


@dataclasses.dataclass(frozen=True)
class Llama4TextConfig:
    hidden_size: int
    intermediate_size: int  # width of each routed expert and of the shared expert
    intermediate_size_mlp: int  # width of the dense feed-forward on layers without experts
    num_attention_heads: int
    num_key_value_heads: int
    num_hidden_layers: int
    head_dim: int
    vocab_size: int
    rms_norm_eps: float
    use_qk_norm: bool
    attention_chunk_size: Optional[int]
    num_local_experts: int
    num_experts_per_tok: int
    moe_layers: tuple[int, ...]  # indices of layers whose feed-forward is routed experts
    no_rope_layers: tuple[int, ...]  # per layer: 1 = rotary + chunked attention, 0 = NoPE + global
    rope_theta: float
    rope_scaling: Optional[RopeScaling]
    attn_temperature_tuning: bool
    floor_scale: float  # (held as an integer where config.json has a whole number, and written back so)
    attn_scale: float
    tie_word_embeddings: bool = False
    torch_dtype: str = "bfloat16"
    max_position_embeddings: Optional[int] = None
    bos_token_id: Optional[int] = None
    eos_token_id: Any = None
    pad_token_id: Optional[int] = None
    interleave_moe_layer_step: int = 1

    # ------------------------------------------------------------------ parse
    @classmethod
    def from_dict(cls, top: Mapping[str, Any]) -> "Llama4TextConfig":
        """``top`` is a whole config.json; the text decoder's keys are under
        ``text_config`` for the multimodal checkpoint (``model.py:229-231``)
        and at top level for the text-only one."""
        d = dict(top["text_config"]) if isinstance(top.get("text_config"), Mapping) else dict(top)
        missing = [k for k in _REQUIRED if d.get(k) is None]
        if missing:
            raise ConfigError(f"config.json lacks required key(s): {', '.join(missing)}")
        L = int(d["num_hidden_layers"])
        heads = int(d["num_attention_heads"])
        head_dim = d.get("head_dim")
        if head_dim is None:
            if int(d["hidden_size"]) % heads:
                raise ConfigError("head_dim is absent and hidden_size is no multiple of num_attention_heads")
            head_dim = int(d["hidden_size"]) // heads

        step = int(d["interleave_moe_layer_step"])
        if d.get("moe_layers") is not None:
            moe_layers = tuple(int(i) for i in d["moe_layers"])
        else:
            if step < 1:
                raise ConfigError(f"interleave_moe_layer_step must be >= 1, got {step}")
            # layer i has experts iff (i + 1) % step == 0  (model.py:558)
            moe_layers = tuple(i for i in range(L) if (i + 1) % step == 0)

        nrl = d.get("no_rope_layers")
        if nrl is None or len(nrl) == 0:
            # the reference's fixed interval: layer i is NoPE iff (i + 1) % 4 == 0  (model.py:203, 913)
            interval = int(d.get("nope_layer_interval", 4))
            nrl = [0 if (i + 1) % interval == 0 else 1 for i in range(L)]
        no_rope_layers = tuple(int(bool(v)) for v in nrl)

        rs = d.get("rope_scaling")
        rope_scaling = None
        if rs is not None:
            kind = rs.get("rope_type", rs.get("type", "llama3"))
            if kind != "llama3":
                raise ConfigError(f"rope_scaling.rope_type {kind!r} is not supported (only 'llama3')")
            try:
                rope_scaling = RopeScaling(
                    factor=float(rs["factor"]),
                    low_freq_factor=float(rs["low_freq_factor"]),
                    high_freq_factor=float(rs["high_freq_factor"]),
                    original_max_position_embeddings=int(rs["original_max_position_embeddings"]),
                )
            except KeyError as e:
                raise ConfigError(f"rope_scaling lacks key {e.args[0]!r}") from None

        chunk = d.get("attention_chunk_size")
        cfg = cls(
            hidden_size=int(d["hidden_size"]),
            intermediate_size=int(d["intermediate_size"]),
            intermediate_size_mlp=int(d.get("intermediate_size_mlp") or d["intermediate_size"]),
            num_attention_heads=heads,
            num_key_value_heads=int(d["num_key_value_heads"]),
            num_hidden_layers=L,
            head_dim=int(head_dim),
            vocab_size=int(d["vocab_size"]),
            rms_norm_eps=float(d["rms_norm_eps"]),
            use_qk_norm=bool(d.get("use_qk_norm", True)),
            attention_chunk_size=None if chunk is None else int(chunk),
            num_local_experts=int(d["num_local_experts"]),
            num_experts_per_tok=int(d["num_experts_per_tok"]),
            moe_layers=moe_layers,
            no_rope_layers=no_rope_layers,
            rope_theta=float(d["rope_theta"]),
            rope_scaling=rope_scaling,
            attn_temperature_tuning=bool(d.get("attn_temperature_tuning", False)),
            floor_scale=_number(d.get("floor_scale", 8192)),
            attn_scale=float(d.get("attn_scale", 0.1)),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", top.get("tie_word_embeddings", False))),
            torch_dtype=str(d.get("torch_dtype", top.get("torch_dtype", "bfloat16"))),
            max_position_embeddings=d.get("max_position_embeddings"),
            bos_token_id=d.get("bos_token_id"),
            eos_token_id=d.get("eos_token_id"),
            pad_token_id=d.get("pad_token_id"),
            interleave_moe_layer_step=step,
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        L = self.num_hidden_layers
        if L < 1:
            raise ConfigError("num_hidden_layers must be >= 1")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads ({self.num_attention_heads}) is no multiple of "
                f"num_key_value_heads ({self.num_key_value_heads})"
            )
        if self.head_dim % 2:
            raise ConfigError(f"head_dim ({self.head_dim}) must be even for rotary pairs")
        if len(self.no_rope_layers) != L:
            raise ConfigError(f"no_rope_layers has {len(self.no_rope_layers)} entries for {L} layers")
        if any(not 0 <= i < L for i in self.moe_layers):
            raise ConfigError(f"moe_layers {list(self.moe_layers)} names a layer outside 0..{L - 1}")
        if not 1 <= self.num_experts_per_tok <= self.num_local_experts:
            raise ConfigError(
                f"num_experts_per_tok ({self.num_experts_per_tok}) must lie in 1..num_local_experts "
                f"({self.num_local_experts})"
            )
        if self.attention_chunk_size is not None and self.attention_chunk_size < 1:
            raise ConfigError("attention_chunk_size must be positive or null")
        if self.tie_word_embeddings:
            raise ConfigError("tie_word_embeddings=true: Llama 4 has an lm_head of its own (model.py:575-592)")
        if self.floor_scale <= 0:
            raise ConfigError("floor_scale must be positive")
        if self.rms_norm_eps <= 0:
            raise ConfigError("rms_norm_eps must be positive")

    # ---------------------------------------------------------------- to_dict
    def to_dict(self, architecture: str = "Llama4ForCausalLM") -> dict[str, Any]:
        """A config.json that :meth:`from_dict` reads back to an equal object."""
        text: dict[str, Any] = {
            "model_type": "llama4_text",
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "intermediate_size_mlp": self.intermediate_size_mlp,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "num_hidden_layers": self.num_hidden_layers,
            "head_dim": self.head_dim,
            "vocab_size": self.vocab_size,
            "rms_norm_eps": self.rms_norm_eps,
            "use_qk_norm": self.use_qk_norm,
            "attention_chunk_size": self.attention_chunk_size,
            "num_local_experts": self.num_local_experts,
            "num_experts_per_tok": self.num_experts_per_tok,
            "interleave_moe_layer_step": self.interleave_moe_layer_step,
            "moe_layers": list(self.moe_layers),
            "no_rope_layers": list(self.no_rope_layers),
            "rope_theta": self.rope_theta,
            "rope_scaling": None
            if self.rope_scaling is None
            else {
                "rope_type": "llama3",
                "factor": self.rope_scaling.factor,
                "low_freq_factor": self.rope_scaling.low_freq_factor,
                "high_freq_factor": self.rope_scaling.high_freq_factor,
                "original_max_position_embeddings": self.rope_scaling.original_max_position_embeddings,
            },
            "attn_temperature_tuning": self.attn_temperature_tuning,
            "floor_scale": self.floor_scale,
            "attn_scale": self.attn_scale,
            "tie_word_embeddings": False,
            "torch_dtype": self.torch_dtype,
        }
        for k in ("max_position_embeddings", "bos_token_id", "eos_token_id", "pad_token_id"):
            if getattr(self, k) is not None:
                text[k] = getattr(self, k)
        if architecture == "Llama4ForConditionalGeneration":
            return {"architectures": [architecture], "model_type": "llama4", "text_config": text,
                    "torch_dtype": self.torch_dtype}
        return {"architectures": [architecture], **text}

    # ------------------------------------------------------------------- plan
    def plan(self) -> ModelPlan:
        """The layer-by-layer description that the generic model is built from.

        RoPE layers attend within their chunk (keys of the query's own
        ``attention_chunk_size``-aligned block), rotate q and k by interleaved
        pairs and, if ``use_qk_norm``, L2-normalise them without a weight
        (``model.py:913-917``).  NoPE layers attend to every earlier key and,
        with ``attn_temperature_tuning``, scale each query by
        ``1 + attn_scale * ln(1 + floor((pos + 1) / floor_scale))``.
        """
        rope = part(
            "rope_interleaved",
            theta=self.rope_theta,
            scaling=None if self.rope_scaling is None else dataclasses.asdict(self.rope_scaling),
        )
        layers = []
        moe = set(self.moe_layers)
        for i in range(self.num_hidden_layers):
            uses_rope = bool(self.no_rope_layers[i])
            common = dict(
                hidden_size=self.hidden_size,
                num_heads=self.num_attention_heads,
                num_kv_heads=self.num_key_value_heads,
                head_dim=self.head_dim,
                softmax_scale=self.head_dim ** -0.5,  # model.py:774
            )
            if uses_rope:
                mixer = part(
                    "attention",
                    **common,
                    position=rope,
                    qk_norm=part("rmsnorm", eps=self.rms_norm_eps, weighted=False) if self.use_qk_norm else None,
                    retention=("all",) if self.attention_chunk_size is None else ("chunk", self.attention_chunk_size),
                    query_scale=None,
                )
            else:
                mixer = part(
                    "attention",
                    **common,
                    position=part("none"),
                    qk_norm=None,
                    retention=("all",),
                    query_scale=part("log_floor_temperature", floor_scale=self.floor_scale, attn_scale=self.attn_scale)
                    if self.attn_temperature_tuning
                    else None,
                )
            if i in moe:
                ffn = part(
                    "moe_sigmoid_shared",
                    hidden_size=self.hidden_size,
                    num_experts=self.num_local_experts,
                    top_k=self.num_experts_per_tok,
                    intermediate_size=self.intermediate_size,
                    shared_intermediate_size=self.intermediate_size,  # one shared expert (model.py:146)
                )
            else:
                ffn = part("dense_swiglu", hidden_size=self.hidden_size, intermediate_size=self.intermediate_size_mlp)
            norm = part("rmsnorm", eps=self.rms_norm_eps, weighted=True, size=self.hidden_size)
            layers.append(LayerSpec(mixer=mixer, feed_forward=ffn, mixer_norm=norm, feed_forward_norm=norm))
        return ModelPlan(
            vocab_size=self.vocab_size,
            hidden_size=self.hidden_size,
            layers=tuple(layers),
            order=default_order(self.num_hidden_layers),
            final_norm=part("rmsnorm", eps=self.rms_norm_eps, weighted=True, size=self.hidden_size),
            tie_word_embeddings=False,
        )
