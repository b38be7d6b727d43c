"""Grouped-query attention over the paged cache.

One class covers both of Llama 4's attention layers, by parameters only:
a position encoding that says how q and k are rotated (or none), an RMS norm of q
and k or none (weightless after the rotation for Llama 4; weights and the place
before the rotation are options), a retention rule (every earlier key, or the keys of the query's own chunk), and an
optional position-dependent query scale.  Formulas:
``llama4/llama4_jax/model.py:891-955`` (projections, rotation, q/k norm, order of
the cache write) and ``model.py:745-794`` (scores times ``softmax_scale``, causal
mask, float32 softmax, values).
"""
from __future__ import annotations

import torch

from .base import CacheNeed, Mixer, ParamSpec, QKPreparation, build_position, first_needed_position, register_mixer


@register_mixer("attention")
class Attention(Mixer):
    def __init__(self, spec) -> None:
        super().__init__()
        self.hidden = int(spec.hidden_size)
        self.num_heads = int(spec.num_heads)
        self.num_kv_heads = int(spec.num_kv_heads)
        self.head_dim = int(spec.head_dim)
        if self.num_heads % self.num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        self.softmax_scale = float(spec.softmax_scale)
        self.retention = tuple(spec.retention)
        self.position = build_position(spec.position, self.head_dim)
        qk_norm = spec.get("qk_norm")
        if qk_norm is not None and qk_norm.kind != "rmsnorm":
            raise ValueError(f"the attention mixer norms q and k with an rmsnorm, not {qk_norm.kind!r}")
        self.qk_norm_eps = None if qk_norm is None else float(qk_norm.eps)
        self.qk_norm_weighted = bool(qk_norm is not None and qk_norm.get("weighted", False))
        self.qk_norm_first = bool(qk_norm is not None and qk_norm.get("before_rotation", False))
        qs = spec.get("query_scale")
        if qs is not None and qs.kind != "log_floor_temperature":
            raise ValueError(f"unknown query_scale kind {qs.kind!r}")
        self.query_scale = None if qs is None else (float(qs.floor_scale), float(qs.attn_scale))
        self.prep = QKPreparation(norm_eps=self.qk_norm_eps, norm_first=self.qk_norm_first,
                                  query_scale=self.query_scale)

    def param_specs(self):
        hq, hk, dh, d = self.num_heads, self.num_kv_heads, self.head_dim, self.hidden
        return {
            # rows: q heads, then k heads, then v heads; each [out, in]
            "wqkv": ParamSpec(((hq + 2 * hk) * dh, d)),
            "wo": ParamSpec((d, hq * dh)),
            **({"q_norm": ParamSpec((dh,), policy="float32", init=("ones",)),
                "k_norm": ParamSpec((dh,), policy="float32", init=("ones",))} if self.qk_norm_weighted else {}),
        }

    def cache_need(self) -> CacheNeed:
        return CacheNeed(kv=(self.num_kv_heads, self.head_dim), retention=self.retention)

    graph_safe = True

    def finalize(self) -> None:
        rot = self.position.rotation()
        if rot is not None:
            rot.inv_freq = rot.inv_freq.to(self.params["wqkv"].device)
        self.prep.rotation = rot
        self.prep.norm_weight_q = self.params.get("q_norm")
        self.prep.norm_weight_k = self.params.get("k_norm")

    def mixing_flops(self, start: int, count: int) -> float:
        """Two products (scores, values) over the keys each query can see."""
        keys = sum(p - first_needed_position(self.retention, p) + 1 for p in range(start, start + count))
        return 4.0 * self.num_heads * self.head_dim * keys

    def forward(self, h: torch.Tensor, ctx, cache) -> torch.Tensor:
        ops = ctx.ops
        qkv = ops.linear(h, self.params["wqkv"])
        o = ops.attention_from_qkv(
            qkv, self.num_heads, self.num_kv_heads, self.head_dim, ctx.positions, ctx.token_segment, self.prep,
            cache.kv, cache.writes, cache.slot_mapping, cache.block_table, self.retention, self.softmax_scale,
            cache.attn_meta,
        )
        return ops.linear(o, self.params["wo"])
