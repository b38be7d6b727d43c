"""Grouped-query attention over the paged cache.

One class covers both of Llama 4's attention layers, by parameters only:
rotary position encoding or none, weightless L2 norm of q and k or none, a
retention rule (every earlier key, or the keys of the query's own chunk), and an
optional position-dependent query scale.  Formulas:
``llama4/llama4_jax/model.py:891-955`` (projections, rotation, q/k norm, order of
the cache write) and ``model.py:745-794`` (scores times ``softmax_scale``, causal
mask, float32 softmax, values).
"""
from __future__ import annotations

import torch

from .base import CacheNeed, Mixer, ParamSpec, build_position, register_mixer


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
        if qk_norm is not None and (qk_norm.kind != "rmsnorm" or qk_norm.get("weighted", False)):
            raise ValueError("the attention mixer supports only a weightless rmsnorm of q and k")
        self.qk_norm_eps = None if qk_norm is None else float(qk_norm.eps)
        qs = spec.get("query_scale")
        if qs is not None and qs.kind != "log_floor_temperature":
            raise ValueError(f"unknown query_scale kind {qs.kind!r}")
        self.query_scale = None if qs is None else (float(qs.floor_scale), float(qs.attn_scale))
        self._inv_freq = None

    def param_specs(self):
        hq, hk, dh, d = self.num_heads, self.num_kv_heads, self.head_dim, self.hidden
        return {
            # rows: q heads, then k heads, then v heads; each [out, in]
            "wqkv": ParamSpec(((hq + 2 * hk) * dh, d)),
            "wo": ParamSpec((d, hq * dh)),
        }

    def cache_need(self) -> CacheNeed:
        return CacheNeed(kv=(self.num_kv_heads, self.head_dim), retention=self.retention)

    def finalize(self) -> None:
        inv = self.position.inv_freq()
        self._inv_freq = None if inv is None else inv.to(self.params["wqkv"].device)

    def forward(self, h: torch.Tensor, ctx, cache) -> torch.Tensor:
        ops = ctx.ops
        qkv = ops.linear(h, self.params["wqkv"])
        q = ops.qk_prepare_kv_write(
            qkv,
            self.num_heads,
            self.num_kv_heads,
            self.head_dim,
            ctx.positions,
            self._inv_freq,
            self.qk_norm_eps,
            self.query_scale,
            cache.kv if cache.writes else None,
            cache.slot_mapping,
        )
        o = ops.paged_attention(
            q, cache.kv, cache.block_table, ctx.positions, ctx.token_segment, self.retention,
            self.softmax_scale, cache.attn_meta,
        )
        return ops.linear(o, self.params["wo"])
