"""The two ends of a decoder: token embedding and output head.

``token_embedding`` (``llama4/llama4_jax/model.py:1195``): row ``token`` of the table, as the first
value of the float32 residual; optionally times a constant (``multiplier``).
``linear_head`` (``model.py:1204``): float32 logits ``h @ W.T`` with a matrix of its own, or, with
``tied``, with the embedding's table; optionally plus a ``bias`` and squashed by a soft cap
(``cap * tanh(logits / cap)``).  Llama 4 uses neither option: its ends are the two kernels alone.
"""
from __future__ import annotations

import torch

from .base import Embedding, OutputHead, ParamSpec, register_embedding, register_head


@register_embedding("token_embedding")
class TokenEmbedding(Embedding):
    def __init__(self, spec) -> None:
        super().__init__()
        self.vocab_size, self.hidden = int(spec.vocab_size), int(spec.hidden_size)
        m = spec.get("multiplier")
        self.multiplier = None if m is None else float(m)

    graph_safe = True

    def param_specs(self):
        return {"weight": ParamSpec((self.vocab_size, self.hidden))}

    def flops_per_token(self) -> float:
        return 0.0

    def forward(self, token_ids: torch.Tensor, ctx) -> torch.Tensor:
        x = ctx.ops.embed(token_ids, self.params["weight"])
        if self.multiplier is not None:
            x.mul_(self.multiplier)
        return x


@register_head("linear_head")
class LinearHead(OutputHead):
    """Its matrix takes the product kernels' streaming layout where it can (a tied one stays as the
    embedding reads it)."""

    def __init__(self, spec) -> None:
        super().__init__()
        self.vocab_size, self.hidden = int(spec.vocab_size), int(spec.hidden_size)
        self.tied = bool(spec.get("tied", False))
        self.biased = bool(spec.get("bias", False))
        cap = spec.get("softcap")
        self.softcap = None if cap is None else float(cap)
        self.tiled = False

    graph_safe = True

    def param_specs(self):
        specs = {} if self.tied else {"weight": ParamSpec((self.vocab_size, self.hidden))}
        if self.biased:
            specs["bias"] = ParamSpec((self.vocab_size,), policy="float32", init=("normal", 0.02))
        return specs

    def finalize(self) -> None:
        from ..ops.layout import can_tile, tile_

        if not self.tied and not self.tiled and can_tile(self.params["weight"]):
            tile_(self.params["weight"])
            self.tiled = True

    def matrix(self, embedding) -> torch.Tensor:
        return embedding.params["weight"] if self.tied else self.params["weight"]

    def step_bytes(self, embedding) -> int:
        w = self.matrix(embedding)
        return self.step_weight_bytes() + (w.numel() * w.element_size() if self.tied else 0)

    def flops_per_token(self) -> float:
        return 2.0 * self.vocab_size * self.hidden

    def forward(self, h: torch.Tensor, ctx, embedding) -> torch.Tensor:
        logits = ctx.ops.lm_head(h, self.matrix(embedding), tiled=self.tiled)
        if self.biased:
            logits.add_(self.params["bias"])
        if self.softcap is not None:
            logits = torch.tanh(logits / self.softcap) * self.softcap
        return logits
