"""RMS norm (``llama4/llama4_jax/model.py:885-888``): ``x / sqrt(mean(x^2) + eps) * weight``,
statistics in float32, eps inside the root, the weight used as it is (not ``1 + weight``)."""
from __future__ import annotations

from .base import Norm, ParamSpec, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    def __init__(self, spec) -> None:
        super().__init__()
        self.eps = float(spec.eps)
        self.weighted = bool(spec.get("weighted", True))
        self.size = spec.get("size")

    graph_safe = True

    def param_specs(self):
        if not self.weighted:
            return {}
        return {"weight": ParamSpec((int(self.size),), policy="float32", init=("ones",))}

    def forward(self, residual, ctx, want32: bool = False, defer: bool = False):
        return residual.normed(ctx, self.params.get("weight"), self.eps, want32, defer)
