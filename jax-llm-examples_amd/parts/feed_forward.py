"""Feed-forward parts.

``dense_swiglu``: ``(silu(x Wg) * (x Wu)) Wd`` (``llama4/llama4_jax/model.py:1142-1153``).
``moe_sigmoid_shared``: router logits in float32, the ``top_k`` largest per token,
gate = sigmoid of the chosen logit, the gate multiplies the expert's *input*
(``model.py:958-972, 1066-1071``), SwiGLU experts (``model.py:1076-1085``), sum
over the chosen experts (``model.py:1111``), plus one shared SwiGLU expert on the
unscaled input (``model.py:1137-1139``).
"""
from __future__ import annotations

from typing import Optional

import torch

from .base import FeedForward, ParamSpec, register_feed_forward


@register_feed_forward("dense_swiglu")
class DenseSwiGLU(FeedForward):
    def __init__(self, spec) -> None:
        super().__init__()
        self.hidden = int(spec.hidden_size)
        self.inter = int(spec.intermediate_size)

    def param_specs(self):
        return {
            "w_gate_up": ParamSpec((2 * self.inter, self.hidden)),  # gate rows, then up rows
            "w_down": ParamSpec((self.hidden, self.inter)),
        }

    graph_safe = True

    def forward(self, h: torch.Tensor, h32: Optional[torch.Tensor], ctx) -> torch.Tensor:
        ops = ctx.ops
        return ops.linear(ops.swiglu_linear(h, self.params["w_gate_up"]), self.params["w_down"])


@register_feed_forward("moe_sigmoid_shared")
class MoESigmoidShared(FeedForward):
    wants_float32_input = True
    # h and h32 go to the kernel set's router and expert products only, which take rows that are not computed yet
    # (the router of a step of few tokens does addition, norm, logits, choice and grouping in one launch)
    accepts_deferred_norm = True

    def __init__(self, spec) -> None:
        super().__init__()
        self.hidden = int(spec.hidden_size)
        self.num_experts = int(spec.num_experts)
        self.top_k = int(spec.top_k)
        self.inter = int(spec.intermediate_size)
        self.shared_inter = int(spec.get("shared_intermediate_size") or 0)
        self.tiled = False  # expert matrices are in the kernels' streaming layout (ops/layout.py)

    def param_specs(self):
        e, f, d = self.num_experts, self.inter, self.hidden
        specs = {
            "router": ParamSpec((e, d), policy="float32"),
            "w_gate_up": ParamSpec((e, 2 * f, d)),  # per expert [out, in]: gate rows, then up rows
            "w_down": ParamSpec((e, d, f)),
        }
        if self.shared_inter:
            specs["shared_gate_up"] = ParamSpec((2 * self.shared_inter, d))
            specs["shared_down"] = ParamSpec((d, self.shared_inter))
        return specs

    graph_safe = True

    def step_weight_bytes(self, observed=None) -> int:
        """Of the routed experts only those that some token of the step chose (``observed``: the
        ``(expert ids, gates)`` this part handed to the step's tap; without it, all)."""
        n = self.num_experts if observed is None else int(torch.unique(observed[0]).numel())
        total = 0
        for name, t in self.params.items():
            b = t.numel() * t.element_size()
            total += b // self.num_experts * n if name in ("w_gate_up", "w_down") else b
        return total

    def flops_per_token(self) -> float:
        per = 0
        for name, t in self.params.items():
            per += t.numel() // self.num_experts * self.top_k if name in ("w_gate_up", "w_down") else t.numel()
        return 2.0 * per

    def finalize(self) -> None:
        from ..ops.layout import can_tile, tile_

        gu, dn = self.params["w_gate_up"], self.params["w_down"]
        if not self.tiled and can_tile(gu) and can_tile(dn) and self.inter % 16 == 0:
            tile_(gu)
            tile_(dn)
            self.tiled = True

    def forward(self, h: torch.Tensor, h32: Optional[torch.Tensor], ctx) -> torch.Tensor:
        ops = ctx.ops
        expert_ids, gates, grouping = ops.moe_route(h32, self.params["router"], self.top_k, group=True)
        tap = getattr(ctx, "tap", None)
        if tap is not None:  # whoever watches the step sees the choice and may replace it
            replaced = tap(self, "routing", (expert_ids, gates))
            if replaced is not None:
                expert_ids, gates = replaced
                grouping = None
        shared = (self.params["shared_gate_up"], self.params["shared_down"]) if self.shared_inter else None
        return ops.moe_experts(h, expert_ids, gates, self.params["w_gate_up"], self.params["w_down"],
                               shared_weights=shared, tiled=self.tiled, grouping=grouping)
