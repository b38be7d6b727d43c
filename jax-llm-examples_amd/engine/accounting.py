"""Bytes a decode step has to read and floating-point operations a prefill step has to
do, counted from the model's own parts (for roofline fractions in benchmarks)."""
from __future__ import annotations

from ..parts.attention import Attention
from ..parts.base import first_needed_position
from ..parts.feed_forward import MoESigmoidShared


def _nbytes(t) -> int:
    return t.numel() * t.element_size()


def decode_step_bytes(model, cache, contexts, distinct_experts=None) -> dict:
    """Every weight the step uses once (of routed experts only those some token chose:
    ``distinct_experts[layer] = count``; embedding: one row per token) plus the keys and values
    visible to each live request (``contexts``: tokens in the cache after the step)."""
    weights = 0
    for i, e in enumerate(model.plan.order):
        b = model.blocks[e.layer]
        for part in b.parts().values():
            if isinstance(part, MoESigmoidShared):
                n = part.num_experts if distinct_experts is None else distinct_experts.get(e.layer, part.num_experts)
                for name, t in part.params.items():
                    if name in ("w_gate_up", "w_down"):
                        weights += _nbytes(t) // part.num_experts * n
                    else:
                        weights += _nbytes(t)
            else:
                weights += sum(_nbytes(t) for t in part.params.values())
    weights += sum(_nbytes(t) for t in model.final_norm.params.values())
    head = model.embed if model.lm_head is None else model.lm_head
    weights += _nbytes(head.params["weight"])
    weights += len(contexts) * model.plan.hidden_size * model.embed.params["weight"].element_size()
    kv = 0
    item = next(iter(cache.groups[0].tensors.values())).element_size() if cache.groups else 0
    for g in cache.groups:
        for c in contexts:
            visible = c - first_needed_position(g.retention, c - 1)
            kv += visible * g.bytes_per_token(item)
    return {"weights": weights, "kv": kv, "total": weights + kv}


def prefill_flops(model, num_tokens: int, start: int = 0) -> float:
    """2 x (weights every token passes through) x tokens, the output head for one row, and
    attention's two products over the keys each query can see."""
    per_token = 0
    attn = 0.0
    for e in model.plan.order:
        b = model.blocks[e.layer]
        m, ff = b.mixer, b.feed_forward
        for name, t in m.params.items():
            per_token += t.numel()
        if isinstance(ff, MoESigmoidShared):
            for name, t in ff.params.items():
                if name in ("w_gate_up", "w_down"):
                    per_token += t.numel() // ff.num_experts * ff.top_k
                else:
                    per_token += t.numel()
        else:
            per_token += sum(t.numel() for t in ff.params.values())
        if isinstance(m, Attention):
            keys = 0
            for p in range(start, start + num_tokens):
                keys += p - first_needed_position(m.retention, p) + 1
            attn += 4.0 * m.num_heads * m.head_dim * keys
    head = model.embed if model.lm_head is None else model.lm_head
    return 2.0 * per_token * num_tokens + 2.0 * head.params["weight"].numel() + attn
