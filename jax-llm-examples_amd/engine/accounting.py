"""Bytes a decode step has to read and floating-point operations a prefill step has to
do, counted by the model's own parts (for roofline fractions in benchmarks).  Every part
reports its own numbers (:meth:`~..parts.base.Part.step_weight_bytes`,
:meth:`~..parts.base.Part.flops_per_token`, :meth:`~..parts.base.Mixer.mixing_flops`); nothing
here knows a kind of part."""
from __future__ import annotations

from ..parts.base import first_needed_position, kept_prefix


def _nbytes(t) -> int:
    return t.numel() * t.element_size()


class StepWatcher:
    """A tap that keeps what the parts of a step hand out, by part (``seen[id(part)][name]``)."""

    def __init__(self) -> None:
        self.seen: dict = {}

    def __call__(self, part, name, value):
        self.seen.setdefault(id(part), {})[name] = value
        return None


def decode_step_bytes(model, cache, contexts, watcher: StepWatcher | None = None) -> dict:
    """Every weight the step uses once (a part that reads only some of its weights counts from what
    it handed to ``watcher`` during such a step; embedding: one row per token) plus the keys and
    values visible to each live request (``contexts``: tokens in the cache after the step)."""
    weights = 0
    for e in model.plan.order:
        for part in model.blocks[e.layer].parts().values():
            seen = watcher.seen.get(id(part)) if watcher is not None else None
            observed = next(iter(seen.values())) if seen else None
            weights += part.step_weight_bytes(observed)
    weights += model.final_norm.step_weight_bytes()
    weights += model.lm_head.step_bytes(model.embed) + model.embed.step_bytes(len(contexts))
    kv = 0
    for g in cache.groups:
        for c in contexts:
            first = first_needed_position(g.retention, c - 1)
            visible = c - first + min(first, kept_prefix(g.retention))
            kv += visible * g.bytes_per_token()
    return {"weights": weights, "kv": kv, "total": weights + kv}


def prefill_flops(model, num_tokens: int, start: int = 0) -> float:
    """Every part's matrix products for each token, what the mixers do between positions, and the
    output head for one row."""
    per_token = 0.0
    mixing = 0.0
    for e in model.plan.order:
        b = model.blocks[e.layer]
        per_token += sum(p.flops_per_token() for p in b.parts().values())
        mixing += b.mixer.mixing_flops(start, num_tokens)
    return per_token * num_tokens + model.lm_head.flops_per_token() + mixing
