"""How a layer's parts are arranged.

``pre_norm`` (``llama4/llama4_jax/model.py:1166-1183``):
``h = x + mixer(norm(x))`` then ``x' = h + feed_forward(norm(h))``.  The residual
sum is kept in float32; adding a branch's output and the following norm are
one kernel, so a branch's output is *pending* on the residual until the next
norm (or the end of the model) applies it.
"""
from __future__ import annotations

from ..config.specs import LayerSpec
from .base import build_feed_forward, build_mixer, build_norm

_ARRANGEMENTS = {}


def register_arrangement(name: str):
    def deco(cls):
        _ARRANGEMENTS[name] = cls
        return cls

    return deco


def build_block(spec: LayerSpec):
    try:
        cls = _ARRANGEMENTS[spec.arrangement]
    except KeyError:
        raise KeyError(f"unknown arrangement {spec.arrangement!r}; registered: {sorted(_ARRANGEMENTS)}") from None
    return cls(spec)


@register_arrangement("pre_norm")
class PreNormBlock:
    def __init__(self, spec: LayerSpec) -> None:
        self.spec = spec
        self.mixer = build_mixer(spec.mixer)
        self.feed_forward = build_feed_forward(spec.feed_forward)
        self.mixer_norm = build_norm(spec.mixer_norm)
        self.feed_forward_norm = build_norm(spec.feed_forward_norm)

    def parts(self):
        return {
            "mixer": self.mixer,
            "feed_forward": self.feed_forward,
            "mixer_norm": self.mixer_norm,
            "feed_forward_norm": self.feed_forward_norm,
        }

    def forward(self, residual, ctx, cache) -> None:
        h, _ = self.mixer_norm.forward(residual, ctx)
        residual.add(self.mixer.forward(h, ctx, cache))
        ff = self.feed_forward
        if getattr(ff, "accepts_deferred_norm", False):  # (it hands the rows to the kernel set only: see there)
            h, h32 = self.feed_forward_norm.forward(residual, ctx, want32=ff.wants_float32_input, defer=True)
        else:
            h, h32 = self.feed_forward_norm.forward(residual, ctx, want32=ff.wants_float32_input)
        residual.add(ff.forward(h, h32, ctx))
