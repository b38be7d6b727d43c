"""Interfaces of the parts a layer is put together from, and their registries.

Four kinds of part exist: *mixers* (what moves information between positions:
attention here), *feed-forwards* (dense or routed experts), *norms* and
*position encodings*.  Each is a class registered under a ``kind`` name and
built from a :class:`~..config.specs.PartSpec`; none knows which model it is
in.  A part declares its parameters (:class:`ParamSpec`), a mixer declares
what it needs from the cache manager (:class:`CacheNeed`: pages of keys and
values with a retention rule, and/or a fixed-size per-request state).

Adding a part = writing a class with the interface below and calling the
matching ``register_*`` once; no framework file has to change.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Callable, Optional

import torch

from ..config.specs import PartSpec


# --------------------------------------------------------------------------- parameters
@dataclasses.dataclass(frozen=True)
class ParamSpec:
    """Shape and storage policy of one parameter tensor.

    ``policy``: ``"compute"`` tensors are held in the run dtype (bfloat16 or
    float32); ``"float32"`` tensors (norm weights, router matrices) are always
    held in float32, which loses nothing of a bfloat16 checkpoint and keeps a
    tensor that the checkpoint stores in 32-bit as it is.
    ``init``: ``("normal", std)`` or ``("ones",)`` for seeded random weights.
    """

    shape: tuple[int, ...]
    policy: str = "compute"
    init: tuple = ("normal", 0.02)


class Part:
    """Base of every part: owns named parameter tensors."""

    def __init__(self) -> None:
        self.params: dict[str, torch.Tensor] = {}

    def param_specs(self) -> dict[str, ParamSpec]:
        return {}

    def allocate(self, dtype: torch.dtype, device: torch.device) -> None:
        for name, ps in self.param_specs().items():
            dt = torch.float32 if ps.policy == "float32" else dtype
            self.params[name] = torch.empty(ps.shape, dtype=dt, device=device)

    def finalize(self) -> None:
        """Called once after all parameters are filled."""


# --------------------------------------------------------------------------- cache needs
@dataclasses.dataclass(frozen=True)
class CacheNeed:
    """What one run of a mixer needs from the cache manager.

    ``kv``: ``None`` or ``(num_kv_heads, head_dim)``, keys and values per token.
    ``retention``: which earlier tokens a query at position ``p`` may still read:
    ``("all",)``; ``("chunk", C)``: those with ``pos >= (p // C) * C``;
    ``("window", W)``: those with ``pos > p - W``.  Pages that hold only
    tokens no later query can read are given back.
    ``state_shape``/``state_dtype``: fixed-size state per request (``None`` if the mixer has none).
    """

    kv: Optional[tuple[int, int]] = None
    retention: tuple = ("all",)
    state_shape: Optional[tuple[int, ...]] = None
    state_dtype: Optional[torch.dtype] = None


def first_needed_position(retention: tuple, next_pos: int) -> int:
    """Smallest position that a query at ``next_pos`` or later can still read."""
    kind = retention[0]
    if kind == "all":
        return 0
    if kind == "chunk":
        c = int(retention[1])
        return (next_pos // c) * c
    if kind == "window":
        return max(0, next_pos - int(retention[1]) + 1)
    raise ValueError(f"unknown retention rule {retention!r}")


# --------------------------------------------------------------------------- interfaces
class Mixer(Part):
    """``forward(h, ctx, cache)``: ``h`` is ``[N, hidden]`` in the run dtype (the
    normed residual of all tokens of the step, segments concatenated); returns
    ``[N, hidden]``.  ``ctx`` is the step's :class:`~..engine.batch.StepContext`
    (positions, segment bounds, state slots, the kernel set); ``cache`` is the
    :class:`~..cache.manager.CacheView` of this run (its key/value pages, block
    tables and slot mapping of its group, its state tensor, whether it writes).
    A mixer must give the same result however a request's tokens are cut into
    steps."""

    def cache_need(self) -> CacheNeed:
        return CacheNeed()

    def forward(self, h: torch.Tensor, ctx: Any, cache: Any) -> torch.Tensor:  # pragma: no cover
        raise NotImplementedError


class FeedForward(Part):
    """``forward(h, h32, ctx)``: token-wise; ``h`` ``[N, hidden]`` in the run dtype,
    ``h32`` the same rows in float32 if ``wants_float32_input`` (for router
    logits), else ``None``.  Returns ``[N, hidden]``."""

    wants_float32_input = False

    def forward(self, h: torch.Tensor, h32: Optional[torch.Tensor], ctx: Any) -> torch.Tensor:  # pragma: no cover
        raise NotImplementedError


class Norm(Part):
    """``forward(residual, ctx, want32)``: ``residual`` is the step's
    :class:`~.residual.Residual`; applies what is pending on it and
    returns the normed rows in the run dtype (and in float32 if asked)."""

    def forward(self, residual: Any, ctx: Any, want32: bool = False):  # pragma: no cover
        raise NotImplementedError


class PositionEncoding:
    """Turns integer positions into what the mixer's kernels take.  For rotary
    kinds that is ``inv_freq`` (float32 ``[head_dim/2]``), from which angles
    ``pos * inv_freq`` are formed in float32 inside the kernel."""

    def __init__(self, spec: PartSpec, head_dim: int) -> None:
        self.spec = spec
        self.head_dim = head_dim

    def inv_freq(self) -> Optional[torch.Tensor]:
        return None


# --------------------------------------------------------------------------- registries
_MIXERS: dict[str, Callable[..., Mixer]] = {}
_FEED_FORWARDS: dict[str, Callable[..., FeedForward]] = {}
_NORMS: dict[str, Callable[..., Norm]] = {}
_POSITIONS: dict[str, Callable[..., PositionEncoding]] = {}


def _register(table: dict, what: str):
    def reg(kind: str, cls=None):
        def deco(c):
            table[kind] = c
            return c

        return deco(cls) if cls is not None else deco

    def build(spec: PartSpec, *args, **kw):
        try:
            cls = table[spec.kind]
        except KeyError:
            raise KeyError(f"unknown {what} kind {spec.kind!r}; registered: {', '.join(sorted(table))}") from None
        return cls(spec, *args, **kw)

    return reg, build


register_mixer, build_mixer = _register(_MIXERS, "mixer")
register_feed_forward, build_feed_forward = _register(_FEED_FORWARDS, "feed-forward")
register_norm, build_norm = _register(_NORMS, "norm")
register_position, build_position = _register(_POSITIONS, "position encoding")
