"""Interfaces of the parts a layer is put together from, and their registries.

A layer is put together from four kinds of part: *mixers* (what moves information
between positions: attention here), *feed-forwards* (dense or routed experts), *norms* and
*position encodings*; a model has an *embedding* before its layers and an *output head*
behind them.  Each is a class registered under a ``kind`` name and
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

    # A part whose ``forward`` only launches work on the current stream (no copy to the host, no size that
    # depends on values on the device) may be recorded into a HIP graph of the decode step.  Parts that do not
    # say so are always run step by step.
    graph_safe = False

    # ------------------------------------------------------------------ what a step costs (for rooflines)
    def step_weight_bytes(self, observed=None) -> int:
        """Bytes of parameters that one step has to read, each once.  ``observed``: what this part
        handed to the step's tap (see :class:`~..engine.batch.StepContext`), if a tap was installed
        and the part offers something; a part that reads only some of its parameters (routed
        experts) counts from it."""
        return sum(t.numel() * t.element_size() for t in self.params.values())

    def flops_per_token(self) -> float:
        """Floating-point operations of the part's matrix products for one token."""
        return 2.0 * sum(t.numel() for t in self.params.values() if t.dim() >= 2)


# --------------------------------------------------------------------------- cache needs
@dataclasses.dataclass(frozen=True)
class CacheNeed:
    """What one run of a mixer needs from the cache manager.

    ``kv``: ``None`` or ``(num_kv_heads, head_dim)``, keys and values per token.
    ``paged``: further per-token tensors in pages (see below).
    ``retention``: which earlier tokens a query at position ``p`` may still read:
    ``("all",)``; ``("chunk", C)``: those with ``pos >= (p // C) * C``;
    ``("window", W)``: those with ``pos > p - W``; or any rule registered with
    :func:`register_retention`.  Pages that hold only tokens no later query can read are given back.
    ``state_shape``/``state_dtype``: fixed-size state per request (``None`` if the mixer has none).
    """

    kv: Optional[tuple[int, int]] = None
    retention: tuple = ("all",)
    state_shape: Optional[tuple[int, ...]] = None
    state_dtype: Optional[torch.dtype] = None
    # Other things kept per token, in pages of their own under the same retention rule: a tuple of
    # ``(name, per-token shape)`` pairs, e.g. ``(("latent", (96,)),)`` or keys and values of different
    # sizes ``(("k", (2, 24)), ("v", (2, 8)))``.  Each becomes a tensor ``[pages, page_size, *shape]`` in the
    # run dtype that the mixer reads and writes through its block table and slot mapping
    # (``CacheView.pages[name]``).  ``kv`` is the layout the attention kernels read (keys ``[page_size,
    # head_dim]`` and values transposed in one tensor).
    paged: tuple = ()


@dataclasses.dataclass(frozen=True)
class RetentionKind:
    """What the cache manager has to know of a retention rule ``(kind, *parameters)``.

    ``first_needed(rule, next_pos)``: the smallest position, beyond the kept prefix, that a query at
    ``next_pos`` or later can still read.  ``held_at_most(rule, max_step_tokens)``: the most tokens of one
    request that are held at any time (what the rule keeps plus one step's portion, whose pages are
    given back only after the step), or ``None`` if only the sequence's length bounds it.
    ``kept_prefix(rule)``: positions ``[0, kept_prefix)`` stay readable for ever."""

    first_needed: Callable[[tuple, int], int]
    held_at_most: Callable[[tuple, int], Optional[int]]
    kept_prefix: Callable[[tuple], int] = lambda rule: 0


_RETENTIONS: dict[str, RetentionKind] = {}


def register_retention(kind: str, first_needed, held_at_most, kept_prefix=None) -> None:
    """A further retention rule for mixers that read their pages themselves (the attention kernels here read
    keys under ``all``, ``chunk`` and ``window``): the cache manager gives pages back by it and sizes pools by it."""
    _RETENTIONS[kind] = RetentionKind(first_needed, held_at_most, kept_prefix or (lambda rule: 0))


def retention_kind(retention: tuple) -> RetentionKind:
    try:
        return _RETENTIONS[retention[0]]
    except KeyError:
        raise ValueError(f"unknown retention rule {retention!r}; registered: {', '.join(sorted(_RETENTIONS))}") from None


register_retention("all", lambda rule, next_pos: 0, lambda rule, step: None)
register_retention("chunk", lambda rule, next_pos: (next_pos // int(rule[1])) * int(rule[1]),
                   lambda rule, step: int(rule[1]) + step)
register_retention("window", lambda rule, next_pos: max(0, next_pos - int(rule[1]) + 1),
                   lambda rule, step: int(rule[1]) + step)


def first_needed_position(retention: tuple, next_pos: int) -> int:
    """Smallest position (beyond the rule's kept prefix) that a query at ``next_pos`` or later can still read."""
    return retention_kind(retention).first_needed(retention, next_pos)


def kept_prefix(retention: tuple) -> int:
    return retention_kind(retention).kept_prefix(retention)


def readable(retention: tuple, query_pos: int, key_pos: int) -> bool:
    """The rule itself: may the query at ``query_pos`` read the key at ``key_pos``?"""
    return key_pos <= query_pos and (key_pos < kept_prefix(retention)
                                     or key_pos >= first_needed_position(retention, query_pos))


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

    def mixing_flops(self, start: int, count: int) -> float:
        """Floating-point operations of moving information between positions (beyond the matrix
        products of :meth:`flops_per_token`) for ``count`` tokens of one request from position ``start``."""
        return 0.0

    def forward(self, h: torch.Tensor, ctx: Any, cache: Any) -> torch.Tensor:  # pragma: no cover
        raise NotImplementedError


class FeedForward(Part):
    """``forward(h, h32, ctx)``: token-wise; ``h`` ``[N, hidden]`` in the run dtype,
    ``h32`` the same rows in float32 if ``wants_float32_input`` (for router
    logits), else ``None``.  Returns ``[N, hidden]``."""

    wants_float32_input = False
    # A feed-forward that only hands ``h`` / ``h32`` on to the kernel set's products and router may say so: it
    # is then given rows that are not computed yet (the kernel set's ``defer_norm``), which a kernel of its own
    # may compute inside its launch.  One that touches the rows itself leaves this off.
    accepts_deferred_norm = False

    def forward(self, h: torch.Tensor, h32: Optional[torch.Tensor], ctx: Any) -> torch.Tensor:  # pragma: no cover
        raise NotImplementedError


class Norm(Part):
    """``forward(residual, ctx, want32)``: ``residual`` is the step's
    :class:`~.residual.Residual`; applies what is pending on it and
    returns the normed rows in the run dtype (and in float32 if asked)."""

    def forward(self, residual: Any, ctx: Any, want32: bool = False):  # pragma: no cover
        raise NotImplementedError


class Embedding(Part):
    """``forward(token_ids, ctx)``: int32 ``[N]`` token ids to the first residual, float32 ``[N, hidden]``."""

    def forward(self, token_ids: torch.Tensor, ctx: Any) -> torch.Tensor:  # pragma: no cover
        raise NotImplementedError

    def step_bytes(self, num_tokens: int) -> int:
        """Bytes a step of ``num_tokens`` tokens reads of this part (a table: a row per token)."""
        return sum(num_tokens * t.shape[-1] * t.element_size() for t in self.params.values() if t.dim() == 2)


class OutputHead(Part):
    """``forward(h, ctx, embedding)``: the normed rows ``[M, hidden]`` whose logits are wanted, in the run
    dtype, to float32 logits ``[M, vocab]``.  ``embedding`` is the model's embedding part (a tied head takes
    its matrix from there)."""

    def forward(self, h: torch.Tensor, ctx: Any, embedding: Any) -> torch.Tensor:  # pragma: no cover
        raise NotImplementedError

    def step_bytes(self, embedding: Any) -> int:
        """Bytes a step reads of the head's parameters (a tied head: of the embedding's)."""
        return self.step_weight_bytes()


@dataclasses.dataclass
class Rotation:
    """A rotary encoding as data: element pairs of a head are turned by ``pos * inv_freq[j]``.

    ``inv_freq``: float32 ``[rotary_dim / 2]``; the angles are formed in float32 inside the kernel.
    ``pairing``: ``"adjacent"`` pairs ``(x[2j], x[2j+1])``; ``"half"`` pairs ``(x[j], x[j + rotary_dim/2])``.
    ``rotary_dim``: the leading elements of a head that are rotated (the rest pass unchanged)."""

    inv_freq: torch.Tensor
    pairing: str = "adjacent"
    rotary_dim: int = 0


@dataclasses.dataclass
class QKPreparation:
    """What happens to the q and k rows of an attention mixer between the projection and the
    scores, as data the preparation kernel takes: the rotation (from the position encoding), an
    RMS norm over the head with or without weights, before or after the rotation, and a
    position-dependent scale of the queries."""

    rotation: Optional[Rotation] = None
    norm_eps: Optional[float] = None  # None: no norm
    norm_weight_q: Optional[torch.Tensor] = None  # float32 [head_dim]; None: weightless
    norm_weight_k: Optional[torch.Tensor] = None
    norm_first: bool = False  # the norm comes before the rotation
    query_scale: Optional[tuple] = None  # (floor_scale, attn_scale): q *= 1 + attn_scale * ln(1 + floor((pos + 1) / floor_scale))

    @property
    def plain(self) -> bool:
        """The case every kernel takes: adjacent pairs over the whole head, weightless norm after the rotation."""
        r = self.rotation
        return ((r is None or (r.pairing == "adjacent" and r.rotary_dim in (0, 2 * r.inv_freq.numel())))
                and self.norm_weight_q is None and self.norm_weight_k is None and not self.norm_first)


class PositionEncoding:
    """Turns integer positions into what the mixer's kernels take.  Rotary kinds return a
    :class:`Rotation` from :meth:`rotation` (frequencies, which elements pair up, how many are
    rotated); the attention mixer hands it to the kernel that prepares q and k.  Another family
    (additive, learned) is applied by the mixer that names it."""

    def __init__(self, spec: PartSpec, head_dim: int) -> None:
        self.spec = spec
        self.head_dim = head_dim

    def rotation(self) -> Optional[Rotation]:
        return None


# --------------------------------------------------------------------------- registries
_MIXERS: dict[str, Callable[..., Mixer]] = {}
_FEED_FORWARDS: dict[str, Callable[..., FeedForward]] = {}
_NORMS: dict[str, Callable[..., Norm]] = {}
_POSITIONS: dict[str, Callable[..., PositionEncoding]] = {}
_EMBEDDINGS: dict[str, Callable[..., Embedding]] = {}
_HEADS: dict[str, Callable[..., OutputHead]] = {}


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
register_embedding, build_embedding = _register(_EMBEDDINGS, "embedding")
register_head, build_head = _register(_HEADS, "output head")
