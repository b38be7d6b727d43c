"""Descriptions of model parts as data.

A model is described by a :class:`ModelPlan`: a list of :class:`LayerSpec`
(one per distinct layer, each naming its mixer, feed-forward, norms and their
arrangement as :class:`PartSpec` values) and an ``order`` (the list of
:class:`OrderEntry` that says which layer runs when and whose cache it uses).
A ``PartSpec`` is only a ``kind`` (the name under which the part's class is
registered) and the part's own sizes and constants.  Nothing here knows an
architecture; architectures produce plans from their configuration.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Mapping


@dataclasses.dataclass(frozen=True)
class PartSpec:
    """``kind`` picks the registered class, ``params`` are its constructor arguments."""

    kind: str
    params: Mapping[str, Any] = dataclasses.field(default_factory=dict)

    def __getattr__(self, name: str) -> Any:
        params = object.__getattribute__(self, "params")
        if name in params:
            return params[name]
        raise AttributeError(f"part spec {object.__getattribute__(self, 'kind')!r} has no parameter {name!r}")

    def get(self, name: str, default: Any = None) -> Any:
        return self.params.get(name, default)

    def __hash__(self) -> int:  # params may hold lists / dicts
        return hash((self.kind, repr(sorted(self.params.items(), key=lambda kv: kv[0]))))


def part(kind: str, **params: Any) -> PartSpec:
    return PartSpec(kind, dict(params))


@dataclasses.dataclass(frozen=True)
class LayerSpec:
    """One decoder layer: which parts it is made of and how they are arranged."""

    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    feed_forward_norm: PartSpec
    arrangement: str = "pre_norm"


@dataclasses.dataclass(frozen=True)
class OrderEntry:
    """One item of the run order.

    ``layer`` indexes ``ModelPlan.layers``.  ``cache`` names the cache this run
    uses (an integer id; runs with the same id see the same keys and values).
    ``writes_cache`` is False for a run that only reads a cache another run
    fills (that run must come earlier in the order).
    """

    layer: int
    cache: int
    writes_cache: bool = True


@dataclasses.dataclass(frozen=True)
class ModelPlan:
    vocab_size: int
    hidden_size: int
    layers: tuple[LayerSpec, ...]
    order: tuple[OrderEntry, ...]
    final_norm: PartSpec
    tie_word_embeddings: bool = False
    # the model's two ends; None: a plain token table and a plain linear head (tied if tie_word_embeddings)
    embedding: PartSpec | None = None
    head: PartSpec | None = None

    def __post_init__(self) -> None:
        seen_write: dict[int, int] = {}
        for pos, e in enumerate(self.order):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"order[{pos}] names layer {e.layer}, the plan has {len(self.layers)} layers")
            if e.writes_cache:
                if e.cache in seen_write:
                    raise ValueError(
                        f"order[{pos}] and order[{seen_write[e.cache]}] both write cache {e.cache}; "
                        "a layer that runs twice needs a cache id for each run"
                    )
                seen_write[e.cache] = pos
            elif e.cache not in seen_write:
                raise ValueError(f"order[{pos}] reads cache {e.cache} before any run has written it")


def default_order(num_layers: int) -> tuple[OrderEntry, ...]:
    """Every layer once, in index order, each with a cache of its own."""
    return tuple(OrderEntry(layer=i, cache=i) for i in range(num_layers))
