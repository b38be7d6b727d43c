"""One registry from an architecture's name (``config.json["architectures"][0]``)
to the object that knows how to read its configuration, plan its layers and
name its checkpoint tensors.

The reference has no registry: ``load_config`` reads ``text_config`` of one
fixed architecture (``llama4/llama4_jax/model.py:229-231``).
"""
from __future__ import annotations

import json
import os
from typing import Any, Mapping, Protocol

from .specs import ModelPlan


class Architecture(Protocol):
    """What an architecture has to provide.

    ``parse_config`` turns a whole config.json into a typed configuration;
    ``plan`` turns that into a :class:`ModelPlan`; ``bindings`` lists, for a
    plan, every checkpoint tensor with its stored shape, the model parameter it
    lands in and how (see ``weights.bindings.TensorBinding``).
    """

    names: tuple[str, ...]

    def parse_config(self, top: Mapping[str, Any]) -> Any: ...

    def plan(self, cfg: Any) -> ModelPlan: ...

    def bindings(self, cfg: Any, plan: ModelPlan) -> list: ...

    def config_to_dict(self, cfg: Any, architecture: str | None = None) -> dict: ...


_ARCHITECTURES: dict[str, Architecture] = {}


class UnknownArchitectureError(KeyError):
    pass


def register_architecture(arch: Architecture) -> Architecture:
    for name in arch.names:
        _ARCHITECTURES[name] = arch
    return arch


def known_architectures() -> list[str]:
    _ensure_builtin()
    return sorted(_ARCHITECTURES)


def get_architecture(name: str) -> Architecture:
    _ensure_builtin()
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise UnknownArchitectureError(
            f"unknown architecture {name!r}; known: {', '.join(sorted(_ARCHITECTURES))}"
        ) from None


def architecture_name(top: Mapping[str, Any]) -> str:
    archs = top.get("architectures")
    if archs:
        return str(archs[0])
    if top.get("model_type"):  # (a folder written without the entry)
        return str(top["model_type"])
    raise UnknownArchitectureError("config.json has neither an 'architectures' entry nor a 'model_type'")


def read_config_json(model_dir: str | os.PathLike) -> dict:
    path = os.path.join(os.fspath(model_dir), "config.json")
    with open(path) as f:
        return json.load(f)


def load_config(model_dir: str | os.PathLike):
    """Returns ``(architecture, typed config)`` for a model folder."""
    top = read_config_json(model_dir)
    arch = get_architecture(architecture_name(top))
    return arch, arch.parse_config(top)


def _ensure_builtin() -> None:
    # importing the module registers the built-in architecture
    from ..parts import llama4 as _llama4  # noqa: F401
