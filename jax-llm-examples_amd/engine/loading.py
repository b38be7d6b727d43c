"""From a model folder (or a configuration) to a model ready to step."""
from __future__ import annotations

import os

import torch

from ..config.registry import architecture_name, get_architecture, read_config_json
from ..parts.model import DecoderModel
from ..weights.loader import load_weights
from ..weights.random_init import init_random_

_DTYPES = {
    "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
    "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"run dtype must be bfloat16 or float32, got {name}")
        return name
    try:
        return _DTYPES[str(name).lower()]
    except KeyError:
        raise ValueError(f"run dtype must be bfloat16 or float32, got {name!r}") from None


def get_ops(device, reference_ops: bool = False):
    """The kernel set for ``device``.  On a GPU that is the compiled HIP library
    (an error if it cannot be built or loaded: there is no fallback).  The plain
    PyTorch ops are handed out only when asked for by name, for tests of the
    engine's logic on a machine without a GPU."""
    device = torch.device(device)
    if reference_ops:
        from ..ops.reference import ReferenceOps

        return ReferenceOps()
    if device.type != "cuda":
        raise RuntimeError(
            f"the engine runs on a GPU (got device {device}); the plain PyTorch ops exist for tests only "
            "and must be asked for with reference_ops=True"
        )
    from ..ops.hip import HipOps

    return HipOps(device)


def build_model(arch, cfg, dtype, device) -> DecoderModel:
    model = DecoderModel(arch.plan(cfg), parse_dtype(dtype), device)
    model.arch, model.config = arch, cfg
    return model


def load_model(model_dir, dtype="bfloat16", device="cuda:0") -> DecoderModel:
    """config.json picks the architecture; model.safetensors fills the weights."""
    top = read_config_json(model_dir)
    arch = get_architecture(architecture_name(top))
    cfg = arch.parse_config(top)
    model = build_model(arch, cfg, dtype, device)
    model.allocate()
    load_weights(model, os.fspath(model_dir), arch.bindings(cfg, model.plan),
                 optional_prefixes=getattr(arch, "optional_prefixes", ()),
                 ignored_prefixes=getattr(arch, "ignored_prefixes", ()))
    return model


def random_model(arch, cfg, seed: int, dtype="bfloat16", device="cuda:0") -> DecoderModel:
    """A model whose weights are drawn in place on the device (benchmarks)."""
    model = build_model(arch, cfg, dtype, device)
    model.allocate()
    init_random_(model, seed)
    return model
