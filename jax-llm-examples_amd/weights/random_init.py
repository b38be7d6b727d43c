"""Seeded random weights.

``write_random_model`` writes a model folder (``config.json`` and
``model.safetensors`` with the checkpoint's own tensor names and layouts) from a
configuration and a seed: every matrix N(0, 0.02), norm weights 1.  Each
tensor's generator is seeded from ``(seed, tensor name)``, so a tensor's values
do not depend on which others exist or in which order they are drawn.  (The
reference draws one key per leaf by splitting one key in pytree order,
``llama4/llama4_jax/model.py:270-307``.)

``init_random_`` fills a model's parameters in place on its device, for
benchmarks whose weights would not fit a disk or host memory.
"""
from __future__ import annotations

import hashlib
import json
import os

import torch

from .bindings import TensorBinding
from .safetensors_io import write_safetensors


def _seed_for(seed: int, name: str) -> int:
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & 0x7FFFFFFFFFFFFFFF


def draw(b: TensorBinding, seed: int, dtype: torch.dtype) -> torch.Tensor:
    if b.init[0] == "ones":
        return torch.ones(b.shape, dtype=dtype)
    if b.init[0] == "normal":
        g = torch.Generator().manual_seed(_seed_for(seed, b.name))
        return (torch.randn(b.shape, generator=g, dtype=torch.float32) * float(b.init[1])).to(dtype)
    raise ValueError(f"unknown init {b.init!r}")


def write_random_model(arch, cfg, out_dir: str, seed: int, dtype: torch.dtype = torch.float32,
                       architecture: str | None = None) -> str:
    os.makedirs(out_dir, exist_ok=True)
    plan = arch.plan(cfg)
    bindings = arch.bindings(cfg, plan)
    prefix = arch.checkpoint_prefix(architecture) if hasattr(arch, "checkpoint_prefix") else ""
    specs = [(prefix + b.name, torch.float32 if b.float32 else dtype, tuple(b.shape)) for b in bindings]

    def gen():
        for b, (name, dt, _) in zip(bindings, specs):
            yield name, draw(b, seed, dt)

    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(arch.config_to_dict(cfg, architecture), f, indent=1)
    write_safetensors(os.path.join(out_dir, "model.safetensors"), gen(), specs)
    return out_dir


@torch.no_grad()
def init_random_(model, seed: int, std: float = 0.02) -> None:
    """Fills every parameter in place on the model's device: matrices N(0, std)
    drawn in float32 and rounded to the parameter's dtype, norm weights 1."""
    specs = model.param_specs()
    params = model.named_parameters()
    for name, t in params.items():
        init = specs[name].init
        if init[0] == "ones":
            t.fill_(1.0)
            continue
        g = torch.Generator(device=t.device).manual_seed(_seed_for(seed, name))
        s = float(init[1]) if init[0] == "normal" else std
        flat = t.view(-1)
        step = 1 << 28  # draw in pieces: no float32 copy of a whole large tensor
        for o in range(0, flat.numel(), step):
            n = min(step, flat.numel() - o)
            flat[o: o + n].copy_(torch.randn(n, generator=g, dtype=torch.float32, device=t.device) * s)
    model.finalize()
