"""Loading a model folder's safetensors into a model, by tensor name.

The reference converts checkpoints in two stages with per-tensor asserts
(``llama4/llama4_jax/chkpt_utils.py:80-159``) and raises on unknown, unexpected,
duplicate and missing names (``chkpt_utils.py:159, 257-261, 274-275``).  Here
the checkpoint is read directly; every problem found (missing tensors,
unexpected tensors, tensors met twice, wrong shapes) is reported in one
:class:`WeightsError`.
"""
from __future__ import annotations

import glob
import json
import os
from typing import Sequence

import torch

from .bindings import TensorBinding
from .safetensors_io import SafetensorsFile


class WeightsError(ValueError):
    def __init__(self, missing, unexpected, wrong_shape, where: str, duplicate=()) -> None:
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.duplicate = list(duplicate)  # (name, where it was met first, where again)
        lines = [f"weights in {where} do not match the model:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.duplicate:
            lines.append(f"  met twice ({len(self.duplicate)}): " + ", ".join(
                f"{n} ({a} and {b})" for n, a, b in self.duplicate))
        if self.wrong_shape:
            lines.append(f"  wrong shape ({len(self.wrong_shape)}): " + ", ".join(
                f"{n} is {list(got)}, expected {list(exp)}" for n, got, exp in self.wrong_shape))
        super().__init__("\n".join(lines))


def _checkpoint_files(model_dir: str) -> list[str]:
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.exists(index):
        with open(index) as f:
            names = sorted(set(json.load(f)["weight_map"].values()))
        return [os.path.join(model_dir, n) for n in names]
    single = os.path.join(model_dir, "model.safetensors")
    if os.path.exists(single):
        return [single]
    files = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
    if not files:
        raise FileNotFoundError(f"no safetensors file in {model_dir}")
    return files


def _canonical(name: str, optional_prefixes: Sequence[str]) -> str:
    for p in optional_prefixes:
        if name.startswith(p):
            return name[len(p):]
    return name


def load_weights(model, model_dir: str, bindings: list[TensorBinding], *, optional_prefixes: Sequence[str] = (),
                 ignored_prefixes: Sequence[str] = ()) -> None:
    """Fills ``model``'s parameters.  Tensors are converted to each parameter's
    own dtype: the run dtype, or float32 for parameters that are always held in
    float32 (norm weights, routers) - so a tensor of those that the checkpoint
    stores in 32-bit stays as it is.  Integer tensors become int32."""
    files = [SafetensorsFile(p) for p in _checkpoint_files(os.fspath(model_dir))]
    try:
        found: dict[str, tuple[SafetensorsFile, str]] = {}
        duplicate = []
        for f in files:
            for raw in f.names():
                if any(raw.startswith(p) for p in ignored_prefixes):
                    continue
                name = _canonical(raw, optional_prefixes)
                if name in found:
                    # in two files, or once with and once without an optional prefix: which one is meant cannot
                    # be known (the reference refuses a parameter that is set twice, chkpt_utils.py:261)
                    f0, raw0 = found[name]
                    duplicate.append((name, f"{raw0} in {os.path.basename(f0.path)}",
                                      f"{raw} in {os.path.basename(f.path)}"))
                    continue
                found[name] = (f, raw)
        expected = {b.name: b for b in bindings}
        missing = [n for n in expected if n not in found]
        unexpected = [n for n in found if n not in expected]
        wrong = []
        for n, b in expected.items():
            if n in found:
                f, raw = found[n]
                if f.shape(raw) != tuple(b.shape):
                    wrong.append((n, f.shape(raw), tuple(b.shape)))
        if missing or unexpected or wrong or duplicate:
            raise WeightsError(missing, unexpected, wrong, os.fspath(model_dir), duplicate)
        params = model.named_parameters()
        for n, b in expected.items():
            f, raw = found[n]
            place(params[b.target], b, f.tensor(raw))
    finally:
        for f in files:
            f.close()
    model.finalize()


def place(target: torch.Tensor, b: TensorBinding, t: torch.Tensor) -> None:
    if not t.dtype.is_floating_point and t.dtype != torch.bool:
        t = t.to(torch.int32)
    if b.transpose is not None:
        t = t.transpose(*b.transpose)
    dst = target if b.rows is None else target[b.rows[0]: b.rows[1]]
    if tuple(dst.shape) != tuple(t.shape):
        raise AssertionError(f"binding {b.name}: {tuple(t.shape)} does not fit {b.target}{tuple(dst.shape)}")
    dst.copy_(t)
