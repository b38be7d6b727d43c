"""Position encodings.

``rope_interleaved``: rotary embedding over adjacent pairs ``(x[2j], x[2j+1])``
(``llama4/llama4_jax/model.py:722-728``) with frequencies
``theta ** -(2j / head_dim)`` (``model.py:706-708``) and, if the configuration has
``rope_scaling``, the llama3 correction (``model.py:654-672``).  Angles are formed
in float32 from integer positions inside the kernel (``model.py:710-718``: a
reduced-precision product here is catastrophic); this part says, as data, which
frequencies there are, which elements pair up and how many of a head are rotated.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from .base import PositionEncoding, Rotation, register_position


@register_position("none")
class NoPosition(PositionEncoding):
    pass


def llama3_scaled_frequencies(inv_freq: torch.Tensor, factor: float, low_freq_factor: float,
                              high_freq_factor: float, original_max_position_embeddings: int) -> torch.Tensor:
    """Wavelengths above ``orig / low`` are stretched by ``factor``; those below
    ``orig / high`` are kept; between, the two are blended linearly in
    ``orig / wavelength``.  With ``low == high`` there is no band between."""
    old = float(original_max_position_embeddings)
    low_wl = old / low_freq_factor
    high_wl = old / high_freq_factor
    wavelen = 2.0 * math.pi / inv_freq
    scaled = torch.where(wavelen > low_wl, inv_freq / factor, inv_freq)
    if high_freq_factor != low_freq_factor:
        smooth = (old / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
        blended = (1.0 - smooth) * scaled / factor + smooth * scaled
        medium = ~(wavelen < high_wl) & ~(wavelen > low_wl)
        scaled = torch.where(medium, blended, scaled)
    return scaled


@register_position("rope_interleaved")
class RopeInterleaved(PositionEncoding):
    def inv_freq(self) -> Optional[torch.Tensor]:
        dh = self.head_dim
        fraction = torch.arange(0, dh, 2, dtype=torch.float32) / dh
        inv = 1.0 / (torch.tensor(float(self.spec.theta), dtype=torch.float32) ** fraction)
        scaling = self.spec.get("scaling")
        if scaling:
            inv = llama3_scaled_frequencies(
                inv,
                float(scaling["factor"]),
                float(scaling["low_freq_factor"]),
                float(scaling["high_freq_factor"]),
                int(scaling["original_max_position_embeddings"]),
            )
        return inv.to(torch.float32)

    def rotation(self) -> Rotation:
        return Rotation(self.inv_freq(), pairing="adjacent", rotary_dim=self.head_dim)
