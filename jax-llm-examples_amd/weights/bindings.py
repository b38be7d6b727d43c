"""How checkpoint tensors land in model parameters."""
from __future__ import annotations

import dataclasses
from typing import Optional


@dataclasses.dataclass(frozen=True)
class TensorBinding:
    """One checkpoint tensor.

    ``name``: its name in the checkpoint (without optional prefixes).
    ``shape``: its shape as stored.  ``target``: the model parameter it fills
    (a key of ``DecoderModel.named_parameters()``).  ``transpose``: two axes of
    the stored tensor to swap first.  ``rows``: the range of the target's first
    axis it fills (the whole target if ``None``) - several tensors can fill one
    fused parameter.  ``init``: how seeded random weights draw it.
    """

    name: str
    shape: tuple[int, ...]
    target: str
    transpose: Optional[tuple[int, int]] = None
    rows: Optional[tuple[int, int]] = None
    init: tuple = ("normal", 0.02)
    float32: bool = False  # stored in 32-bit by the random-weights writer whatever the run dtype
