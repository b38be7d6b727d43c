"""Per-request sampling options.

The reference's Llama 4 path is greedy only (``jnp.argmax``,
``llama4/llama4_jax/model.py:1266, 1275``); other packages of the repository
sample with a temperature among the ``k`` most likely tokens
(``sample_top(key, logits, k=16, temp=1.0)``, ``gemma4/gemma4_jax/model.py:1485-1506``,
``gpt_oss/gpt_oss_jax/model.py:1125-1148``: greedy when ``temp <= 1e-3``).  The names
``sample_temp`` and ``sample_topk`` are theirs.
"""
from __future__ import annotations

import dataclasses


@dataclasses.dataclass(frozen=True)
class SamplingParams:
    sample_temp: float = 0.0  # 0 (or <= 1e-3): greedy, lowest id among equal logits
    sample_topk: int = 0  # with a temperature: sample among this many most likely tokens (0 = all)
    seed: int = 0  # same seed + same logits -> same token, whatever else is in the batch
    max_decode_length: int = 64  # tokens to generate at most (the reference's ServingConfig name)
    eos_tokens: tuple = ()  # generation ends after one of these
    ignore_eos: bool = False

    @property
    def greedy(self) -> bool:
        return self.sample_temp <= 1e-3
