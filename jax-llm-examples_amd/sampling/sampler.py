"""Chooses next tokens from float32 logits on the device, one kernel call per step."""
from __future__ import annotations

from typing import Sequence

import torch

from .params import SamplingParams


class Sampler:
    def __init__(self, ops, device) -> None:
        self.ops = ops
        self.device = torch.device(device)

    def __call__(self, logits: torch.Tensor, params: Sequence[SamplingParams], counters: Sequence[int]) -> list[int]:
        """``counters[i]``: how many tokens request ``i`` has generated so far (it numbers
        the random draw, so a request's draws do not depend on the batch)."""
        m = logits.shape[0]
        assert m == len(params) == len(counters)
        temp = torch.tensor([0.0 if p.greedy else float(p.sample_temp) for p in params], dtype=torch.float32)
        topk = torch.tensor([int(p.sample_topk) for p in params], dtype=torch.int32)
        seeds = torch.tensor([int(p.seed) & 0x7FFFFFFF for p in params], dtype=torch.int32)
        ctr = torch.tensor([int(c) & 0x7FFFFFFF for c in counters], dtype=torch.int32)
        dev = self.device
        packed = torch.stack([topk, seeds, ctr]).to(dev)  # one copy for the three integer rows
        any_top_k = any(not p.greedy and 0 < p.sample_topk for p in params)
        out = self.ops.sample(logits, temp.to(dev), packed[0], packed[1], packed[2], any_top_k=any_top_k)
        return [int(t) for t in out.cpu().tolist()]
