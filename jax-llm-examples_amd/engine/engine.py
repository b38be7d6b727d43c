"""The Python entry point: model + cache + scheduler + sampler.

The reference's programmatic use is ``prefill(tokens, weights, cache, cfg)`` then a
loop of ``decode_step`` (``llama4/main.py:68-74``); :meth:`Engine.generate` is that
loop with continuous batching, and :meth:`Engine.prefill` / :meth:`Engine.decode_step`
keep the two-call form.
"""
from __future__ import annotations

import itertools
from typing import Optional, Sequence

import torch

from ..cache.manager import CacheManager
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .batch import StepEntry
from .loading import get_ops, load_model
from .runner import ModelRunner
from .scheduler import Request, Scheduler, SchedulerConfig


class Engine:
    def __init__(self, model, *, cache_tokens: int, page_size: int = 16, decode_batch_size: int = 64,
                 max_num_batched_tokens: int = 2048, keep_free_pages: int = 0, reference_ops: bool = False,
                 poison: bool = False) -> None:
        """``cache_tokens``: tokens each layer group's page pool can hold."""
        self.model = model
        self.ops = get_ops(model.device, reference_ops=reference_ops)
        num_pages = -(-cache_tokens // page_size)
        self.cache = CacheManager(model.cache_needs(), page_size=page_size, num_pages=num_pages,
                                  max_requests=decode_batch_size, dtype=model.dtype, device=model.device,
                                  poison=poison)
        self.runner = ModelRunner(model, self.cache, self.ops)
        self.scheduler = Scheduler(SchedulerConfig(max_num_batched_tokens, decode_batch_size, keep_free_pages),
                                   self.cache)
        self.sampler = Sampler(self.ops, model.device)
        self._ids = itertools.count()

    @classmethod
    def from_folder(cls, ckpt_path: str, dtype="bfloat16", device="cuda:0", **kw) -> "Engine":
        return cls(load_model(ckpt_path, dtype, device), **kw)

    # ------------------------------------------------------------------ continuous batching
    def add_request(self, prompt: Sequence[int], params: Optional[SamplingParams] = None, rid=None) -> Request:
        r = Request(next(self._ids) if rid is None else rid, list(prompt), params or SamplingParams())
        self.scheduler.add(r)
        return r

    def step(self) -> list:
        """One scheduler step; returns the requests that finished in it."""
        plan = self.scheduler.schedule()
        done = list(plan.dropped)
        if plan.segments:
            logits = self.runner.step(plan.entries())
            samplers = [s.request for s in plan.segments if s.samples]
            tokens = self.sampler(logits, [r.params for r in samplers], [len(r.output) for r in samplers]) \
                if samplers else []
            done += self.scheduler.update(plan, tokens)
        return done

    def generate(self, prompts: Sequence[Sequence[int]], params=None) -> list:
        """Generates for every prompt (token ids in, token ids out, in prompt order)."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        reqs = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        while self.scheduler.has_work():
            self.step()
        return [r.output for r in reqs]

    # ------------------------------------------------------------------ the reference's two calls
    def prefill(self, tokens: Sequence[Sequence[int]], ids: Optional[Sequence] = None):
        """Whole prompts in one step.  Returns ``(next_tokens, logits, ids)``: the greedy
        next token of every prompt, the float32 logits at each prompt's last token, and
        the handles to pass to :meth:`decode_step` (``model.py:1243-1267``)."""
        ids = list(ids) if ids is not None else [f"req{next(self._ids)}" for _ in tokens]
        logits = self.runner.step([StepEntry(i, list(t), [len(t) - 1]) for i, t in zip(ids, tokens)])
        return torch.argmax(logits, dim=-1).tolist(), logits, ids

    def decode_step(self, last_tokens: Sequence[int], ids: Sequence):
        """One token for each live request (``model.py:1270-1277``); returns ``(next_tokens, logits)``."""
        logits = self.runner.step([StepEntry(i, [int(t)], [0]) for i, t in zip(ids, last_tokens)])
        return torch.argmax(logits, dim=-1).tolist(), logits

    def release(self, ids: Sequence) -> None:
        for i in ids:
            self.runner.finish(i)
