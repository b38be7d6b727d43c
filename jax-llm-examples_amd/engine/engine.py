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

from ..cache.manager import CacheManager, pool_sizes
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .batch import StepEntry
from .loading import get_ops, load_model
from .runner import ModelRunner
from .scheduler import Request, Scheduler, SchedulerConfig


class Engine:
    DEFAULT_KV_MEMORY_FRACTION = 0.9

    def __init__(self, model, *, cache_tokens: Optional[int] = None, kv_memory_fraction: Optional[float] = None,
                 page_size: int = 16, decode_batch_size: int = 64, max_num_batched_tokens: int = 2048,
                 max_seq_len: Optional[int] = None, keep_free_pages: int = 0, reference_ops: bool = False,
                 poison: bool = False, decode_graphs: Optional[bool] = None) -> None:
        """The page pools are sized either by ``cache_tokens`` (tokens that a layer group which keeps
        every token can hold) or by ``kv_memory_fraction`` (that part of the device memory free now,
        after the weights).  With neither: ``decode_batch_size * max_seq_len`` tokens if ``max_seq_len``
        is given, else (on a GPU) 0.9 of the free memory.  Groups whose retention rule
        lets go of old tokens (chunked attention) get only what ``decode_batch_size`` requests can
        hold of them.  ``max_seq_len``: a request ends with reason ``"length"`` when prompt and
        output reach it; default: the configuration's ``max_position_embeddings``, if it has one.
        ``decode_graphs``: replay steps of single tokens as recorded HIP graphs (default: on a GPU)."""
        self.model = model
        self.max_num_batched_tokens = max_num_batched_tokens
        self.ops = get_ops(model.device, reference_ops=reference_ops)
        limit = getattr(getattr(model, "config", None), "max_position_embeddings", None)
        asked_len = max_seq_len
        if max_seq_len is None:
            max_seq_len = limit
        elif limit is not None and max_seq_len > limit:
            raise ValueError(f"max_seq_len {max_seq_len} is beyond the model's max_position_embeddings {limit}")
        self.max_seq_len = max_seq_len
        needs = model.cache_needs()
        item = torch.empty((), dtype=model.dtype).element_size()
        memory = None
        if kv_memory_fraction is not None:
            if cache_tokens is not None:
                raise ValueError("give cache_tokens or kv_memory_fraction, not both")
            if not 0.0 < kv_memory_fraction <= 1.0 or model.device.type != "cuda":
                raise ValueError("kv_memory_fraction must lie in (0, 1] and needs a GPU")
            free, _ = torch.cuda.mem_get_info(model.device)
            memory = int(free * kv_memory_fraction)
        elif cache_tokens is None:
            if asked_len is not None:
                cache_tokens = decode_batch_size * asked_len
            elif model.device.type == "cuda":
                # (the configuration's own limit may be millions of positions: take what the device has)
                free, _ = torch.cuda.mem_get_info(model.device)
                memory = int(free * self.DEFAULT_KV_MEMORY_FRACTION)
            else:
                raise ValueError("give cache_tokens, kv_memory_fraction or max_seq_len")
        num_pages = pool_sizes(needs, page_size=page_size, itemsize=item, max_requests=decode_batch_size,
                               max_step_tokens=max_num_batched_tokens, max_seq_len=max_seq_len,
                               cache_tokens=cache_tokens, memory_bytes=memory)
        self.cache = CacheManager(needs, page_size=page_size, num_pages=num_pages,
                                  max_requests=decode_batch_size, dtype=model.dtype, device=model.device,
                                  poison=poison)
        self.runner = ModelRunner(model, self.cache, self.ops, decode_graphs=decode_graphs)
        self.scheduler = Scheduler(SchedulerConfig(max_num_batched_tokens, decode_batch_size, keep_free_pages,
                                                   max_seq_len), self.cache)
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
        """Whole prompts.  Returns ``(next_tokens, logits, ids)``: the greedy next token of every prompt, the
        float32 logits at each prompt's last token, and the handles to pass to :meth:`decode_step`
        (``model.py:1243-1267``).  Prompts that together fit the step's token budget
        (``max_num_batched_tokens``) are one step; longer ones are run in portions of at most that many
        tokens, which is what the page pools of layers that let go of old tokens are sized for."""
        ids = list(ids) if ids is not None else [f"req{next(self._ids)}" for _ in tokens]
        prompts = [list(t) for t in tokens]
        if any(len(t) < 1 for t in prompts):
            raise ValueError("a prompt needs at least one token")
        done = [0] * len(prompts)
        rows: dict = {}
        while any(d < len(t) for d, t in zip(done, prompts)):
            left, entries, closing = self.max_num_batched_tokens, [], []
            for j, t in enumerate(prompts):
                n = min(len(t) - done[j], left)
                if n < 1:
                    continue
                last = done[j] + n == len(t)
                entries.append(StepEntry(ids[j], t[done[j]: done[j] + n], [n - 1] if last else []))
                if last:
                    closing.append(j)
                done[j] += n
                left -= n
            logits = self.runner.step(entries)
            # (a step of single tokens hands out a buffer that the next such step writes again: what is kept
            # and handed on is a copy)
            for r, j in enumerate(closing):
                rows[j] = logits[r].clone()
        logits = torch.stack([rows[j] for j in range(len(prompts))])
        return self._greedy(logits), logits, ids

    def decode_step(self, last_tokens: Sequence[int], ids: Sequence):
        """One token for each live request (``model.py:1270-1277``); returns ``(next_tokens, logits)``."""
        logits = self.runner.step([StepEntry(i, [int(t)], [0]) for i, t in zip(ids, last_tokens)])
        return self._greedy(logits), logits.clone()  # (the step's own buffer may be written again by the next step)

    def _greedy(self, logits) -> list:
        """The largest logit of each row, lowest id among equals (the sampling kernel's greedy case)."""
        m = logits.shape[0]
        return self.sampler(logits, [SamplingParams()] * m, [0] * m)

    def release(self, ids: Sequence) -> None:
        for i in ids:
            self.runner.finish(i)
