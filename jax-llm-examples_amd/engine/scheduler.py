"""Continuous batching on one GPU: admits requests, cuts prompts into portions
under a token budget, decodes, finishes and frees.

The reference's serving loop (``serving/serving_jax/serving_loop.py``) keeps a fixed
number of decode slots (``decode_batch_size``, ``:422-434``), prefills whole prompts
in their own batches (``:697-758``), lets decode go first (``:794-795``), finishes a
request on an EOS token or after ``max_decode_length`` tokens (``:656-660``; here also when
prompt and output reach ``max_seq_len``, the configuration's context limit), and has
no answer to a full cache.  Here one step holds decode tokens of running
requests beside portions of prompts; the option names ``decode_batch_size``,
``max_decode_length`` and ``eos_tokens`` keep the reference's meaning.

When pages run out: the request admitted last is *preempted* - everything it
holds goes back, and it returns to the head of the waiting queue to be computed
again from its prompt plus the tokens it has generated (which are kept).  If
the only running request cannot get its pages, it ends with reason
``"out_of_pages"``.

The scheduler only decides; it owns no tensors.  It asks the cache manager how
many pages a plan would take and frees what preempted and finished requests hold.
"""
from __future__ import annotations

import collections
import dataclasses
from typing import Any, Optional, Sequence

from ..sampling.params import SamplingParams
from .batch import StepEntry

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"


@dataclasses.dataclass
class SchedulerConfig:
    max_num_batched_tokens: int = 2048  # tokens one step may hold
    decode_batch_size: int = 64  # requests that may be running at once
    keep_free_pages: int = 0  # pages per group that admitting a new request must leave free
    max_seq_len: Optional[int] = None  # a request ends when its prompt and output together reach this many tokens


@dataclasses.dataclass
class Request:
    id: Any
    prompt: list
    params: SamplingParams = dataclasses.field(default_factory=SamplingParams)
    output: list = dataclasses.field(default_factory=list)
    num_computed: int = 0  # tokens whose keys and values are in the cache
    state: str = WAITING
    finish_reason: Optional[str] = None
    preemptions: int = 0

    @property
    def tokens(self) -> list:
        return self.prompt + self.output

    @property
    def num_pending(self) -> int:
        return len(self.prompt) + len(self.output) - self.num_computed


@dataclasses.dataclass
class ScheduledSegment:
    request: Request
    start: int
    count: int
    samples: bool  # the segment ends at the request's last known token: its logits give the next one


@dataclasses.dataclass
class StepPlan:
    segments: list
    preempted: list
    dropped: list  # requests ended because they can never fit

    @property
    def num_tokens(self) -> int:
        return sum(s.count for s in self.segments)

    def entries(self) -> list:
        out = []
        for s in self.segments:
            toks = s.request.tokens[s.start: s.start + s.count]
            out.append(StepEntry(s.request.id, toks, [s.count - 1] if s.samples else []))
        return out


class Scheduler:
    def __init__(self, cfg: SchedulerConfig, cache) -> None:
        if cfg.max_num_batched_tokens < 1 or cfg.decode_batch_size < 1:
            raise ValueError("max_num_batched_tokens and decode_batch_size must be positive")
        self.cfg = cfg
        self.cache = cache
        self.waiting: collections.deque = collections.deque()
        self.running: list = []  # in order of admission
        self.stats = collections.Counter()

    # ------------------------------------------------------------------ queue
    def add(self, request: Request) -> None:
        if not request.prompt:
            raise ValueError(f"request {request.id!r} has an empty prompt")
        limit = self.cfg.max_seq_len
        if limit is not None and len(request.prompt) > limit:
            # the reference asserts the same of a prompt (llama4/llama4_jax/model.py:1248)
            raise ValueError(f"request {request.id!r}: a prompt of {len(request.prompt)} tokens is longer than "
                             f"max_seq_len {limit}")
        request.state = WAITING
        self.waiting.append(request)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ------------------------------------------------------------------ planning
    def _needed(self, r: Request, n: int) -> list:
        if self.cache.has_request(r.id):
            return self.cache.pages_needed(r.id, n)
        return self.cache.pages_needed_new(n)

    def _preempt(self, r: Request) -> None:
        if self.cache.has_request(r.id):
            self.cache.free(r.id)
        self.running.remove(r)
        r.num_computed = 0
        r.state = WAITING
        r.preemptions += 1
        self.waiting.appendleft(r)
        self.stats["preemptions"] += 1

    def _finish(self, r: Request, reason: str) -> None:
        if self.cache.has_request(r.id):
            self.cache.free(r.id)
        if r in self.running:
            self.running.remove(r)
        r.state = FINISHED
        r.finish_reason = reason

    def schedule(self) -> StepPlan:
        cfg = self.cfg
        budget = cfg.max_num_batched_tokens
        free = list(self.cache.num_free_pages())
        segments, preempted, dropped = [], [], []
        planned: set = set()

        def take(r: Request, n: int, keep: int) -> bool:
            need = self._needed(r, n)
            if any(x + keep > f for x, f in zip(need, free)):
                return False
            for g, x in enumerate(need):
                free[g] -= x
            segments.append(ScheduledSegment(r, r.num_computed, n, r.num_computed + n == len(r.prompt) + len(r.output)))
            planned.add(id(r))
            return True

        def recount() -> None:
            """Free pages after a request gave back what it held, less what this step's segments will take."""
            free[:] = self.cache.num_free_pages()
            for s in segments:
                for g, x in enumerate(self._needed(s.request, s.count)):
                    free[g] -= x

        # 1. running requests, decoding ones first, each in order of admission
        order = [r for r in self.running if r.num_pending == 1] + [r for r in self.running if r.num_pending != 1]
        for r in order:
            if r.state != RUNNING or budget <= 0:
                continue
            n = min(r.num_pending, budget)
            while not take(r, n, 0):
                # the request admitted last gives way (possibly r itself)
                victim = next((v for v in reversed(self.running) if id(v) not in planned), None)
                if victim is None or (victim is r and len(self.running) == 1):
                    if victim is r:
                        self._finish(r, "out_of_pages")
                        dropped.append(r)
                        recount()
                    break
                self._preempt(victim)
                preempted.append(victim)
                recount()
                if victim is r:
                    break
            if id(r) in planned:
                budget -= n
        # 2. waiting requests, first come first served, none overtakes
        while self.waiting and budget > 0 and len(self.running) < cfg.decode_batch_size:
            r = self.waiting[0]
            if r in preempted and self.running:
                break  # it has just been preempted: let the others go on first
            if self.cache.slots.num_free < 1 and not self.cache.has_request(r.id):
                break
            n = min(r.num_pending, budget)
            if not take(r, n, cfg.keep_free_pages if self.running else 0):
                if not self.running and not segments:
                    # nothing else holds pages and it still does not fit
                    self.waiting.popleft()
                    self._finish(r, "out_of_pages")
                    dropped.append(r)
                    continue
                break
            self.waiting.popleft()
            r.state = RUNNING
            self.running.append(r)
            budget -= n
        self.stats["steps"] += 1
        self.stats["tokens"] += sum(s.count for s in segments)
        return StepPlan(segments, preempted, dropped)

    # ------------------------------------------------------------------ after the step
    def update(self, plan: StepPlan, sampled: Sequence[int]) -> list:
        """``sampled``: one token per segment with ``samples`` set, in plan order.
        Returns the requests that finished."""
        finished = []
        it = iter(sampled)
        for s in plan.segments:
            r = s.request
            r.num_computed += s.count
            if not s.samples:
                continue
            tok = int(next(it))
            r.output.append(tok)
            p = r.params
            if not p.ignore_eos and tok in p.eos_tokens:
                self._finish(r, "eos")
            elif len(r.output) >= p.max_decode_length:
                self._finish(r, "length")
            elif self.cfg.max_seq_len is not None and len(r.prompt) + len(r.output) >= self.cfg.max_seq_len:
                self._finish(r, "length")  # the context limit: there is no position for a further token
            if r.state == FINISHED:
                finished.append(r)
        return finished
