"""The step function: one batch of (request, its next tokens) through the model.

The reference has two separate programs over rectangular padded batches,
``prefill`` and ``decode_step`` (``llama4/llama4_jax/model.py:1243-1277``).  Here
one function runs whatever it is given - portions of prompts beside single
decoded tokens, cut anywhere - as one flat batch, from the paged cache, and
returns float32 logits at the wanted places.
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch

from ..cache.manager import CacheManager
from ..cache.pages import OutOfPages
from .batch import StepEntry, build_context


class ModelRunner:
    def __init__(self, model, cache: CacheManager, ops, decode_graphs: Optional[bool] = None) -> None:
        self.model = model
        self.cache = cache
        self.ops = ops
        # steps of single tokens as recorded graphs: on by default where the kernels run and every part allows it
        self.graphs = None
        if decode_graphs is None or decode_graphs:
            from .decode_graph import DecodeGraphs

            graphs = DecodeGraphs(model, cache, ops)
            if graphs.safe:
                self.graphs = graphs
            elif decode_graphs:
                raise ValueError("decode graphs were asked for, but the kernels do not run here or a part of the "
                                 "model does not say graph_safe")
        self.steps_run = 0
        self.tokens_run = 0

    @torch.no_grad()
    def step(self, entries: Sequence[StepEntry], *, tap=None) -> torch.Tensor:
        """Runs only the tokens it is given.  A request not yet known to the
        cache is added.  Pages for the new tokens are taken first (for all
        entries or for none: :class:`OutOfPages` leaves the cache unchanged);
        after the model has run, the tokens are counted and pages that a
        retention rule has passed are given back.  Returns ``[wanted, vocab]``
        float32, in the order of the entries and of each entry's ``want``.  ``tap``: see
        :class:`~.batch.StepContext`.  A step of single tokens may be the replay of a recorded
        graph (:mod:`.decode_graph`); its logits then lie in that recording's buffer, which the next
        step of the same shape writes again."""
        cache = self.cache
        seen = set()
        for e in entries:
            if e.rid in seen:
                raise ValueError(f"request {e.rid!r} appears twice in one step")
            seen.add(e.rid)
        added, reserved = [], []
        try:
            for e in entries:
                if not cache.has_request(e.rid):
                    cache.add_request(e.rid)
                    added.append(e.rid)
                cache.reserve(e.rid, len(e.tokens))
                reserved.append(e.rid)
        except Exception:
            for rid in reserved:
                cache.cancel(rid)
            for rid in added:
                cache.free(rid)
            raise
        try:
            logits = None
            if self.graphs is not None and self.graphs.fits(entries, tap):
                logits = self.graphs.run(entries)
                num_tokens = len(entries)
            if logits is None:
                ctx = build_context(self.ops, self.model.dtype, self.model.device, cache, entries,
                                    self.model.plan.vocab_size, tap)
                logits = self.model.forward(ctx, cache)
                num_tokens = ctx.num_tokens
        except Exception:
            for rid in reserved:
                cache.cancel(rid)
            for rid in added:
                cache.free(rid)
            raise
        for e in entries:
            cache.commit(e.rid)
        self.steps_run += 1
        self.tokens_run += num_tokens
        return logits

    def finish(self, rid) -> None:
        """The request is over: its pages and its state slot go back."""
        self.cache.free(rid)


__all__ = ["ModelRunner", "StepEntry", "OutOfPages"]
