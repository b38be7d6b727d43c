"""The decode fast path: steps that hold one token of every request are recorded once as a
HIP graph and replayed.

The reference runs its decode steps as one compiled program (``llama4/llama4_jax/model.py:1270-1277``;
its serving loop scans several decode steps inside one jit, ``serving/serving_jax/serving_loop.py:511-522``).
Here a step of single tokens is a few hundred kernel launches whose sizes depend on two numbers
only: how many requests there are, and the bound on their context lengths that the kernels' work
is laid out for (:func:`~.batch.decode_bucket`).  For each such pair the launches are recorded once;
everything that changes from step to step (token ids, positions, block tables, slots) lies in one
persistent device buffer that is refreshed by a single copy before the replay.  Nothing is
allocated and nothing is cleared with a memset inside a recording.

A recording is made only of models whose parts all say ``graph_safe``; a step that is watched
(``tap``) runs launch by launch.  Recorded and unrecorded steps launch the same kernels with the
same arguments, so their logits are equal bit for bit.
"""
from __future__ import annotations

import collections
from typing import Sequence

import numpy as np
import torch

from .batch import StepEntry, StepLayout, context_over, decode_bucket, fill_step


class _Recording:
    """One (number of requests, context bound) pair: its buffers, its context, its graph."""

    def __init__(self, model, cache, ops, num_requests: int, bucket: int) -> None:
        R = num_requests
        self.R, self.bucket = R, bucket
        width = -(-bucket // cache.page_size)
        self.layout = StepLayout(R, R, R, [width] * len(cache.groups))
        total = self.layout.size
        self.mirror = np.zeros(total, np.int32)  # what the device buffer shall hold, kept from step to step
        for g in cache.groups:
            self.layout.view(self.mirror, f"block_table{g.index}")[:] = -1
        self.stamps = [None] * R  # per row: the stamp of the block tables it holds (see fill_step)
        # two pinned staging buffers: the copy of one step may still be on its way when the next is laid out
        self.staging = [torch.empty(total, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self.staged = [None, None]  # the event after each buffer's last copy
        self.turn = 0
        self.device_buf = torch.zeros(total, dtype=torch.int32, device=model.device)
        self.ctx = context_over(self.layout, self.device_buf, cache, ops, model.dtype, model.device,
                                seg_lens=[1] * R, seg_starts=None, max_context_len=bucket, bucket=bucket)
        self.graph = None
        self.logits = None

    def lay_out(self, cache, entries: Sequence[StepEntry], vocab_size: int) -> None:
        """This step's numbers into the mirror (every row's logits are computed; the caller picks the wanted
        ones), then one copy to the device."""
        fill_step(self.layout, self.mirror, cache, [StepEntry(e.rid, e.tokens, (0,)) for e in entries], vocab_size,
                  stamps=self.stamps)
        b = self.turn
        self.turn ^= 1
        if self.staged[b] is not None:
            self.staged[b].synchronize()
        self.staging[b].numpy()[:] = self.mirror
        self.device_buf.copy_(self.staging[b], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self.staged[b] = ev


class DecodeGraphs:
    MAX_RECORDINGS = 16
    RECORD_AFTER = 2  # a (requests, bound) pair is recorded when it comes the second time: one that comes once is not worth it

    def __init__(self, model, cache, ops) -> None:
        self.model, self.cache, self.ops = model, cache, ops
        self.recordings: "collections.OrderedDict[tuple, _Recording]" = collections.OrderedDict()
        self.pool = None
        self.seen: "collections.Counter[tuple]" = collections.Counter()
        self.replays = 0
        self.captures = 0
        self.safe = (getattr(ops, "name", "") == "hip" and model.device.type == "cuda"
                     and all(getattr(p, "graph_safe", False) for b in model.blocks for p in b.parts().values())
                     and all(getattr(p, "graph_safe", False) for p in (model.final_norm, model.embed, model.lm_head)))

    def fits(self, entries: Sequence[StepEntry], tap) -> bool:
        return self.safe and tap is None and all(len(e.tokens) == 1 for e in entries)

    @torch.no_grad()
    def run(self, entries: Sequence[StepEntry]):
        """The entries hold reservations for their one token.  Returns float32 logits of the wanted rows; they
        lie in the recording's own output buffer until the next step of the same shape.  ``None``: this step is
        better run launch by launch (its shape has not come often enough to be recorded)."""
        cache, model = self.cache, self.model
        longest = max(cache.requests[e.rid].num_tokens for e in entries) + 1
        key = (len(entries), decode_bucket(longest))
        rec = self.recordings.get(key)
        if rec is None:
            self.seen[key] += 1
            if self.seen[key] < self.RECORD_AFTER:
                if len(self.seen) > 4096:
                    self.seen.clear()
                return None
            rec = _Recording(model, cache, self.ops, *key)
            self.recordings[key] = rec
            while len(self.recordings) > self.MAX_RECORDINGS:
                self.recordings.popitem(last=False)
        else:
            self.recordings.move_to_end(key)
        rec.lay_out(cache, entries, model.plan.vocab_size)
        if rec.graph is None:
            # once launch by launch (kernel plans are made, work lists uploaded, libraries warm), then recorded:
            # a recording runs nothing, and what the step writes (keys, values) it writes again with the same
            # values when the recording is replayed below
            model.forward(rec.ctx, cache)
            torch.cuda.current_stream().synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, pool=self.pool):
                rec.logits = model.forward(rec.ctx, cache)
            if self.pool is None:
                self.pool = graph.pool()
            rec.graph = graph
            self.captures += 1
        rec.graph.replay()
        self.replays += 1
        wanted = [i for i, e in enumerate(entries) for _ in e.want]
        if wanted == list(range(len(entries))):
            return rec.logits
        if not wanted:
            return rec.logits[:0]
        return rec.logits[torch.tensor(wanted, device=rec.logits.device)]
