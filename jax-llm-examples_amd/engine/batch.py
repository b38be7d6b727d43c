"""One step's batch: segments of different requests laid end to end.

``StepEntry`` is what a caller hands in: a request, its next tokens (a portion
of its prompt, cut anywhere, or one decoded token) and the places among them
whose logits are wanted.  ``StepContext`` is what the model's parts see: flat
per-token arrays on the device, per-segment arrays, per cache group the block
tables and the slot of every token, plus host copies of the sizes that pick
kernels.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Optional, Sequence

import numpy as np
import torch


DECODE_BUCKET = 1024


def decode_bucket(max_context_len: int) -> int:
    return -(-max_context_len // DECODE_BUCKET) * DECODE_BUCKET


@dataclasses.dataclass
class StepEntry:
    rid: Any
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclasses.dataclass
class GroupContext:
    block_table: torch.Tensor  # int32 [R, width]
    slot_mapping: torch.Tensor  # int32 [N]
    width: int
    retention: tuple
    seg_lens: list = dataclasses.field(default_factory=list)  # host copies, for kernel work lists
    seg_starts: list = dataclasses.field(default_factory=list)
    meta: dict = dataclasses.field(default_factory=dict)  # kernel launch plans, filled lazily
    # In a step of single tokens only: the context length the kernels' work is laid out for, a multiple of
    # DECODE_BUCKET that no request of the step exceeds.  Grids and key ranges then depend on the number of
    # requests and this bound alone, so a recorded graph of the step fits every step with the same two numbers.
    decode_bucket: Optional[int] = None


@dataclasses.dataclass
class StepContext:
    ops: Any
    dtype: torch.dtype
    device: torch.device
    num_tokens: int
    num_segments: int
    token_ids: torch.Tensor  # int32 [N]
    positions: torch.Tensor  # int32 [N]
    token_segment: torch.Tensor  # int32 [N]
    cu_seqlens: torch.Tensor  # int32 [R + 1]
    context_lens: torch.Tensor  # int32 [R]: tokens of the request after this step
    state_slots: torch.Tensor  # int32 [R]
    logits_indices: torch.Tensor  # int32 [M]
    groups: list[GroupContext]
    # host copies
    seg_lens: list[int]
    seg_starts: list[int]  # position of each segment's first token
    max_seg_len: int
    max_context_len: int
    page_size: int
    # ``tap(part, name, value)``: installed by whoever wants to watch a step (tests, benchmarks).  A part may
    # hand it named intermediate values; if the tap returns something, the part goes on with that instead.
    tap: Optional[Any] = None
    scratch: dict = dataclasses.field(default_factory=dict)


class StepLayout:
    """Where each of a step's arrays lies in ONE flat int32 buffer: per token (ids, positions, segment),
    per segment (bounds, context lengths, state slots), the wanted rows, and per cache group a block table
    ``[segments, width]`` and the slot of every token.  The step function builds such a buffer afresh for
    every step; a recorded step keeps one on the device for good.  Both fill it with :func:`fill_step`
    and make their :class:`StepContext` with :func:`context_over`, so a new per-step array is added in
    these three places and nowhere else."""

    def __init__(self, num_tokens: int, num_segments: int, num_wanted: int, widths: Sequence[int]) -> None:
        N, R = num_tokens, num_segments
        self.num_tokens, self.num_segments, self.num_wanted, self.widths = N, R, num_wanted, list(widths)
        fields = [("token_ids", N), ("positions", N), ("token_segment", N), ("cu_seqlens", R + 1),
                  ("context_lens", R), ("state_slots", R), ("logits_indices", num_wanted)]
        for g, w in enumerate(self.widths):
            fields += [(f"block_table{g}", R * w), (f"slot_mapping{g}", N)]
        self.bounds, o = {}, 0
        for name, n in fields:
            self.bounds[name] = (o, o + n)
            o += n
        self.size = o

    def view(self, flat, name: str):
        lo, hi = self.bounds[name]
        return flat[lo:hi]


def table_widths(cache, entries: Sequence[StepEntry]) -> list:
    """The block tables' widths that this step needs: the longest table of each group."""
    return [max(len(cache.table(e.rid, g.index)) for e in entries) for g in cache.groups]


def fill_step(layout: StepLayout, flat: np.ndarray, cache, entries: Sequence[StepEntry], vocab_size: int,
              stamps: Optional[list] = None):
    """Writes the step's numbers into ``flat`` (int32, ``layout.size`` long).  Every entry's request must
    hold a reservation for ``len(tokens)`` tokens in ``cache``.  ``stamps``: a list with one place per
    segment that the caller keeps between steps over the same buffer; a block-table row is then written
    only if the request in that row, this life of it, or its tables changed since the row was written
    (:meth:`~..cache.manager.CacheManager.table_stamp`).  Returns ``(seg_lens, seg_starts)``."""
    ps = cache.page_size
    v = lambda name: layout.view(flat, name)
    tok, pos, seg, cu = v("token_ids"), v("positions"), v("token_segment"), v("cu_seqlens")
    ctx_lens, slots, want = v("context_lens"), v("state_slots"), v("logits_indices")
    tables = [v(f"block_table{g.index}") for g in cache.groups]
    maps = [v(f"slot_mapping{g.index}") for g in cache.groups]
    seg_lens, seg_starts = [], []
    o = w = 0
    cu[0] = 0
    for i, e in enumerate(entries):
        n = len(e.tokens)
        if n < 1:
            raise ValueError("every entry of a step needs at least one token")
        start = cache.num_tokens(e.rid)
        if n == 1:
            t = int(e.tokens[0])
            if not 0 <= t < vocab_size:
                raise ValueError(f"request {e.rid!r}: token id outside 0..{vocab_size - 1}")
            tok[o], pos[o], seg[o] = t, start, i
        else:
            t = np.asarray(e.tokens, dtype=np.int64)
            if t.min() < 0 or t.max() >= vocab_size:
                raise ValueError(f"request {e.rid!r}: token id outside 0..{vocab_size - 1}")
            tok[o: o + n] = t
            pos[o: o + n] = np.arange(start, start + n)
            seg[o: o + n] = i
        for x in e.want:
            if not 0 <= x < n:
                raise ValueError(f"request {e.rid!r}: wanted place {x} outside its {n} tokens")
            if w < layout.num_wanted:
                want[w] = o + x
            w += 1
        cu[i + 1] = o + n
        ctx_lens[i], slots[i] = start + n, cache.slot(e.rid)
        stamp = cache.table_stamp(e.rid) if stamps is not None else None
        fresh = stamps is None or stamps[i] != stamp
        for g, width, bt, sm in zip(cache.groups, layout.widths, tables, maps):
            table = cache.table(e.rid, g.index)
            if len(table) > width:
                raise AssertionError(f"request {e.rid!r}: {len(table)} pages in a block table of {width}")
            if fresh:
                row = bt[i * width: (i + 1) * width]
                row[: len(table)] = table
                row[len(table):] = -1
            if n == 1:
                page = table[start // ps] if start // ps < len(table) else -1
                if page < 0:
                    raise AssertionError(f"request {e.rid!r}: a new token has no page in group {g.index}")
                sm[o] = page * ps + start % ps
            else:
                p = pos[o: o + n]
                pages = np.asarray(table, np.int64)[p // ps] if (start + n - 1) // ps < len(table) else np.array([-1])
                if (pages < 0).any():
                    raise AssertionError(f"request {e.rid!r}: a new token has no page in group {g.index}")
                sm[o: o + n] = pages * ps + p % ps
        if stamps is not None:
            stamps[i] = stamp
        seg_lens.append(n)
        seg_starts.append(start)
        o += n
    if o != layout.num_tokens or len(entries) != layout.num_segments:
        raise AssertionError("the entries do not fit the layout they are written into")
    return seg_lens, seg_starts


def context_over(layout: StepLayout, flat: torch.Tensor, cache, ops, dtype, device, *, seg_lens, seg_starts,
                 max_context_len: int, bucket: Optional[int], tap=None) -> StepContext:
    """The :class:`StepContext` whose arrays are views of ``flat`` (on the device the model runs on).
    ``bucket``: see :class:`GroupContext`."""
    R = layout.num_segments
    d = lambda name: layout.view(flat, name)
    groups = []
    for g, width in zip(cache.groups, layout.widths):
        groups.append(GroupContext(block_table=d(f"block_table{g.index}").view(R, width),
                                   slot_mapping=d(f"slot_mapping{g.index}"), width=width, retention=g.retention,
                                   seg_lens=seg_lens, seg_starts=seg_starts, decode_bucket=bucket))
    return StepContext(
        ops=ops, dtype=dtype, device=torch.device(device), num_tokens=layout.num_tokens, num_segments=R,
        token_ids=d("token_ids"), positions=d("positions"), token_segment=d("token_segment"),
        cu_seqlens=d("cu_seqlens"), context_lens=d("context_lens"), state_slots=d("state_slots"),
        logits_indices=d("logits_indices"), groups=groups, seg_lens=seg_lens, seg_starts=seg_starts,
        max_seg_len=max(seg_lens), max_context_len=max_context_len, page_size=cache.page_size, tap=tap)


def build_context(ops, dtype, device, cache, entries: Sequence[StepEntry], vocab_size: int,
                  tap=None) -> StepContext:
    """Lays the entries end to end, in one buffer sent to the device in one copy.  Every entry's request
    must hold a reservation for ``len(tokens)`` tokens in ``cache``."""
    if len(entries) == 0:
        raise ValueError("a step needs at least one entry and every entry at least one token")
    layout = StepLayout(sum(len(e.tokens) for e in entries), len(entries), sum(len(e.want) for e in entries),
                        table_widths(cache, entries))
    flat = np.empty(layout.size, np.int32)
    seg_lens, seg_starts = fill_step(layout, flat, cache, entries, vocab_size)
    host = torch.from_numpy(flat)
    dev = host.to(device, non_blocking=False) if torch.device(device).type != "cpu" else host
    longest = max(s + n for s, n in zip(seg_starts, seg_lens))
    return context_over(layout, dev, cache, ops, dtype, device, seg_lens=seg_lens, seg_starts=seg_starts,
                        max_context_len=longest, bucket=decode_bucket(longest) if max(seg_lens) == 1 else None,
                        tap=tap)
