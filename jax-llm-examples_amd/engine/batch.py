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


def build_context(ops, dtype, device, cache, entries: Sequence[StepEntry], vocab_size: int,
                  tap=None) -> StepContext:
    """Lays the entries end to end.  Every entry's request must hold a
    reservation for ``len(tokens)`` tokens in ``cache``."""
    ps = cache.page_size
    R = len(entries)
    seg_lens = [len(e.tokens) for e in entries]
    if R == 0 or min(seg_lens) < 1:
        raise ValueError("a step needs at least one entry and every entry at least one token")
    N = sum(seg_lens)
    seg_starts = [cache.num_tokens(e.rid) for e in entries]
    tok = np.empty(N, np.int32)
    pos = np.empty(N, np.int32)
    seg = np.empty(N, np.int32)
    cu = np.zeros(R + 1, np.int32)
    want = []
    o = 0
    for i, e in enumerate(entries):
        n = seg_lens[i]
        t = np.asarray(e.tokens, dtype=np.int64)
        if t.min() < 0 or t.max() >= vocab_size:
            raise ValueError(f"request {e.rid!r}: token id outside 0..{vocab_size - 1}")
        tok[o : o + n] = t
        pos[o : o + n] = np.arange(seg_starts[i], seg_starts[i] + n)
        seg[o : o + n] = i
        for w in e.want:
            if not 0 <= w < n:
                raise ValueError(f"request {e.rid!r}: wanted place {w} outside its {n} tokens")
            want.append(o + w)
        o += n
        cu[i + 1] = o
    ctx_lens = np.asarray([s + n for s, n in zip(seg_starts, seg_lens)], np.int32)
    slots = np.asarray([cache.slot(e.rid) for e in entries], np.int32)

    pieces = [tok, pos, seg, cu, ctx_lens, slots, np.asarray(want, np.int32)]
    group_shapes = []
    for g in cache.groups:
        width = max(len(cache.table(e.rid, g.index)) for e in entries)
        bt = np.full((R, width), -1, np.int32)
        sm = np.empty(N, np.int32)
        o = 0
        for i, e in enumerate(entries):
            table = cache.table(e.rid, g.index)
            bt[i, : len(table)] = table
            p = pos[o : o + seg_lens[i]]
            pages = bt[i, p // ps]
            if (pages < 0).any():
                raise AssertionError(f"request {e.rid!r}: a new token has no page in group {g.index}")
            sm[o : o + seg_lens[i]] = pages * ps + p % ps
            o += seg_lens[i]
        pieces += [bt.reshape(-1), sm]
        group_shapes.append(width)

    flat = np.concatenate(pieces)
    host = torch.from_numpy(flat)
    dev = host.to(device, non_blocking=False) if torch.device(device).type != "cpu" else host
    views = []
    o = 0
    for p in pieces:
        views.append(dev[o : o + p.size])
        o += p.size
    token_ids, positions, token_segment, cu_seqlens, context_lens, state_slots, logits_indices = views[:7]
    groups = []
    for gi, g in enumerate(cache.groups):
        bt = views[7 + 2 * gi].view(R, group_shapes[gi])
        sm = views[8 + 2 * gi]
        groups.append(GroupContext(block_table=bt, slot_mapping=sm, width=group_shapes[gi], retention=g.retention,
                                   seg_lens=seg_lens, seg_starts=seg_starts,
                                   decode_bucket=decode_bucket(int(ctx_lens.max())) if max(seg_lens) == 1 else None))
    return StepContext(
        ops=ops, dtype=dtype, device=torch.device(device), num_tokens=N, num_segments=R,
        token_ids=token_ids, positions=positions, token_segment=token_segment, cu_seqlens=cu_seqlens,
        context_lens=context_lens, state_slots=state_slots, logits_indices=logits_indices, groups=groups,
        seg_lens=seg_lens, seg_starts=seg_starts, max_seg_len=max(seg_lens),
        max_context_len=int(ctx_lens.max()), page_size=ps,
        tap=tap,
    )
