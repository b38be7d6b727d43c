"""The cache manager: keys and values in pages with a block table per request,
a page pool per group of layers with the same needs, and slots of fixed-size
per-request state.

The reference's Llama 4 cache is a dense ring buffer per layer with one shared
cursor (``llama4/llama4_jax/model.py:595-640``); its paged cache for another
model keeps ``block_tables``, ``lengths`` and a ``free_pages`` mask
(``llama3/llama3_jax/model.py:457-560``) and gives pages back only when a slot is
overwritten.  Here pages are given back when a request ends and as soon as a
group's retention rule (chunk or window) has passed them.

Runs of the model's order with the same ``(kv heads, head size, retention)``
form a *group*: they share page ids and one block table per request, and each
has a tensor ``[num_pages, 2, kv_heads, page_size, head_dim]`` of its own.
"""
from __future__ import annotations

import dataclasses
from typing import Optional

import torch

from ..parts.base import CacheNeed, first_needed_position
from .pages import OutOfPages, OutOfSlots, PagePool, SlotPool


@dataclasses.dataclass
class CacheGroup:
    index: int
    kv_heads: int
    head_dim: int
    retention: tuple
    cache_ids: list[int]
    pool: PagePool
    tensors: dict[int, torch.Tensor]

    def bytes_per_token(self, itemsize: int) -> int:
        return len(self.cache_ids) * 2 * self.kv_heads * self.head_dim * itemsize


@dataclasses.dataclass
class RequestEntry:
    slot: int
    num_tokens: int = 0  # tokens whose keys and values are written (committed)
    reserved: int = 0  # tokens beyond num_tokens that have pages for the running step
    tables: list[list[int]] = dataclasses.field(default_factory=list)  # per group: page id or -1 per page index


@dataclasses.dataclass
class CacheView:
    """What one run of a mixer sees during a step (filled by the step function)."""

    cache_id: int
    writes: bool
    kv: Optional[torch.Tensor] = None
    block_table: Optional[torch.Tensor] = None
    slot_mapping: Optional[torch.Tensor] = None
    state: Optional[torch.Tensor] = None
    attn_meta: Optional[object] = None
    group: Optional[int] = None


class CacheManager:
    def __init__(
        self,
        needs: dict[int, CacheNeed],
        *,
        page_size: int,
        num_pages: int | dict[int, int],
        max_requests: int,
        dtype: torch.dtype,
        device: torch.device | str,
        poison: bool = False,
    ) -> None:
        if page_size < 1:
            raise ValueError("page_size must be positive")
        self.page_size = page_size
        self.max_requests = max_requests
        self.dtype = dtype
        self.device = torch.device(device)
        self.poison = poison
        self.slots = SlotPool(max_requests)
        self.groups: list[CacheGroup] = []
        self.group_of: dict[int, int] = {}
        self.state: dict[int, torch.Tensor] = {}
        self.requests: dict[object, RequestEntry] = {}
        by_key: dict[tuple, CacheGroup] = {}
        for cid in sorted(needs):
            need = needs[cid]
            if need.kv is not None:
                key = (need.kv[0], need.kv[1], tuple(need.retention))
                g = by_key.get(key)
                if g is None:
                    n = num_pages[len(self.groups)] if isinstance(num_pages, dict) else num_pages
                    g = CacheGroup(len(self.groups), need.kv[0], need.kv[1], tuple(need.retention), [], PagePool(n), {})
                    by_key[key] = g
                    self.groups.append(g)
                g.cache_ids.append(cid)
                self.group_of[cid] = g.index
            if need.state_shape is not None:
                self.state[cid] = torch.zeros(
                    (max_requests, *need.state_shape), dtype=need.state_dtype or torch.float32, device=self.device
                )
        fill = float("nan") if poison else 0.0
        for g in self.groups:
            for cid in g.cache_ids:
                g.tensors[cid] = torch.full(
                    (g.pool.num_pages, 2, g.kv_heads, page_size, g.head_dim), fill, dtype=dtype, device=self.device
                )

    # ------------------------------------------------------------------ requests
    def add_request(self, rid) -> RequestEntry:
        if rid in self.requests:
            raise KeyError(f"request {rid!r} is already live")
        slot = self.slots.alloc()
        for t in self.state.values():
            t[slot].zero_()
        e = RequestEntry(slot=slot, tables=[[] for _ in self.groups])
        self.requests[rid] = e
        return e

    def has_request(self, rid) -> bool:
        return rid in self.requests

    def _pages_missing(self, e: RequestEntry, g: CacheGroup, upto: int) -> list[int]:
        """Page indices that positions ``[num_tokens, upto)`` need and the table lacks."""
        table = e.tables[g.index]
        first = e.num_tokens // self.page_size
        last = (upto - 1) // self.page_size
        return [j for j in range(first, last + 1) if j >= len(table) or table[j] < 0]

    def pages_needed(self, rid, n_new: int) -> list[int]:
        """Pages each group would have to hand out to append ``n_new`` tokens."""
        e = self.requests[rid]
        upto = e.num_tokens + n_new
        return [len(self._pages_missing(e, g, upto)) for g in self.groups]

    def pages_needed_new(self, n_new: int) -> list[int]:
        """The same for a request that is not live yet."""
        n = -(-n_new // self.page_size)
        return [n for _ in self.groups]

    def can_reserve(self, rid, n_new: int, keep_free: int = 0) -> bool:
        need = self.pages_needed(rid, n_new) if rid in self.requests else self.pages_needed_new(n_new)
        return all(n + keep_free <= g.pool.num_free for n, g in zip(need, self.groups))

    def reserve(self, rid, n_new: int) -> None:
        """Gives the request pages for its next ``n_new`` tokens in every group, or
        raises :class:`OutOfPages` and changes nothing."""
        e = self.requests[rid]
        if e.reserved:
            raise AssertionError(f"request {rid!r} already has a reservation of {e.reserved} tokens")
        upto = e.num_tokens + n_new
        missing = [self._pages_missing(e, g, upto) for g in self.groups]
        for g, m in zip(self.groups, missing):
            if len(m) > g.pool.num_free:
                raise OutOfPages(
                    f"group {g.index} ({g.retention}): request {rid!r} needs {len(m)} pages, {g.pool.num_free} free"
                )
        for g, m in zip(self.groups, missing):
            table = e.tables[g.index]
            got = g.pool.alloc(len(m))
            for j, p in zip(m, got):
                while len(table) <= j:
                    table.append(-1)
                table[j] = p
        e.reserved = n_new

    def commit(self, rid) -> None:
        """The step that wrote the reserved tokens is done: count them and give back
        every page that no later query of this request can read."""
        e = self.requests[rid]
        e.num_tokens += e.reserved
        e.reserved = 0
        for g in self.groups:
            keep_from = first_needed_position(g.retention, e.num_tokens)
            table = e.tables[g.index]
            # page j holds positions [j*ps, (j+1)*ps): free iff (j+1)*ps <= keep_from
            gone = [j for j in range(min(len(table), keep_from // self.page_size)) if table[j] >= 0]
            if gone:
                self._release(g, [table[j] for j in gone])
                for j in gone:
                    table[j] = -1

    def cancel(self, rid) -> None:
        """Drop a reservation whose step did not run (pages beyond what the
        committed tokens use go back)."""
        e = self.requests[rid]
        e.reserved = 0
        last_used = (e.num_tokens - 1) // self.page_size if e.num_tokens else -1
        for g in self.groups:
            table = e.tables[g.index]
            extra = [j for j in range(last_used + 1, len(table)) if table[j] >= 0]
            if extra:
                self._release(g, [table[j] for j in extra])
            del table[last_used + 1 :]

    def free(self, rid) -> None:
        e = self.requests.pop(rid)
        for g in self.groups:
            pages = [p for p in e.tables[g.index] if p >= 0]
            if pages:
                self._release(g, pages)
        self.slots.release(e.slot)

    def _release(self, g: CacheGroup, pages: list[int]) -> None:
        g.pool.release(pages)
        if self.poison and pages:
            idx = torch.tensor(pages, dtype=torch.long, device=self.device)
            for t in g.tensors.values():
                t.index_fill_(0, idx, float("nan"))

    # ------------------------------------------------------------------ queries
    def num_tokens(self, rid) -> int:
        return self.requests[rid].num_tokens

    def slot(self, rid) -> int:
        return self.requests[rid].slot

    def table(self, rid, group: int) -> list[int]:
        return self.requests[rid].tables[group]

    def num_free_pages(self) -> list[int]:
        return [g.pool.num_free for g in self.groups]

    def num_live(self) -> int:
        return len(self.requests)

    def check(self) -> None:
        """Invariants: no page lost, held twice, or held by nobody."""
        for g in self.groups:
            g.pool.check()
            held = []
            for e in self.requests.values():
                held += [p for p in e.tables[g.index] if p >= 0]
            if len(set(held)) != len(held):
                raise AssertionError(f"group {g.index}: a page is in two block tables")
            if len(held) != g.pool.num_held:
                raise AssertionError(
                    f"group {g.index}: {g.pool.num_held} pages are out of the pool but block tables hold {len(held)}"
                )

    def bytes_per_token(self) -> int:
        item = torch.empty((), dtype=self.dtype).element_size()
        return sum(g.bytes_per_token(item) for g in self.groups)


__all__ = ["CacheManager", "CacheView", "CacheGroup", "OutOfPages", "OutOfSlots"]
