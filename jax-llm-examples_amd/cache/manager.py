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
(and the same further per-token tensors, if any) form a *group*: they share page
ids and one block table per request, and each has a tensor ``[num_pages, 2,
kv_heads, page_size, head_dim]`` of its own (and ``[num_pages, page_size,
*shape]`` for every further per-token tensor it declares).  Every group has a
pool of its own size: a group whose retention rule lets go of old tokens never
holds more than a chunk (or window) plus one step's portion per request, so it
needs far fewer pages than a group that keeps everything (:func:`pool_sizes`).
"""
from __future__ import annotations

import dataclasses
from typing import Optional

import torch

from ..parts.base import CacheNeed, first_needed_position, kept_prefix, retention_kind
from .pages import OutOfPages, OutOfSlots, PagePool, SlotPool


@dataclasses.dataclass
class CacheGroup:
    index: int
    kv_heads: int  # 0: no keys and values in the attention kernels' layout
    head_dim: int
    retention: tuple
    cache_ids: list[int]
    pool: PagePool
    tensors: dict[int, torch.Tensor]  # per run: [pages, 2, kv_heads, page_size, head_dim]
    paged: tuple = ()  # further per-token tensors: (name, shape) pairs
    pages: dict[int, dict[str, torch.Tensor]] = dataclasses.field(default_factory=dict)  # per run, by name
    itemsize: int = 2

    def bytes_per_token(self, itemsize: int | None = None) -> int:
        """Bytes one token takes in this group, over all its runs."""
        if itemsize is None:
            itemsize = self.itemsize
        per_run = 2 * self.kv_heads * self.head_dim
        for _, shape in self.paged:
            n = 1
            for d in shape:
                n *= d
            per_run += n
        return len(self.cache_ids) * per_run * itemsize


@dataclasses.dataclass
class RequestEntry:
    slot: int
    num_tokens: int = 0  # tokens whose keys and values are written (committed)
    reserved: int = 0  # tokens beyond num_tokens that have pages for the running step
    tables: list[list[int]] = dataclasses.field(default_factory=list)  # per group: page id or -1 per page index
    versions: list[int] = dataclasses.field(default_factory=list)  # per group: counts the changes of its table
    serial: int = 0  # which life of which request this is: no two calls of add_request give the same
    freed_upto: list[int] = dataclasses.field(default_factory=list)  # per group: pages below this index (and beyond
    # the rule's kept prefix) have been given back


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
    pages: Optional[dict] = None  # further per-token tensors of this run, by name: [pages, page_size, *shape]


def group_key(need: CacheNeed):
    """Runs whose needs give the same key share page ids and block tables; ``None``: no pages."""
    if need.kv is None and not need.paged:
        return None
    kv = (0, 0) if need.kv is None else (int(need.kv[0]), int(need.kv[1]))
    paged = tuple((str(n), tuple(int(d) for d in shape)) for n, shape in need.paged)
    return (kv, paged, tuple(need.retention))


def plan_groups(needs: dict[int, CacheNeed]) -> list[tuple[tuple, list[int]]]:
    """The groups the manager will form, in its order: ``(key, cache ids)``."""
    out: list[tuple[tuple, list[int]]] = []
    index: dict[tuple, int] = {}
    for cid in sorted(needs):
        key = group_key(needs[cid])
        if key is None:
            continue
        if key not in index:
            index[key] = len(out)
            out.append((key, []))
        out[index[key]][1].append(cid)
    return out


def tokens_held_at_most(retention: tuple, max_step_tokens: int, max_seq_len: Optional[int]) -> Optional[int]:
    """The most tokens of one request that a group with this retention rule holds at any time
    (``None``: no bound but the sequence's length): what the rule keeps for the next query plus the
    portion of the running step, whose pages are given back only after it."""
    cap = retention_kind(retention).held_at_most(retention, max_step_tokens)
    if max_seq_len is not None:
        cap = max_seq_len if cap is None else min(cap, max_seq_len)
    return cap


def pool_sizes(needs: dict[int, CacheNeed], *, page_size: int, itemsize: int, max_requests: int,
               max_step_tokens: int, max_seq_len: Optional[int] = None, cache_tokens: Optional[int] = None,
               memory_bytes: Optional[int] = None) -> dict[int, int]:
    """Pages for every group's pool.  Either ``cache_tokens`` (the tokens that a group which keeps
    everything can hold) or ``memory_bytes`` (what all pools together may take: then the largest
    such number of tokens that fits).  A group that lets go of old tokens gets at most what
    ``max_requests`` requests can hold of it (whole pages, and one more per request for a portion
    that does not start at a page's edge)."""
    groups = plan_groups(needs)
    caps, page_bytes = [], []
    for (kv, paged, retention), cids in groups:
        held = tokens_held_at_most(retention, max_step_tokens, max_seq_len)
        caps.append(None if held is None else max_requests * (-(-held // page_size) + 1))
        per = 2 * kv[0] * kv[1]
        for _, shape in paged:
            n = 1
            for d in shape:
                n *= d
            per += n
        page_bytes.append(len(cids) * per * page_size * itemsize)

    def sizes(pages_unbounded: int) -> list[int]:
        return [pages_unbounded if c is None else min(c, pages_unbounded) for c in caps]

    if cache_tokens is not None:
        want = -(-cache_tokens // page_size)
    elif memory_bytes is not None:
        def total(p):
            return sum(b * n for b, n in zip(page_bytes, sizes(p)))

        lo, hi = 0, 1
        while total(hi) <= memory_bytes and hi < (1 << 40):
            if all(c is not None and c <= hi for c in caps):
                break  # every pool is at its bound: more pages would hold nothing
            lo, hi = hi, hi * 2
        if total(hi) <= memory_bytes:
            lo = hi
        while lo + 1 < hi:
            mid = (lo + hi) // 2
            if total(mid) <= memory_bytes:
                lo = mid
            else:
                hi = mid
        want = lo
        if want < 1:
            raise ValueError(f"{memory_bytes} bytes do not hold one page of every group "
                             f"({sum(page_bytes)} bytes)")
    else:
        raise ValueError("give cache_tokens or memory_bytes")
    return dict(enumerate(sizes(want)))


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
        self._lives = 0  # requests added so far
        item = torch.empty((), dtype=dtype).element_size()
        for key, cids in plan_groups(needs):
            (hk, dh), paged, retention = key
            retention_kind(retention)  # (an unknown rule is an error here, not at the first page given back)
            i = len(self.groups)
            n = num_pages[i] if isinstance(num_pages, dict) else num_pages
            g = CacheGroup(i, hk, dh, retention, list(cids), PagePool(n), {}, paged=paged, itemsize=item)
            self.groups.append(g)
            for cid in cids:
                self.group_of[cid] = i
        for cid in sorted(needs):
            need = needs[cid]
            if need.state_shape is not None:
                self.state[cid] = torch.zeros(
                    (max_requests, *need.state_shape), dtype=need.state_dtype or torch.float32, device=self.device
                )
        fill = float("nan") if poison else 0.0
        for g in self.groups:
            for cid in g.cache_ids:
                if g.kv_heads:
                    g.tensors[cid] = torch.full(
                        (g.pool.num_pages, 2, g.kv_heads, page_size, g.head_dim), fill, dtype=dtype, device=self.device
                    )
                g.pages[cid] = {
                    name: torch.full((g.pool.num_pages, page_size, *shape), fill, dtype=dtype, device=self.device)
                    for name, shape in g.paged
                }

    # ------------------------------------------------------------------ requests
    def add_request(self, rid) -> RequestEntry:
        if rid in self.requests:
            raise KeyError(f"request {rid!r} is already live")
        slot = self.slots.alloc()
        for t in self.state.values():
            t[slot].zero_()
        self._lives += 1
        e = RequestEntry(slot=slot, tables=[[] for _ in self.groups], versions=[0 for _ in self.groups],
                         serial=self._lives, freed_upto=[0 for _ in self.groups])
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
            if got:
                e.versions[g.index] += 1
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
            # page j holds positions [j*ps, (j+1)*ps): free iff it lies wholly in [kept prefix, keep_from)
            first = max(e.freed_upto[g.index], -(-kept_prefix(g.retention) // self.page_size))
            upto = min(len(table), keep_from // self.page_size)
            gone = [j for j in range(first, upto) if table[j] >= 0]
            e.freed_upto[g.index] = max(e.freed_upto[g.index], upto)
            if gone:
                self._release(g, [table[j] for j in gone])
                e.versions[g.index] += 1
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
            if len(table) > last_used + 1:
                e.versions[g.index] += 1
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
            for named in g.pages.values():
                for t in named.values():
                    t.index_fill_(0, idx, float("nan"))

    # ------------------------------------------------------------------ queries
    def num_tokens(self, rid) -> int:
        return self.requests[rid].num_tokens

    def slot(self, rid) -> int:
        return self.requests[rid].slot

    def table(self, rid, group: int) -> list[int]:
        return self.requests[rid].tables[group]

    def table_version(self, rid, group: int) -> int:
        """Changes whenever the request's block table of this group does (a copy kept elsewhere is then stale)."""
        return self.requests[rid].versions[group]

    def table_stamp(self, rid) -> tuple:
        """Equal stamps mean equal block tables: a copy of this request's tables kept elsewhere (a recorded
        step's device buffer) is good as long as the stamp it was made under comes again.  The stamp names
        this life of the request (a request that ended and was added again under the same id, as after a
        preemption, has another: its version counts start again, its pages are others) and counts the
        changes of every group's table."""
        e = self.requests[rid]
        return (e.serial, *e.versions)

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
        return sum(g.bytes_per_token() for g in self.groups)

    def pool_bytes(self) -> int:
        """Device memory of all page pools."""
        return sum(g.bytes_per_token() * self.page_size * g.pool.num_pages for g in self.groups)


__all__ = ["CacheManager", "CacheView", "CacheGroup", "OutOfPages", "OutOfSlots", "pool_sizes", "plan_groups",
           "tokens_held_at_most"]
