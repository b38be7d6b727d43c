"""Page and slot allocators (host-side bookkeeping only)."""
from __future__ import annotations


class OutOfPages(RuntimeError):
    """Raised when a pool cannot give the pages asked for; nothing was taken."""


class OutOfSlots(RuntimeError):
    pass


class PagePool:
    """Fixed set of page ids with a LIFO free list: the page given back last is
    handed out first, so stale contents are met as early as possible."""

    def __init__(self, num_pages: int) -> None:
        if num_pages < 0:
            raise ValueError("num_pages must be >= 0")
        self.num_pages = num_pages
        self._free = list(range(num_pages - 1, -1, -1))
        self._held = bytearray(num_pages)
        self.handed_out = 0  # pages given out so far (more than num_pages: pages were used again)

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_held(self) -> int:
        return self.num_pages - len(self._free)

    def alloc(self, n: int) -> list[int]:
        if n > len(self._free):
            raise OutOfPages(f"asked for {n} pages, {len(self._free)} of {self.num_pages} free")
        out = [self._free.pop() for _ in range(n)]
        self.handed_out += n
        for p in out:
            if self._held[p]:
                raise AssertionError(f"page {p} handed out twice")
            self._held[p] = 1
        return out

    def release(self, pages) -> None:
        for p in pages:
            if not 0 <= p < self.num_pages:
                raise AssertionError(f"page {p} does not belong to this pool")
            if not self._held[p]:
                raise AssertionError(f"page {p} given back twice")
            self._held[p] = 0
            self._free.append(p)

    def check(self) -> None:
        """Every page is either free exactly once or held."""
        if len(set(self._free)) != len(self._free):
            raise AssertionError("a page is on the free list twice")
        for p in self._free:
            if self._held[p]:
                raise AssertionError(f"page {p} is both free and held")
        if sum(self._held) + len(self._free) != self.num_pages:
            raise AssertionError("a page was lost")


class SlotPool:
    """Slots for fixed-size per-request state; lowest free index first."""

    def __init__(self, num_slots: int) -> None:
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))
        self._held = bytearray(num_slots)

    @property
    def num_free(self) -> int:
        return len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise OutOfSlots(f"all {self.num_slots} request slots are in use")
        s = self._free.pop()
        self._held[s] = 1
        return s

    def release(self, s: int) -> None:
        if not self._held[s]:
            raise AssertionError(f"slot {s} given back twice")
        self._held[s] = 0
        self._free.append(s)
        self._free.sort(reverse=True)
