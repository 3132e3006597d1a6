"""Host-side bookkeeping of cache pages and of fixed-size state slots.

A ``PagePool`` hands out page ids from a fixed set and takes them back; it knows
nothing of tensors.  The reference's pool tracks Free / Reserved / Live / Retired blocks
with typed, side-effect-free exhaustion (crates/macllm-kv/src/cache.rs:294-299,
:649-658); with one stream every later kernel is ordered after the earlier ones, so a
page is reusable as soon as it is freed and two states are enough.
"""
from __future__ import annotations

from typing import Dict, List


class CacheExhausted(RuntimeError):
    """A reservation asked for more pages (or slots) than are free.  Nothing was changed.
    (crates/macllm-kv/src/cache.rs:649-658; src/architecture.rs:930-936)"""

    def __init__(self, what: str, requested: int, free: int, total: int):
        self.what, self.requested, self.free, self.total = what, requested, free, total
        super().__init__(f"cache exhausted: {requested} {what} requested, only {free} of {total} are free")


class PagePool:
    """``total`` page ids 0..total-1.  The most recently freed page is handed out first,
    so a small pool reuses pages at once."""

    def __init__(self, total: int):
        if total <= 0:
            raise ValueError("a page pool needs at least one page")
        self.total = total
        self._free: List[int] = list(range(total - 1, -1, -1))
        self._held = [False] * total

    @property
    def free_count(self) -> int:
        return len(self._free)

    @property
    def used_count(self) -> int:
        return self.total - len(self._free)

    def alloc(self, count: int) -> List[int]:
        if count < 0:
            raise ValueError("negative page count")
        if count > len(self._free):
            raise CacheExhausted("pages", count, len(self._free), self.total)
        pages = [self._free.pop() for _ in range(count)]
        for page in pages:
            self._held[page] = True
        return pages

    def free(self, pages) -> None:
        pages = list(pages)
        for page in pages:
            if not (0 <= page < self.total) or not self._held[page]:
                raise RuntimeError(f"page {page} is freed but is not held")
            self._held[page] = False
        self._free.extend(pages)

    def check(self, held_elsewhere: List[int]) -> None:
        """Every page is either free or in ``held_elsewhere``, exactly once
        (the scan-based cross-check of crates/macllm-kv/src/cache.rs:3810-3841)."""
        seen = sorted(self._free) + sorted(held_elsewhere)
        if sorted(seen) != list(range(self.total)):
            raise AssertionError("page accounting is broken: a page is lost or held twice")
        for page in held_elsewhere:
            if not self._held[page]:
                raise AssertionError(f"page {page} is in a block table but marked free")


class SlotPool:
    """Ids of the fixed-size per-request state slots."""

    def __init__(self, total: int):
        if total <= 0:
            raise ValueError("a slot pool needs at least one slot")
        self.total = total
        self._free: List[int] = list(range(total - 1, -1, -1))
        self._held = [False] * total

    @property
    def free_count(self) -> int:
        return len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise CacheExhausted("state slots", 1, 0, self.total)
        slot = self._free.pop()
        self._held[slot] = True
        return slot

    def free(self, slot: int) -> None:
        if not (0 <= slot < self.total) or not self._held[slot]:
            raise RuntimeError(f"state slot {slot} is freed but is not held")
        self._held[slot] = False
        self._free.append(slot)


class BlockTable:
    """One request's pages in one group: logical page index -> page id, or -1 once a
    window has passed the page and it was given back
    (crates/macllm-kv/src/cache.rs:1434-1440)."""

    def __init__(self):
        self.pages: List[int] = []
        self.first_live = 0          # logical pages before this one were given back

    def live_pages(self) -> List[int]:
        return [page for page in self.pages if page >= 0]
