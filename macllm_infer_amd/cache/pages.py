"""Host-side bookkeeping of cache pages and of fixed-size state slots.

A ``PagePool`` hands out page ids from a fixed set and takes them back; it knows
nothing of tensors.  The reference's pool tracks Free / Reserved / Live / Retired blocks
with typed, side-effect-free exhaustion (crates/macllm-kv/src/cache.rs:294-299,
:649-658); with one stream every later kernel is ordered after the earlier ones, so a
page is reusable as soon as it is freed and two states are enough.

The pools and tables themselves live in the host-side core (``csrc/hostcore.cpp``); the
classes here are views of them.
"""
from __future__ import annotations

from typing import List

import numpy as np

from . import native


class CacheExhausted(RuntimeError):
    """A reservation asked for more pages (or slots) than are free.  Nothing was changed.
    (crates/macllm-kv/src/cache.rs:649-658; src/architecture.rs:930-936)"""

    def __init__(self, what: str, requested: int, free: int, total: int):
        self.what, self.requested, self.free, self.total = what, requested, free, total
        super().__init__(f"cache exhausted: {requested} {what} requested, only {free} of {total} are free")


class PagePool:
    """``total`` page ids 0..total-1.  The most recently freed page is handed out first,
    so a small pool reuses pages at once.  ``PagePool(total)`` makes a pool of its own;
    ``PagePool.view(pointer, owner)`` looks at one inside a cache core."""
    what = "pages"

    def __init__(self, total: int):
        if total <= 0:
            raise ValueError("a pool needs at least one id")
        self._lib = native.lib()
        self._pool = self._lib.hc_pool_create(total)
        self._owner = None

    @classmethod
    def view(cls, pointer, owner):
        pool = cls.__new__(cls)
        pool._lib = native.lib()
        pool._pool = pointer
        pool._owner = owner                  # keeps the core alive
        return pool

    def __del__(self):
        if getattr(self, "_owner", True) is None and getattr(self, "_pool", None):
            self._lib.hc_pool_destroy(self._pool)
            self._pool = None

    @property
    def total(self) -> int:
        return self._lib.hc_pool_total(self._pool)

    @property
    def free_count(self) -> int:
        return self._lib.hc_pool_free_count(self._pool)

    @property
    def used_count(self) -> int:
        return self.total - self.free_count

    def alloc(self, count: int) -> List[int]:
        if count < 0:
            raise ValueError("negative count")
        out = np.empty(max(count, 1), dtype=np.int32)
        if self._lib.hc_pool_take(self._pool, count, native.int_pointer(out)) != 0:
            raise CacheExhausted(self.what, count, self.free_count, self.total)
        return out[:count].tolist()

    def free(self, pages) -> None:
        ids = native.as_ints(list(pages))
        if self._lib.hc_pool_give(self._pool, native.int_pointer(ids), len(ids)) != 0:
            raise RuntimeError(f"one of the {self.what} {ids.tolist()} is freed but is not held")

    def check(self, held_elsewhere: List[int]) -> None:
        """Every id is either free or in ``held_elsewhere``, exactly once
        (the scan-based cross-check of crates/macllm-kv/src/cache.rs:3810-3841)."""
        ids = native.as_ints(list(held_elsewhere))
        code = self._lib.hc_pool_check(self._pool, native.int_pointer(ids), len(ids))
        if code == 1:
            raise AssertionError(f"accounting of {self.what} is broken: one is lost or held twice")
        if code == 2:
            raise AssertionError(f"one of the {self.what} is in a block table but marked free")


class SlotPool(PagePool):
    """Ids of the fixed-size per-request state slots."""
    what = "state slots"

    def alloc(self) -> int:                      # one slot at a time
        return PagePool.alloc(self, 1)[0]

    def free(self, slot: int) -> None:
        PagePool.free(self, [slot])


class BlockTable:
    """One request's pages in one group: logical page index -> page id, or -1 once a
    window has passed the page and it was given back
    (crates/macllm-kv/src/cache.rs:1434-1440).  A view of the core's table."""

    def __init__(self, core, group: int, slot: int):
        self._core, self._group, self._slot = core, group, slot

    @property
    def pages(self) -> List[int]:
        lib = native.lib()
        count = lib.hc_table(self._core.pointer, self._group, self._slot, None, 0)
        out = np.empty(max(count, 1), dtype=np.int32)
        lib.hc_table(self._core.pointer, self._group, self._slot, native.int_pointer(out), count)
        return out[:count].tolist()

    @property
    def first_live(self) -> int:
        """Logical pages before this one were given back."""
        return native.lib().hc_first_live(self._core.pointer, self._group, self._slot)

    def live_pages(self) -> List[int]:
        return [page for page in self.pages if page >= 0]
