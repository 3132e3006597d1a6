"""The cache manager: keys and values in pages with a block table per request, one pool
per group of layers with the same needs, and slots for per-request state of fixed size.

What a mixer needs is declared by the mixer (``KVNeed`` / ``StateNeed``); the manager
groups equal ``KVNeed``s (same heads, head size and window) into one ``PagedGroup`` whose
pages hold every member layer, so one block table per request serves all of them
(layout [page, layer, K|V, kv_head, token x dim], V transposed inside its block; crates/macllm-kv/src/cache.rs:558-566,
one pool per geometry :165-169).  Layers that keep all keys and layers that keep a
window are different groups: a window group gives a page back as soon as every query
still to come is past it.

Before a step all lanes' growth is reserved at once, all or nothing
(crates/macllm-kv/src/cache.rs:2331-2445); ``commit`` advances the lengths after the
step; ``finish`` gives everything back (:1840-1852).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import torch

from .pages import BlockTable, CacheExhausted, PagePool, SlotPool


@dataclass(frozen=True)
class KVNeed:
    """Token-proportional cache: K and V of ``num_kv_heads`` x ``head_dim`` per token;
    ``window`` = how many of the most recent tokens must stay (None = all)."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateNeed:
    """Fixed-size per-request state ``name`` of ``shape``; dtype "activation" or "float32"."""
    name: str
    shape: Tuple[int, ...]
    dtype: str = "float32"


class PagedGroup:
    def __init__(self, need: KVNeed, page_size: int, num_pages: int):
        self.need = need
        self.page_size = page_size
        self.pool = PagePool(num_pages)
        self.members: List[Hashable] = []
        self.tables: Dict[Hashable, BlockTable] = {}
        self.storage: Optional[torch.Tensor] = None

    def add_member(self, key: Hashable) -> int:
        self.members.append(key)
        return len(self.members) - 1

    def allocate(self, dtype: torch.dtype, device) -> None:
        need = self.need
        # one page more than the pool hands out: the scratch page padding lanes of a captured step write to
        self.storage = torch.zeros((self.pool.total + 1, len(self.members), 2, need.num_kv_heads,
                                    self.page_size * need.head_dim), dtype=dtype, device=device)

    @property
    def scratch_page(self) -> int:
        return self.pool.total

    def layer_views(self, layer: int):
        """One layer's K pages [pages, Hkv, page_size, dh] and V pages [pages, Hkv, dh, page_size]
        (V is kept transposed: its product contracts over tokens)."""
        need = self.need
        return (self.storage[:, layer, 0].unflatten(-1, (self.page_size, need.head_dim)),
                self.storage[:, layer, 1].unflatten(-1, (need.head_dim, self.page_size)))

    def bytes_per_page(self, element_size: int) -> int:
        need = self.need
        return 2 * len(self.members) * need.num_kv_heads * self.page_size * need.head_dim * element_size

    # -- per request
    def pages_missing(self, request: Hashable, new_length: int) -> int:
        table = self.tables[request]
        wanted = -(-new_length // self.page_size)
        return max(0, wanted - len(table.pages))

    def grow(self, request: Hashable, new_length: int) -> None:
        table = self.tables[request]
        table.pages.extend(self.pool.alloc(self.pages_missing(request, new_length)))

    def release_passed(self, request: Hashable, length: int) -> None:
        """Give back the pages every later query is past: with a window w the next query
        (position ``length``) sees keys >= length - w + 1."""
        window = self.need.window
        if window is None:
            return
        table = self.tables[request]
        first_needed_key = length - window + 1
        if first_needed_key <= 0:
            return
        first_needed_page = min(first_needed_key // self.page_size, len(table.pages))
        passed = [table.pages[index] for index in range(table.first_live, first_needed_page)]
        if passed:
            self.pool.free(passed)
            for index in range(table.first_live, first_needed_page):
                table.pages[index] = -1
            table.first_live = first_needed_page

    def release_all(self, request: Hashable) -> None:
        table = self.tables.pop(request)
        self.pool.free(table.live_pages())

    def check(self) -> None:
        held = [page for table in self.tables.values() for page in table.live_pages()]
        self.pool.check(held)


class RequestCache:
    def __init__(self, slot: int):
        self.slot = slot
        self.length = 0          # tokens whose keys, values and state are in the cache


@dataclass
class EntryCache:
    """What one mixer of one schedule entry sees: its layer's K and V views of a paged
    group (``owns_kv`` False when it reads another entry's) and its state tensors
    [slots, *shape]."""
    group: Optional[int] = None
    k_cache: Optional[torch.Tensor] = None
    v_cache: Optional[torch.Tensor] = None
    owns_kv: bool = True
    states: Optional[Dict[str, torch.Tensor]] = None


class CacheManager:
    def __init__(self, needs: Dict[Hashable, Sequence[object]], shared_kv: Dict[Hashable, Hashable],
                 page_size: int, capacity_tokens: int, max_requests: int, dtype: torch.dtype, device):
        """``needs``: (entry, mixer) key -> the mixer's needs.  ``shared_kv``: key of a mixer
        that reads -> key of the mixer whose K/V it reads."""
        if page_size <= 0 or capacity_tokens <= 0 or max_requests <= 0:
            raise ValueError("page_size, capacity_tokens and max_requests must be positive")
        self.page_size = page_size
        self.dtype = dtype
        self.device = torch.device(device)
        num_pages = -(-capacity_tokens // page_size)
        self.groups: List[PagedGroup] = []
        self.entries: Dict[Hashable, EntryCache] = {}
        self.slots = SlotPool(max_requests)
        self.requests: Dict[Hashable, RequestCache] = {}
        self._state_tensors: List[torch.Tensor] = []
        group_of: Dict[KVNeed, int] = {}
        layer_of: Dict[Hashable, Tuple[int, int]] = {}
        for key, key_needs in needs.items():
            entry = EntryCache(states={})
            for need in key_needs:
                if isinstance(need, KVNeed):
                    if key in shared_kv:
                        continue
                    if need not in group_of:
                        group_of[need] = len(self.groups)
                        self.groups.append(PagedGroup(need, page_size, num_pages))
                    group = group_of[need]
                    layer_of[key] = (group, self.groups[group].add_member(key))
                elif isinstance(need, StateNeed):
                    state_dtype = dtype if need.dtype == "activation" else torch.float32
                    # one slot more than the pool hands out: the scratch slot of padding lanes
                    tensor = torch.zeros((max_requests + 1,) + tuple(need.shape), dtype=state_dtype,
                                         device=self.device)
                    entry.states[need.name] = tensor
                    self._state_tensors.append(tensor)
                else:
                    raise TypeError(f"unknown cache need {need!r}")
            self.entries[key] = entry
        for group in self.groups:
            group.allocate(dtype, self.device)
        for key, entry in self.entries.items():
            source = shared_kv.get(key, key)
            if source in layer_of:
                if key in shared_kv:
                    own = [need for need in needs[key] if isinstance(need, KVNeed)]
                    theirs = self.groups[layer_of[source][0]].need
                    if not own or own[0] != theirs:
                        raise ValueError(f"{key} cannot read the cache of {source}: their needs differ")
                group, layer = layer_of[source]
                entry.group = group
                entry.k_cache, entry.v_cache = self.groups[group].layer_views(layer)
                entry.owns_kv = key not in shared_kv
            elif key in shared_kv:
                raise ValueError(f"{key} reads the cache of {source}, which keeps none")

    @property
    def scratch_slot(self) -> int:
        return self.slots.total

    # ------------------------------------------------------------------ requests
    def add_request(self, request: Hashable) -> RequestCache:
        if request in self.requests:
            raise KeyError(f"request {request!r} is already live")
        slot = self.slots.alloc()
        record = RequestCache(slot)
        self.requests[request] = record
        for group in self.groups:
            group.tables[request] = BlockTable()
        if self._state_tensors:                       # a fresh request starts from zeros
            torch._foreach_zero_([tensor[slot] for tensor in self._state_tensors])
        return record

    def can_ever_fit(self, total_tokens: int) -> bool:
        """Whether a request of ``total_tokens`` fits an empty cache
        (the admission check of src/engine.rs:2839-2863)."""
        return all(-(-total_tokens // group.page_size) <= group.pool.total for group in self.groups)

    def reserve(self, growth: Sequence[Tuple[Hashable, int]]) -> None:
        """Pages for ``tokens`` more tokens of every listed request, all or nothing."""
        for request, tokens in growth:
            if request not in self.requests:
                raise KeyError(f"request {request!r} is not live")
            if tokens <= 0:
                raise ValueError("a lane needs at least one token")
        for group in self.groups:
            missing = sum(group.pages_missing(request, self.requests[request].length + tokens)
                          for request, tokens in growth)
            if missing > group.pool.free_count:
                raise CacheExhausted("pages", missing, group.pool.free_count, group.pool.total)
        for group in self.groups:
            for request, tokens in growth:
                group.grow(request, self.requests[request].length + tokens)

    def commit(self, request: Hashable, tokens: int) -> None:
        record = self.requests[request]
        record.length += tokens
        for group in self.groups:
            group.release_passed(request, record.length)

    def finish(self, request: Hashable) -> None:
        record = self.requests.pop(request)
        for group in self.groups:
            group.release_all(request)
        self.slots.free(record.slot)

    # ------------------------------------------------------------------ views and reports
    def entry(self, key: Hashable) -> EntryCache:
        return self.entries[key]

    def table(self, group: int, request: Hashable) -> BlockTable:
        return self.groups[group].tables[request]

    def stats(self) -> dict:
        return {
            "groups": [{"window": group.need.window, "layers": len(group.members),
                        "total_pages": group.pool.total, "free_pages": group.pool.free_count,
                        "used_pages": group.pool.used_count} for group in self.groups],
            "total_slots": self.slots.total, "free_slots": self.slots.free_count,
            "live_requests": len(self.requests),
        }

    def check(self) -> None:
        for group in self.groups:
            group.check()
