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

import numpy as np
import torch

from . import native
from .pages import BlockTable, CacheExhausted, PagePool, SlotPool


@dataclass(frozen=True)
class KVNeed:
    """Token-proportional cache: per token, keys of ``num_kv_heads`` x ``head_dim`` and values of
    ``num_kv_heads`` x ``value_dim`` (None: the keys' width); ``window`` = how many of the most recent
    tokens must stay (None = all)."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    value_dim: Optional[int] = None
    token_proportional = True             # what tells this need from one of fixed size, whatever its class

    @property
    def value_width(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim


@dataclass(frozen=True)
class StateNeed:
    """Fixed-size per-request state ``name`` of ``shape``; dtype "activation" (the engine's 16- or 32-bit
    dtype), "float32", or any ``torch.dtype``."""
    name: str
    shape: Tuple[int, ...]
    dtype: object = "float32"
    token_proportional = False

    def storage_dtype(self, activation: torch.dtype) -> torch.dtype:
        if isinstance(self.dtype, torch.dtype):
            return self.dtype
        if self.dtype == "activation":
            return activation
        if self.dtype == "float32":
            return torch.float32
        raise ValueError(f"state {self.name!r}: dtype {self.dtype!r} is neither 'activation', 'float32' nor a torch.dtype")


class Core:
    """The host-side core of one cache manager (``csrc/hostcore.cpp``): every group's page pool
    and block tables, the slot pool and the requests' lengths."""

    def __init__(self, page_sizes: Sequence[int], num_pages: Sequence[int], windows: Sequence[Optional[int]],
                 max_requests: int):
        self.lib = native.lib()
        sizes, pages = native.as_ints(list(page_sizes)), native.as_ints(list(num_pages))
        spans = native.as_ints([window or -1 for window in windows])
        self.pointer = self.lib.hc_create(len(sizes), native.int_pointer(sizes), native.int_pointer(pages),
                                          native.int_pointer(spans), max_requests)
        if not self.pointer:
            raise ValueError("page sizes, page counts and the number of requests must be positive")

    def __del__(self):
        if getattr(self, "pointer", None):
            self.lib.hc_destroy(self.pointer)
            self.pointer = None


class PagedGroup:
    """The layers with one ``KVNeed``: their storage, and a view of the group's pool and tables
    in the core."""

    def __init__(self, need: KVNeed, page_size: int, num_pages: int):
        self.need = need
        self.page_size = page_size
        self.num_pages = num_pages
        self.members: List[Hashable] = []
        self.tables: Dict[Hashable, BlockTable] = {}
        self.storage: Optional[torch.Tensor] = None
        self.pool: Optional[PagePool] = None          # set once the core exists

    def add_member(self, key: Hashable) -> int:
        self.members.append(key)
        return len(self.members) - 1

    def allocate(self, dtype: torch.dtype, device) -> None:
        need = self.need
        # one page more than the pool hands out: the scratch page padding lanes of a captured step write to.
        # A layer's share of a page: its keys [kv head, token, key dim], then its values [kv head, value dim, token]
        self.storage = torch.zeros((self.num_pages + 1, len(self.members),
                                    need.num_kv_heads * self.page_size * (need.head_dim + need.value_width)),
                                   dtype=dtype, device=device)

    @property
    def scratch_page(self) -> int:
        return self.num_pages

    def layer_views(self, layer: int):
        """One layer's K pages [pages, Hkv, page_size, key dim] and V pages [pages, Hkv, value dim, page_size]
        (V is kept transposed: its product contracts over tokens)."""
        need = self.need
        keys = need.num_kv_heads * self.page_size * need.head_dim
        return (self.storage[:, layer, :keys].unflatten(-1, (need.num_kv_heads, self.page_size, need.head_dim)),
                self.storage[:, layer, keys:].unflatten(-1, (need.num_kv_heads, need.value_width, self.page_size)))

    def bytes_per_page(self, element_size: int) -> int:
        need = self.need
        return (len(self.members) * need.num_kv_heads * self.page_size * (need.head_dim + need.value_width)
                * element_size)

    def check(self) -> None:
        held = [page for table in self.tables.values() for page in table.live_pages()]
        self.pool.check(held)


class RequestCache:
    """A live request: its state slot (which is also its handle in the core) and its length."""

    def __init__(self, core: Core, slot: int):
        self._core = core
        self.slot = slot

    @property
    def length(self) -> int:
        """Tokens whose keys, values and state are in the cache."""
        return self._core.lib.hc_length(self._core.pointer, self.slot)


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
        self.max_requests = max_requests
        self.requests: Dict[Hashable, RequestCache] = {}
        self._state_tensors: List[torch.Tensor] = []
        group_of: Dict[KVNeed, int] = {}
        layer_of: Dict[Hashable, Tuple[int, int]] = {}
        for key, key_needs in needs.items():
            entry = EntryCache(states={})
            for need in key_needs:
                if getattr(need, "token_proportional", False):
                    if key in shared_kv:
                        continue
                    if need not in group_of:
                        group_of[need] = len(self.groups)
                        self.groups.append(PagedGroup(need, page_size, num_pages))
                    group = group_of[need]
                    layer_of[key] = (group, self.groups[group].add_member(key))
                elif isinstance(need, StateNeed):
                    state_dtype = need.storage_dtype(dtype)
                    # one slot more than the pool hands out: the scratch slot of padding lanes
                    tensor = torch.zeros((max_requests + 1,) + tuple(need.shape), dtype=state_dtype,
                                         device=self.device)
                    entry.states[need.name] = tensor
                    self._state_tensors.append(tensor)
                else:
                    raise TypeError(f"unknown cache need {need!r}")
            self.entries[key] = entry
        self.core = Core([group.page_size for group in self.groups], [group.num_pages for group in self.groups],
                         [group.need.window for group in self.groups], max_requests)
        self.slots = SlotPool.view(self.core.lib.hc_slot_pool(self.core.pointer), self.core)
        for index, group in enumerate(self.groups):
            group.pool = PagePool.view(self.core.lib.hc_group_pool(self.core.pointer, index), self.core)
            group.allocate(dtype, self.device)
        for key, entry in self.entries.items():
            source = shared_kv.get(key, key)
            if source in layer_of:
                if key in shared_kv:
                    own = [need for need in needs[key] if getattr(need, "token_proportional", False)]
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
        return self.max_requests

    # ------------------------------------------------------------------ requests
    def add_request(self, request: Hashable) -> RequestCache:
        if request in self.requests:
            raise KeyError(f"request {request!r} is already live")
        slot = self.core.lib.hc_add_request(self.core.pointer)
        if slot < 0:
            raise CacheExhausted("state slots", 1, 0, self.max_requests)
        record = RequestCache(self.core, slot)
        self.requests[request] = record
        for index, group in enumerate(self.groups):
            group.tables[request] = BlockTable(self.core, index, slot)
        if self._state_tensors:                       # a fresh request starts from zeros
            torch._foreach_zero_([tensor[slot] for tensor in self._state_tensors])
        return record

    def can_ever_fit(self, total_tokens: int) -> bool:
        """Whether a request of ``total_tokens`` fits an empty cache
        (the admission check of src/engine.rs:2839-2863)."""
        return all(-(-total_tokens // group.page_size) <= group.num_pages for group in self.groups)

    def slots_of(self, requests: Sequence[Hashable]) -> np.ndarray:
        """The core's handles of live requests (KeyError for one that is not live)."""
        records = self.requests
        try:
            return np.fromiter((records[request].slot for request in requests), dtype=np.int32, count=len(requests))
        except KeyError as error:
            raise KeyError(f"request {error.args[0]!r} is not live") from None

    def lengths_of(self, slots: np.ndarray) -> np.ndarray:
        out = np.empty(len(slots), dtype=np.int32)
        self.core.lib.hc_lengths(self.core.pointer, len(slots), native.int_pointer(slots), native.int_pointer(out))
        return out

    def reserve(self, growth: Sequence[Tuple[Hashable, int]]) -> None:
        """Pages for ``tokens`` more tokens of every listed request, all or nothing."""
        self.reserve_slots(self.slots_of([request for request, _ in growth]),
                           native.as_ints([tokens for _, tokens in growth]))

    def reserve_slots(self, slots: np.ndarray, tokens: np.ndarray) -> None:
        info = np.zeros(4, dtype=np.int32)
        code = self.core.lib.hc_reserve(self.core.pointer, len(slots), native.int_pointer(slots),
                                        native.int_pointer(tokens), native.int_pointer(info))
        if code == 1:
            raise CacheExhausted("pages", int(info[1]), int(info[2]), int(info[3]))
        if code != 0:
            raise ValueError(f"lane {int(info[0])} of the reservation: a request named twice, or no tokens")

    def commit(self, request: Hashable, tokens: int) -> None:
        self.commit_slots(self.slots_of([request]), native.as_ints([tokens]))

    def commit_slots(self, slots: np.ndarray, tokens: np.ndarray) -> None:
        """The step ran: lengths advance and window groups give back the pages all later queries
        are past."""
        if self.core.lib.hc_commit(self.core.pointer, len(slots), native.int_pointer(slots),
                                   native.int_pointer(tokens)) != 0:
            raise RuntimeError("commit of a request that is not live, or broken page accounting")

    def finish(self, request: Hashable) -> None:
        record = self.requests.pop(request)
        for group in self.groups:
            del group.tables[request]
        if self.core.lib.hc_finish(self.core.pointer, record.slot) != 0:
            raise RuntimeError(f"request {request!r}: its slot or pages were not held")

    # ------------------------------------------------------------------ views and reports
    def entry(self, key: Hashable) -> EntryCache:
        return self.entries[key]

    def table(self, group: int, request: Hashable) -> BlockTable:
        return self.groups[group].tables[request]

    def stats(self) -> dict:
        return {
            "groups": [{"window": group.need.window, "layers": len(group.members),
                        "total_pages": group.num_pages, "free_pages": group.pool.free_count,
                        "used_pages": group.pool.used_count} for group in self.groups],
            "total_slots": self.max_requests, "free_slots": self.slots.free_count,
            "live_requests": len(self.requests),
        }

    def check(self) -> None:
        """No page lost, held twice or held by a request that is gone."""
        for group in self.groups:
            group.check()
        code = self.core.lib.hc_check(self.core.pointer)
        if code != 0:
            raise AssertionError(f"page accounting of group {code - 1} is broken")
