"""The description of one step's batch, as the kernels read it.

A step runs a list of lanes; a lane is a run of consecutive tokens of one request
starting at that request's current length: a portion of a prompt or one decoded
token.  Lanes are packed without padding in submission order
(reference: src/decoder.rs:4248-4260, lane struct paged_decode.metal:51-58).
All index arrays are written by the host-side core (``csrc/hostcore.cpp``) into one buffer and
uploaded in one copy; tables that a mixer declares for itself (``StepTable``) are written behind them
by the mixer's own function and travel in the same copy.

``StaticStep`` keeps the arrays of a batch of single-token lanes at fixed addresses and
fixed shapes, so that a captured HIP graph can be replayed on them; lanes beyond the
batch's real ones are padding that reads and writes the cache's scratch page and slot.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from itertools import chain
from typing import Callable, Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache import native
from ..kernels import ops


NO_TILES = 1 << 30     # the table of runs then has one run per lane: no mixer of the model reads it


@dataclass
class Lane:
    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()         # places among ``tokens`` whose logits are asked for
    # (int32 tensor on the device, row): the lane's one token is not known to the host yet; it is that element
    # of the tensor (what a sampler left there for the step before) and ``tokens`` holds any valid id in its place
    feed: Optional[tuple] = None


@dataclass
class StepContext:
    num_tokens: int
    num_lanes: int
    token_ids: torch.Tensor          # [T] int32
    positions: torch.Tensor          # [T] absolute position of each token in its request
    lane_of_token: torch.Tensor      # [T]
    cu_seqlens: torch.Tensor         # [lanes+1] first token of each lane
    start_pos: torch.Tensor          # [lanes] request length before the step
    seq_lens: torch.Tensor           # [lanes] request length after the step
    slot_ids: torch.Tensor           # [lanes] state slot of each lane's request
    want_rows: torch.Tensor          # [wanted] token rows whose logits are returned
    query_tiles: torch.Tensor        # [tiles, 2] (lane, first token row) of runs of up to ``query_tile`` tokens of one lane
    query_tile: int = 0              # the longest run of that table (0: one run a lane, whatever its length)
    block_tables: List[torch.Tensor] = field(default_factory=list)   # per group [lanes, max_pages]
    slot_mappings: List[torch.Tensor] = field(default_factory=list)  # per group [T] page*page_size+offset
    lane_lengths: Optional[List[int]] = field(default_factory=list)   # host copies; None in a step of fixed capacity
    lane_starts: Optional[List[int]] = field(default_factory=list)
    max_query_len: int = 0           # the longest lane (its upper bound in a step of fixed capacity)
    max_seq_len: int = 0             # an upper bound of the longest context in the batch
    derived: dict = field(default_factory=dict)   # tables parts derive from the step, shared by the layers
    chunk_tables: dict = field(default_factory=dict)   # chunk size -> ChunkTable, for the sizes the model's mixers name
    tables: dict = field(default_factory=dict)         # name -> int32 tensor, for the tables the model's mixers declare


@dataclass
class LoweredLanes:
    """A step's lanes as the arrays the host-side core reads."""
    slots: np.ndarray            # [lanes] the requests' handles in the core (their state slots)
    lengths: np.ndarray          # [lanes] tokens of each lane
    tokens: np.ndarray           # [T] all lanes' tokens, lane after lane
    want_counts: np.ndarray      # [lanes] wanted places of each lane
    wants: np.ndarray            # [wanted] the places, lane after lane
    feeds: tuple = ()            # (token row, int32 tensor on the device, its row) of tokens the host does not know yet


def lower_lanes(lanes: Sequence[Lane], cache) -> LoweredLanes:
    """KeyError for a request that is not live, OverflowError / ValueError / TypeError for a token
    or place that is no 32-bit integer."""
    count = len(lanes)
    slots = cache.slots_of([lane.request for lane in lanes])
    lengths = np.fromiter((len(lane.tokens) for lane in lanes), dtype=np.int32, count=count)
    want_counts = np.fromiter((len(lane.want) for lane in lanes), dtype=np.int32, count=count)
    tokens = np.fromiter(chain.from_iterable(lane.tokens for lane in lanes), dtype=np.int64, count=int(lengths.sum()))
    wants = np.fromiter(chain.from_iterable(lane.want for lane in lanes), dtype=np.int64, count=int(want_counts.sum()))
    if tokens.size and (tokens.min() < -(1 << 31) or tokens.max() >= (1 << 31)):
        raise OverflowError("a token id does not fit 32 bits")
    if wants.size and (wants.min() < -(1 << 31) or wants.max() >= (1 << 31)):
        raise OverflowError("a wanted place does not fit 32 bits")
    return LoweredLanes(slots, lengths, tokens.astype(np.int32), want_counts, wants.astype(np.int32))


def apply_feeds(token_ids: torch.Tensor, feeds) -> None:
    """Write the tokens that are still on the device into the step's token ids (after their upload, before the
    forward pass or the graph's replay, on the same stream)."""
    if not feeds:
        return
    by_source = {}
    for row, source, index in feeds:
        by_source.setdefault(id(source), (source, [], []))
        by_source[id(source)][1].append(row)
        by_source[id(source)][2].append(index)
    for source, rows, indices in by_source.values():
        ops.feed_tokens(token_ids, source, rows, indices)


@dataclass(frozen=True)
class StepTable:
    """An int32 table of a step that a mixer declares (``Mixer.step_tables``) and finds, on the device, in
    ``step.tables[name]``: written on the host with the step's other index arrays, uploaded in the same copy,
    and at a fixed address and of a fixed size in a step that a captured graph reads.

    ``words(lanes, tokens)``: the table's size for a step of that many lanes and tokens, and never smaller for
    fewer of either: a step of fixed capacity holds the table of its capacity.
    ``fill(out, packed)``: writes all of ``out`` (int32 [words], zeros before) from ``packed``, a
    ``PackedLanes`` of every lane of the step, padding lanes included."""
    name: str
    words: Callable[[int, int], int]
    fill: Callable[[np.ndarray, "PackedLanes"], None]


@dataclass
class PackedLanes:
    """The lanes of a packed step as the host sees them (views of the buffer that is uploaded): what the fill
    function of a ``StepTable`` reads.  Padding lanes of a captured step stand at the end, on ``scratch_slot``."""
    num_lanes: int
    num_tokens: int
    positions: np.ndarray        # [T] absolute position of each token row
    lane_of_token: np.ndarray    # [T]
    first_token: np.ndarray      # [lanes + 1] first token row of each lane
    start_pos: np.ndarray        # [lanes] request length before the step
    seq_lens: np.ndarray         # [lanes] request length after the step
    slot_ids: np.ndarray         # [lanes] state slot of each lane's request
    scratch_slot: int            # the state slot that padding lanes read and write


def _fill_tables(tables: Sequence[StepTable], host: np.ndarray, sizes, table_sizes, cache) -> None:
    """Write the declared tables behind the core's sections of ``host`` (whose sizes are ``sizes``)."""
    if not tables:
        return
    views = _split(host, sizes)
    lanes = views[4].size
    packed = PackedLanes(lanes, views[0].size, views[1], views[2], views[3], views[4], views[5], views[6],
                         int(cache.scratch_slot))
    offset = int(sum(sizes))
    for table, size in zip(tables, table_sizes):
        out = host[offset:offset + size]
        out[:] = 0
        table.fill(out, packed)
        offset += size


def _table_sizes(tables: Sequence[StepTable], lanes: int, tokens: int) -> List[int]:
    sizes = []
    for table in tables:
        size = int(table.words(lanes, tokens))
        if size < 0:
            raise ValueError(f"the step table {table.name!r} declares a negative size")
        sizes.append(size)
    return sizes


_NO_LANES = LoweredLanes(*(np.zeros(0, dtype=np.int32) for _ in range(5)))


@dataclass
class ChunkTable:
    """Every lane of a step cut from its first token into chunks of ``chunk_size`` tokens (the last one of a
    lane may be short).  ``chunks`` int32 [num_chunks, 4] = (lane, first token row, tokens, index within the
    lane); ``lane_chunks`` int32 [lanes, 2] = (first chunk, number of chunks).  In a step of fixed capacity
    ``num_chunks`` is the table's capacity: rows past the step's own chunks hold lane -1 and no tokens."""
    chunk_size: int
    num_tokens: int
    num_lanes: int
    num_chunks: int
    chunks: torch.Tensor
    lane_chunks: torch.Tensor


def _pack(lowered: LoweredLanes, cache, out: Optional[np.ndarray], pad_lengths: Sequence[int] = (),
          max_pages: Optional[int] = None, want_rows: Optional[np.ndarray] = None, query_tile: int = 0,
          chunk_sizes: Sequence[int] = (), tiles_cap: int = 0, wants_cap: int = 0, chunks_cap: Sequence[int] = ()):
    """The core writes the step's sections (in the order of ``_assemble``) into ``out``.  Returns
    (words written or, negated, words needed when ``out`` is too small or None; section sizes;
    block-table shapes; longest context after the step; the step's own chunks per chunk size).
    ``pad_lengths``: lanes appended on the scratch page and slot.  ``want_rows`` replaces the lanes' own
    wanted rows.  ``query_tile``: the longest run of one lane's tokens in the table of runs (what the
    model's mixers ask for; 0: none does).  ``chunk_sizes``: the chunk tables the model's mixers ask for.
    ``tiles_cap``, ``wants_cap``, ``chunks_cap``: fixed sizes of the sections that depend on how the tokens
    fall into lanes (a step of fixed capacity); ValueError when the step does not fit them."""
    core = cache.core
    pads = native.as_ints(list(pad_lengths))
    groups = len(cache.groups)
    kinds = len(chunk_sizes)
    meta = np.zeros(9 + 3 * groups + 3 * kinds + 1, dtype=np.int32)
    fixed = native.as_ints(want_rows) if want_rows is not None else None
    sizes_in = native.as_ints(list(chunk_sizes))
    caps_in = native.as_ints(list(chunks_cap) if len(chunks_cap) else [0] * kinds)
    written = core.lib.hc_pack(
        core.pointer, len(lowered.slots), native.int_pointer(lowered.slots), native.int_pointer(lowered.lengths),
        native.int_pointer(lowered.tokens), native.int_pointer(lowered.want_counts), native.int_pointer(lowered.wants),
        len(pads), native.int_pointer(pads), max_pages or 0, query_tile or NO_TILES,
        native.int_pointer(fixed) if fixed is not None else None, len(fixed) if fixed is not None else 0,
        int(tiles_cap), int(wants_cap), kinds, native.int_pointer(sizes_in), native.int_pointer(caps_in),
        native.int_pointer(out) if out is not None else None, out.size if out is not None else 0,
        native.int_pointer(meta))
    if written == -1:
        raise ValueError("the step cannot be packed: a request is not live, a wanted place lies outside its "
                         "lane, or the step's pages were not reserved")
    if written == -2:
        raise ValueError("the step does not fit the fixed capacity it is packed for")
    if written < 0:
        written += 2                                     # -(words needed) - 2
    lanes = len(lowered.slots) + len(pads)
    count = 9 + 2 * groups + 2 * kinds
    sizes = meta[:count].tolist()
    shapes = [(lanes, int(width)) for width in meta[count:count + groups]]
    return int(written), sizes, shapes, int(meta[count + groups]), meta[count + groups + 1:count + groups + 1 + kinds].tolist()


def _assemble(views, group_shapes, lengths, starts, max_seq_len, chunk_sizes=(), num_tokens=None, num_lanes=None,
              max_query_len=None, query_tile: int = 0, tables: Sequence[StepTable] = ()) -> StepContext:
    """``lengths`` / ``starts``: the lanes' host copies, or None for a step of fixed capacity, whose lanes
    differ from fill to fill (``num_tokens``, ``num_lanes`` and ``max_query_len`` are then its capacities)."""
    tokens = sum(lengths) if lengths is not None else num_tokens
    lanes = len(lengths) if lengths is not None else num_lanes
    context = StepContext(
        num_tokens=tokens, num_lanes=lanes, token_ids=views[0], positions=views[1],
        lane_of_token=views[2], cu_seqlens=views[3], start_pos=views[4], seq_lens=views[5], slot_ids=views[6],
        want_rows=views[7], query_tiles=views[8].view(-1, 2), query_tile=int(query_tile or 0),
        lane_lengths=list(lengths) if lengths is not None else None,
        lane_starts=list(starts) if starts is not None else None,
        max_query_len=max(lengths) if lengths is not None else max_query_len, max_seq_len=max_seq_len)
    groups = len(group_shapes)
    for index, shape in enumerate(group_shapes):
        context.slot_mappings.append(views[9 + 2 * index])
        context.block_tables.append(views[10 + 2 * index].view(shape))
    for index, chunk_size in enumerate(chunk_sizes):
        chunks, lane_chunks = views[9 + 2 * groups + 2 * index], views[10 + 2 * groups + 2 * index]
        context.chunk_tables[chunk_size] = ChunkTable(chunk_size, tokens, lanes, chunks.numel() // 4, chunks, lane_chunks)
    first = 9 + 2 * groups + 2 * len(chunk_sizes)
    for index, table in enumerate(tables):                 # the declared tables lie behind the core's sections
        context.tables[table.name] = views[first + index]
    return context


def _split(buffer: torch.Tensor, sizes):
    views, offset = [], 0
    for size in sizes:
        views.append(buffer[offset:offset + size])
        offset += size
    return views


def build_step_context(lanes: Sequence[Lane], cache, device, lowered: Optional[LoweredLanes] = None,
                       query_tile: int = 0, chunk_sizes: Sequence[int] = (),
                       tables: Sequence[StepTable] = ()) -> StepContext:
    """``cache``: the CacheManager, after the step's pages were reserved.  ``query_tile``, ``chunk_sizes``:
    see ``_pack``; ``tables``: the tables the model's mixers declare (``DecoderModel.step_layout`` holds all
    three for a whole model)."""
    if lowered is None:
        lowered = lower_lanes(lanes, cache)
    needed, _, _, _, _ = _pack(lowered, cache, None, query_tile=query_tile, chunk_sizes=chunk_sizes)
    table_sizes = _table_sizes(tables, len(lowered.slots), int(lowered.lengths.sum()))
    host = torch.empty(-needed + sum(table_sizes), dtype=torch.int32)
    if torch.device(device).type == "cuda":
        host = host.pin_memory()
    _, sizes, shapes, longest, _ = _pack(lowered, cache, host.numpy(), query_tile=query_tile, chunk_sizes=chunk_sizes)
    _fill_tables(tables, host.numpy(), sizes, table_sizes, cache)
    packed = host.to(device, non_blocking=True)
    starts = cache.lengths_of(lowered.slots).tolist()
    context = _assemble(_split(packed, sizes + table_sizes), shapes, lowered.lengths.tolist(), starts, longest,
                        chunk_sizes, query_tile=query_tile, tables=tables)
    context._keepalive = host
    return context


class StaticStep:
    """The arrays of a step at fixed device addresses and of fixed sizes, which a captured graph reads:

    * ``lanes`` single-token lanes whose logits are all wanted (a decode step), or lanes of ``lengths`` tokens
      with the wanted rows ``want_rows``; or
    * with ``tokens``: a step of fixed *capacity*: up to ``lanes`` lanes that hold ``tokens`` tokens together,
      whatever their lengths, and up to ``wants`` wanted rows.  The tables that depend on how the tokens fall
      into lanes (runs of a lane's tokens, chunks) have the size of the worst case and are rewritten with the
      rest; what the step's own lanes leave of the capacity is padding lanes on the cache's scratch page and
      slot, the first ones of one token and the last one with the remainder.

    ``fill`` rewrites the arrays for the real lanes of a step."""

    def __init__(self, cache, lanes: int, max_seq_len: int, device, lengths: Sequence[int] = (),
                 want_rows: Sequence[int] = (), query_tile: int = 0, chunk_sizes: Sequence[int] = (),
                 tokens: int = 0, wants: int = 0, tables: Sequence[StepTable] = ()):
        self.cache = cache
        self.query_tile = query_tile
        self.chunk_sizes = tuple(chunk_sizes)
        self.tables = tuple(tables)
        self.lanes = lanes
        self.tokens = tokens
        self.max_pages = max(-(-max_seq_len // group.page_size) for group in cache.groups) if cache.groups else 1
        self.capacity = tokens > 0
        if self.capacity:
            if tokens < lanes or wants <= 0:
                raise ValueError("a step of fixed capacity holds at least one token a lane and wants a row")
            self.lengths = None
            self.want_rows = None
            tile = query_tile or NO_TILES
            self.caps = dict(tiles_cap=-(-tokens // tile) + lanes, wants_cap=wants,
                             chunks_cap=[-(-tokens // size) + lanes for size in self.chunk_sizes])
            first_pads = self._pads(0, 0)
        else:
            self.lengths = list(lengths) if lengths else [1] * lanes
            self.want_rows = (np.asarray(want_rows, dtype=np.int32) if lengths
                              else np.arange(lanes, dtype=np.int32))             # every lane's row is wanted
            self.caps = {}
            first_pads = self.lengths
        pack = dict(max_pages=self.max_pages, want_rows=self.want_rows, query_tile=query_tile,
                    chunk_sizes=self.chunk_sizes, **self.caps)
        needed, sizes, shapes, _, _ = _pack(_NO_LANES, cache, None, first_pads, **pack)
        # the declared tables, at the size of this step's capacity, behind the core's sections
        self._core_sizes = sizes
        self._table_sizes = _table_sizes(self.tables, lanes, tokens if self.capacity else sum(self.lengths))
        needed -= sum(self._table_sizes)
        sizes = sizes + self._table_sizes
        # The host packs a step into pinned memory and queues its copy to the fixed device addresses; the
        # copy runs when the stream gets there, so the memory it reads must stay as it is until then.  A few
        # host buffers are filled in turn, each guarded by an event recorded behind its copy: the host may
        # run that many steps ahead of the GPU and no further.
        on_gpu = torch.device(device).type == "cuda"
        self._hosts = []
        for _ in range(self.HOST_BUFFERS):
            host = torch.empty(-needed, dtype=torch.int32)
            self._hosts.append(host.pin_memory() if on_gpu else host)
        self._copied = [torch.cuda.Event() if on_gpu else None for _ in self._hosts]
        self._pending = [False] * len(self._hosts)
        self._turn = 0
        self.device_buffer = torch.empty(-needed, dtype=torch.int32, device=device)
        _pack(_NO_LANES, cache, self._hosts[0].numpy(), first_pads, **pack)
        _fill_tables(self.tables, self._hosts[0].numpy(), self._core_sizes, self._table_sizes, cache)
        self.device_buffer.copy_(self._hosts[0])
        if self.capacity:
            self.context = _assemble(_split(self.device_buffer, sizes), shapes, None, None, max_seq_len,
                                     self.chunk_sizes, num_tokens=tokens, num_lanes=lanes, max_query_len=tokens,
                                     query_tile=query_tile, tables=self.tables)
        else:
            self.context = _assemble(_split(self.device_buffer, sizes), shapes, self.lengths, [0] * lanes, max_seq_len,
                                     self.chunk_sizes, query_tile=query_tile, tables=self.tables)

    HOST_BUFFERS = 2

    def _pads(self, real_lanes: int, real_tokens: int) -> List[int]:
        """The padding lanes of a step of fixed capacity beside ``real_lanes`` lanes of ``real_tokens`` tokens."""
        pads, rest = self.lanes - real_lanes, self.tokens - real_tokens
        if pads < 0 or rest < pads or (pads == 0 and rest != 0):
            raise ValueError(f"{real_lanes} lanes of {real_tokens} tokens do not fit a step of {self.lanes} lanes and "
                             f"{self.tokens} tokens")
        return [1] * (pads - 1) + [rest - (pads - 1)] if pads else []

    @staticmethod
    def fits(lanes_cap: int, tokens_cap: int, lanes: int, tokens: int) -> bool:
        """Whether a step of ``lanes`` lanes and ``tokens`` tokens can be padded to the capacity."""
        pads, rest = lanes_cap - lanes, tokens_cap - tokens
        return pads >= 0 and ((pads == 0 and rest == 0) or (pads > 0 and rest >= pads))

    def fill(self, lowered: LoweredLanes) -> None:
        """``lowered``: the real lanes (a step of fixed lanes: their lengths are the first of this step's; the
        rest is padding)."""
        real = len(lowered.slots)
        if self.capacity:
            pads = self._pads(real, int(lowered.lengths.sum()))
        else:
            pads = self.lengths[real:]
        turn = self._turn
        self._turn = (turn + 1) % len(self._hosts)
        if self._pending[turn]:
            self._copied[turn].synchronize()          # the copy that last read this buffer has run
        host = self._hosts[turn]
        _pack(lowered, self.cache, host.numpy(), pads, max_pages=self.max_pages, want_rows=self.want_rows,
              query_tile=self.query_tile, chunk_sizes=self.chunk_sizes, **self.caps)
        _fill_tables(self.tables, host.numpy(), self._core_sizes, self._table_sizes, self.cache)
        self.device_buffer.copy_(host, non_blocking=True)
        if self._copied[turn] is not None:
            self._copied[turn].record()
            self._pending[turn] = True
