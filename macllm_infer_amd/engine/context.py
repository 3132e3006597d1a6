"""The description of one step's batch, as the kernels read it.

A step runs a list of lanes; a lane is a run of consecutive tokens of one request
starting at that request's current length: a portion of a prompt or one decoded
token.  Lanes are packed without padding in submission order
(reference: src/decoder.rs:4248-4260, lane struct paged_decode.metal:51-58).
All index arrays are built on the host and uploaded in one copy.

``StaticStep`` keeps the arrays of a batch of single-token lanes at fixed addresses and
fixed shapes, so that a captured HIP graph can be replayed on them; lanes beyond the
batch's real ones are padding that reads and writes the cache's scratch page and slot.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable, List, Optional, Sequence

import numpy as np
import torch


QUERY_TILE = 64        # tokens of one lane that one workgroup of the prefill attention kernel takes


@dataclass
class Lane:
    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()         # places among ``tokens`` whose logits are asked for


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
    query_tiles: torch.Tensor        # [tiles, 2] (lane, first token row) of runs of up to 64 tokens of one lane
    block_tables: List[torch.Tensor] = field(default_factory=list)   # per group [lanes, max_pages]
    slot_mappings: List[torch.Tensor] = field(default_factory=list)  # per group [T] page*page_size+offset
    lane_lengths: List[int] = field(default_factory=list)            # host copies
    lane_starts: List[int] = field(default_factory=list)
    max_query_len: int = 0
    max_seq_len: int = 0             # an upper bound of the longest context in the batch
    derived: dict = field(default_factory=dict)   # tables parts derive from the step, shared by the layers


def _pack(lanes: Sequence[Lane], cache, pad_lanes: int = 0, max_pages: Optional[int] = None,
          pad_lengths: Sequence[int] = ()):
    """Numpy sections of the step (in the order of ``_assemble``) and the block-table shapes.
    ``pad_lanes`` single-token lanes on the scratch page and slot are appended (or lanes of
    ``pad_lengths`` tokens, all of them on the scratch page)."""
    pad_lengths = list(pad_lengths) if pad_lengths else [1] * pad_lanes
    pad_lanes = len(pad_lengths)
    lengths = [len(lane.tokens) for lane in lanes] + pad_lengths
    starts = [cache.requests[lane.request].length for lane in lanes] + [0] * pad_lanes
    Ln = len(lengths)
    T = sum(lengths)
    token_ids = np.concatenate([np.asarray(lane.tokens, dtype=np.int32) for lane in lanes]
                               + [np.zeros(sum(pad_lengths), dtype=np.int32)])
    positions = np.concatenate([np.arange(start, start + length, dtype=np.int32)
                                for start, length in zip(starts, lengths)])
    lane_of_token = np.repeat(np.arange(Ln, dtype=np.int32), lengths)
    cu = np.zeros(Ln + 1, dtype=np.int32)
    cu[1:] = np.cumsum(lengths)
    start_pos = np.asarray(starts, dtype=np.int32)
    seq_lens = start_pos + np.asarray(lengths, dtype=np.int32)
    slot_ids = np.asarray([cache.requests[lane.request].slot for lane in lanes]
                          + [cache.scratch_slot] * pad_lanes, dtype=np.int32)
    want_rows = np.asarray([cu[index] + place for index, lane in enumerate(lanes) for place in lane.want],
                           dtype=np.int32)
    tiles = np.asarray([(index, row) for index in range(Ln) for row in range(cu[index], cu[index + 1], QUERY_TILE)],
                       dtype=np.int32).reshape(-1)
    sections = [token_ids, positions, lane_of_token, cu, start_pos, seq_lens, slot_ids, want_rows, tiles]
    group_shapes = []
    for group in cache.groups:
        page_size = group.page_size
        tables = ([group.tables[lane.request].pages for lane in lanes]
                  + [[group.scratch_page] * -(-length // page_size) for length in pad_lengths])
        width = max_pages if max_pages is not None else max(1, max(len(pages) for pages in tables))
        table = np.zeros((Ln, width), dtype=np.int32)
        mapping = np.empty(T, dtype=np.int32)
        for row, pages in enumerate(tables):
            pages = np.asarray(pages, dtype=np.int32)
            table[row, :len(pages)] = np.maximum(pages, 0)
            lane_positions = positions[cu[row]:cu[row + 1]]
            mapping[cu[row]:cu[row + 1]] = pages[lane_positions // page_size] * page_size + lane_positions % page_size
        sections += [mapping, table.reshape(-1)]
        group_shapes.append((Ln, width))
    return sections, group_shapes, lengths, starts


def _assemble(views, group_shapes, lengths, starts, max_seq_len) -> StepContext:
    context = StepContext(
        num_tokens=sum(lengths), num_lanes=len(lengths), token_ids=views[0], positions=views[1],
        lane_of_token=views[2], cu_seqlens=views[3], start_pos=views[4], seq_lens=views[5], slot_ids=views[6],
        want_rows=views[7], query_tiles=views[8].view(-1, 2), lane_lengths=list(lengths), lane_starts=list(starts), max_query_len=max(lengths),
        max_seq_len=max_seq_len)
    for index, shape in enumerate(group_shapes):
        context.slot_mappings.append(views[9 + 2 * index])
        context.block_tables.append(views[10 + 2 * index].view(shape))
    return context


def _split(buffer: torch.Tensor, sections):
    views, offset = [], 0
    for section in sections:
        views.append(buffer[offset:offset + section.size])
        offset += section.size
    return views


def build_step_context(lanes: Sequence[Lane], cache, device) -> StepContext:
    """``cache``: the CacheManager, after the step's pages were reserved."""
    sections, group_shapes, lengths, starts = _pack(lanes, cache)
    host = torch.from_numpy(np.concatenate(sections))
    if torch.device(device).type == "cuda":
        host = host.pin_memory()
    packed = host.to(device, non_blocking=True)
    context = _assemble(_split(packed, sections), group_shapes, lengths, starts,
                        max(start + length for start, length in zip(starts, lengths)))
    context._keepalive = host
    return context


class StaticStep:
    """The arrays of a step of fixed shape at fixed device addresses: ``lanes`` single-token lanes
    whose logits are all wanted, or lanes of ``lengths`` tokens with the wanted rows ``want_rows``.
    ``fill`` rewrites them for the real lanes of a step of that shape."""

    def __init__(self, cache, lanes: int, max_seq_len: int, device, lengths: Sequence[int] = (),
                 want_rows: Sequence[int] = ()):
        self.cache = cache
        self.lanes = lanes
        self.lengths = list(lengths)
        self.max_pages = max(-(-max_seq_len // group.page_size) for group in cache.groups) if cache.groups else 1
        self.want_rows = (np.asarray(want_rows, dtype=np.int32) if self.lengths
                          else np.arange(lanes, dtype=np.int32))             # every lane's row is wanted
        sections, group_shapes, lengths, starts = _pack([], cache, pad_lanes=lanes, max_pages=self.max_pages,
                                                        pad_lengths=self.lengths)
        sections[7] = self.want_rows
        total = sum(section.size for section in sections)
        self.host = torch.empty(total, dtype=torch.int32).pin_memory()
        self.device_buffer = torch.empty(total, dtype=torch.int32, device=device)
        self.host.copy_(torch.from_numpy(np.concatenate(sections)))
        self.device_buffer.copy_(self.host)
        self.context = _assemble(_split(self.device_buffer, sections), group_shapes, lengths, starts, max_seq_len)

    def fill(self, lanes: Sequence[Lane]) -> None:
        sections, _, _, _ = _pack(lanes, self.cache, pad_lanes=self.lanes - len(lanes), max_pages=self.max_pages)
        sections[7] = self.want_rows
        self.host.copy_(torch.from_numpy(np.concatenate(sections)))
        self.device_buffer.copy_(self.host, non_blocking=True)
