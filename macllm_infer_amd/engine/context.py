"""The description of one step's batch, as the kernels read it.

A step runs a list of lanes; a lane is a run of consecutive tokens of one request
starting at that request's current length: a portion of a prompt or one decoded
token.  Lanes are packed without padding in submission order
(reference: src/decoder.rs:4248-4260, lane struct paged_decode.metal:51-58).
All index arrays are built on the host and uploaded in one copy.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable, List, Sequence

import numpy as np
import torch


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
    block_tables: List[torch.Tensor] = field(default_factory=list)   # per group [lanes, max_pages]
    slot_mappings: List[torch.Tensor] = field(default_factory=list)  # per group [T] page*page_size+offset
    lane_lengths: List[int] = field(default_factory=list)            # host copies
    lane_starts: List[int] = field(default_factory=list)
    max_query_len: int = 0
    max_seq_len: int = 0


def build_step_context(lanes: Sequence[Lane], cache, device) -> StepContext:
    """``cache``: the CacheManager, after the step's pages were reserved."""
    lengths = [len(lane.tokens) for lane in lanes]
    starts = [cache.requests[lane.request].length for lane in lanes]
    T = sum(lengths)
    Ln = len(lanes)
    token_ids = np.concatenate([np.asarray(lane.tokens, dtype=np.int32) for lane in lanes])
    positions = np.concatenate([np.arange(start, start + length, dtype=np.int32)
                                for start, length in zip(starts, lengths)])
    lane_of_token = np.repeat(np.arange(Ln, dtype=np.int32), lengths)
    cu = np.zeros(Ln + 1, dtype=np.int32)
    cu[1:] = np.cumsum(lengths)
    start_pos = np.asarray(starts, dtype=np.int32)
    seq_lens = start_pos + np.asarray(lengths, dtype=np.int32)
    slot_ids = np.asarray([cache.requests[lane.request].slot for lane in lanes], dtype=np.int32)
    want_rows = np.asarray([cu[index] + place for index, lane in enumerate(lanes) for place in lane.want],
                           dtype=np.int32)
    sections = [token_ids, positions, lane_of_token, cu, start_pos, seq_lens, slot_ids, want_rows]
    group_shapes = []
    for index, group in enumerate(cache.groups):
        page_size = group.page_size
        tables = [group.tables[lane.request].pages for lane in lanes]
        max_pages = max(1, max(len(pages) for pages in tables))
        table = np.zeros((Ln, max_pages), dtype=np.int32)
        mapping = np.empty(T, dtype=np.int32)
        for row, pages in enumerate(tables):
            pages = np.asarray(pages, dtype=np.int32)
            table[row, :len(pages)] = np.maximum(pages, 0)
            lane_positions = positions[cu[row]:cu[row + 1]]
            mapping[cu[row]:cu[row + 1]] = pages[lane_positions // page_size] * page_size + lane_positions % page_size
        sections += [mapping, table.reshape(-1)]
        group_shapes.append((Ln, max_pages))
    packed = np.concatenate(sections) if sections else np.zeros(0, dtype=np.int32)
    host = torch.from_numpy(packed)
    if torch.device(device).type == "cuda":
        host = host.pin_memory()
    packed_device = host.to(device, non_blocking=True)
    views = []
    offset = 0
    for section in sections:
        views.append(packed_device[offset:offset + section.size])
        offset += section.size
    context = StepContext(
        num_tokens=T, num_lanes=Ln, token_ids=views[0], positions=views[1], lane_of_token=views[2],
        cu_seqlens=views[3], start_pos=views[4], seq_lens=views[5], slot_ids=views[6], want_rows=views[7],
        lane_lengths=lengths, lane_starts=starts, max_query_len=max(lengths),
        max_seq_len=int(seq_lens.max()))
    for index, shape in enumerate(group_shapes):
        context.slot_mappings.append(views[8 + 2 * index])
        context.block_tables.append(views[9 + 2 * index].view(shape))
    context._keepalive = host
    return context
