"""Steps as captured HIP graphs.

A step whose lanes all hold one token is launch-bound: hundreds of small kernels.  For
each batch-size bucket the forward pass over a ``StaticStep`` is captured once and
replayed; only the index arrays are rewritten between replays.  Buckets are powers of
two; missing lanes are padding on the cache's scratch page and slot.  A graph also fixes how
long a context it can hold (the width of its block tables, the runs of keys its attention is
launched for), so graphs come in buckets of context length as well, powers of two from 2,048
tokens up to the longest the cache can hold: a model that allows 262,144 tokens does not pay
for them while its requests are short.

Prompt portions are launch-bound too once the kernels are fast (a portion of 2,048 tokens is
some 700 launches).  A scheduler cuts long prompts into portions of one size, so the shape of
a step (the lengths of its lanes and the places wanted) repeats.  A capture costs as much as some
ten steps' launches, and the last portion of every prompt has a length of its own, so a shape is
captured only at its third sighting among the last 32 steps with portions, and replayed from then
on; a few shapes are kept, the least recently used one goes.
"""
from __future__ import annotations

from collections import OrderedDict, deque
from typing import Dict, Optional, Sequence

import torch

from .context import Lane, LoweredLanes, StaticStep, lower_lanes


def bucket_for(lanes: int) -> int:
    bucket = 1
    while bucket < lanes:
        bucket <<= 1
    return bucket


CONTEXT_BUCKET_FROM = 2048


class DecodeGraphs:
    def __init__(self, model, cache, device, max_seq_len: int):
        self.model = model
        self.cache = cache
        self.device = device
        self.max_seq_len = max_seq_len
        self._graphs: Dict[tuple, tuple] = {}
        self._portion_graphs: "OrderedDict[tuple, tuple]" = OrderedDict()
        self._portion_recent: deque = deque(maxlen=self.PORTION_RECENT)
        self.counts = {"decode_replays": 0, "portion_replays": 0, "portion_captures": 0, "portion_eager": 0}

    PORTION_MIN_TOKENS = 64        # shorter steps are cheap to launch one by one
    PORTION_GRAPHS = 8
    PORTION_RECENT = 32            # steps with portions whose shapes are remembered
    PORTION_SIGHTINGS = 3          # sightings among them before a shape is captured

    def context_bucket(self, lowered: LoweredLanes) -> int:
        """The smallest bucket of context length that holds every lane of the step after it ran."""
        longest = int((self.cache.lengths_of(lowered.slots) + lowered.lengths).max())
        bucket = CONTEXT_BUCKET_FROM
        while bucket < longest:
            bucket <<= 1
        return min(bucket, self.max_seq_len)

    def run_portion(self, lanes: Sequence[Lane], lowered: LoweredLanes) -> Optional[torch.Tensor]:
        """Logits of a step with prompt portions from a captured graph of its shape, or None when
        the shape has no graph (yet): the caller then runs it launch by launch.

        Lanes do not depend on each other, so the shape is taken in a canonical order (longest
        first, then by the places wanted) and the single-token lanes are padded to a power of two:
        a scheduler that rotates its requests, or whose decoding set grows by one, meets the same
        graph again.  The logits come back in the caller's order."""
        if sum(len(lane.tokens) for lane in lanes) < self.PORTION_MIN_TOKENS:
            self.counts["portion_eager"] += 1
            return None
        order = sorted(range(len(lanes)), key=lambda index: (-len(lanes[index].tokens), tuple(lanes[index].want), index))
        ordered = [lanes[index] for index in order]
        singles = sum(1 for lane in ordered if len(lane.tokens) == 1)
        padding = bucket_for(singles) - singles if singles else 0
        # padding lanes stand last, as single tokens whose logits are computed and dropped
        lengths = tuple(len(lane.tokens) for lane in ordered) + (1,) * padding
        wants = tuple(tuple(lane.want) for lane in ordered) + ((0,),) * padding
        context = self.context_bucket(lowered)
        key = (lengths, wants, context)
        entry = self._portion_graphs.get(key)
        if entry is None:
            self._portion_recent.append(key)
            if sum(1 for recent in self._portion_recent if recent == key) < self.PORTION_SIGHTINGS:
                self.counts["portion_eager"] += 1
                return None
            first, rows = 0, []
            for length, want in zip(lengths, wants):
                rows += [first + place for place in want]
                first += length
            static = StaticStep(self.cache, len(lengths), context, self.device, lengths=lengths, want_rows=rows,
                                query_tile=self.model.query_tile)
            entry = self._capture(0, static, warm_runs=1)      # the libraries have seen these sizes already
            self.counts["portion_captures"] += 1
            while len(self._portion_graphs) >= self.PORTION_GRAPHS:
                self._portion_graphs.popitem(last=False)
            self._portion_graphs[key] = entry
        else:
            self._portion_graphs.move_to_end(key)
        static, graph, logits = entry
        static.fill(lowered if order == list(range(len(lanes))) else lower_lanes(ordered, self.cache))
        graph.replay()
        self.counts["portion_replays"] += 1
        if padding == 0 and order == list(range(len(lanes))):
            return logits.clone()
        # rows of the canonical order -> the caller's order
        first_row, starts = 0, {}
        for index, lane in zip(order, ordered):
            starts[index] = first_row
            first_row += len(lane.want)
        rows = [starts[index] + offset for index, lane in enumerate(lanes) for offset in range(len(lane.want))]
        return logits[torch.tensor(rows, dtype=torch.long, device=logits.device)] if rows else logits[:0].clone()

    def _capture(self, bucket: int, static: Optional[StaticStep] = None, warm_runs: int = 2, context: int = 0):
        if static is None:
            static = StaticStep(self.cache, bucket, context or self.max_seq_len, self.device,
                                query_tile=self.model.query_tile)
        # a first run outside the graph lets the libraries set themselves up; every lane is padding,
        # so only the scratch page and slot are touched
        side = torch.cuda.Stream(device=self.device)
        side.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(side):
            for _ in range(warm_runs):
                self.model.forward(static.context, self.cache)
        torch.cuda.current_stream(self.device).wait_stream(side)
        torch.cuda.synchronize(self.device)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = self.model.forward(static.context, self.cache)
        return static, graph, logits

    def run(self, lanes: Sequence[Lane], lowered: LoweredLanes) -> torch.Tensor:
        """Logits [wanted, vocab] of single-token lanes (a copy: the graph's own output tensor is
        overwritten by the next replay)."""
        key = (bucket_for(len(lanes)), self.context_bucket(lowered))
        if key not in self._graphs:
            self._graphs[key] = self._capture(key[0], context=key[1])
        static, graph, logits = self._graphs[key]
        static.fill(lowered)
        graph.replay()
        self.counts["decode_replays"] += 1
        if int(lowered.want_counts.min()) > 0:
            return logits[:len(lanes)].clone()
        rows = [index for index, lane in enumerate(lanes) if len(lane.want) > 0]
        if not rows:
            return logits[:0].clone()
        return logits[torch.tensor(rows, device=logits.device)]
