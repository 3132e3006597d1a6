"""Steps as captured HIP graphs.

A step whose lanes all hold one token is launch-bound: hundreds of small kernels.  For
each batch-size bucket the forward pass over a ``StaticStep`` is captured once and
replayed; only the index arrays are rewritten between replays.  Buckets are powers of
two; missing lanes are padding on the cache's scratch page and slot.

Prompt portions are launch-bound too once the kernels are fast (a portion of 2,048 tokens is
some 700 launches).  A scheduler cuts long prompts into portions of one size, so the shape of
a step (the lengths of its lanes and the places wanted) repeats: a shape seen a second time is
captured and replayed from then on; a few shapes are kept, the least recently used one goes.
"""
from __future__ import annotations

from collections import OrderedDict
from typing import Dict, Optional, Sequence

import torch

from .context import Lane, StaticStep


def bucket_for(lanes: int) -> int:
    bucket = 1
    while bucket < lanes:
        bucket <<= 1
    return bucket


class DecodeGraphs:
    def __init__(self, model, cache, device, max_seq_len: int):
        self.model = model
        self.cache = cache
        self.device = device
        self.max_seq_len = max_seq_len
        self._graphs: Dict[int, tuple] = {}
        self._portion_graphs: "OrderedDict[tuple, tuple]" = OrderedDict()
        self._portion_seen: Dict[tuple, int] = {}

    PORTION_MIN_TOKENS = 64        # shorter steps are cheap to launch one by one
    PORTION_GRAPHS = 4

    def run_portion(self, lanes: Sequence[Lane]) -> Optional[torch.Tensor]:
        """Logits of a step with prompt portions from a captured graph of its shape, or None when
        the shape has no graph (yet): the caller then runs it launch by launch."""
        lengths = tuple(len(lane.tokens) for lane in lanes)
        if sum(lengths) < self.PORTION_MIN_TOKENS:
            return None
        key = (lengths, tuple(tuple(lane.want) for lane in lanes))
        entry = self._portion_graphs.get(key)
        if entry is None:
            seen = self._portion_seen.get(key, 0) + 1
            self._portion_seen[key] = seen
            if seen < 2:
                if len(self._portion_seen) > 1024:
                    self._portion_seen.clear()
                return None
            first, rows = 0, []
            for lane in lanes:
                rows += [first + place for place in lane.want]
                first += len(lane.tokens)
            static = StaticStep(self.cache, len(lanes), self.max_seq_len, self.device, lengths=lengths, want_rows=rows)
            entry = self._capture(0, static)
            while len(self._portion_graphs) >= self.PORTION_GRAPHS:
                self._portion_graphs.popitem(last=False)
            self._portion_graphs[key] = entry
        else:
            self._portion_graphs.move_to_end(key)
        static, graph, logits = entry
        static.fill(lanes)
        graph.replay()
        return logits.clone()

    def _capture(self, bucket: int, static: Optional[StaticStep] = None):
        if static is None:
            static = StaticStep(self.cache, bucket, self.max_seq_len, self.device)
        # a first run outside the graph lets the libraries set themselves up; every lane is padding,
        # so only the scratch page and slot are touched
        side = torch.cuda.Stream(device=self.device)
        side.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(side):
            for _ in range(2):
                self.model.forward(static.context, self.cache)
        torch.cuda.current_stream(self.device).wait_stream(side)
        torch.cuda.synchronize(self.device)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = self.model.forward(static.context, self.cache)
        return static, graph, logits

    def run(self, lanes: Sequence[Lane]) -> torch.Tensor:
        """Logits [wanted, vocab] of single-token lanes (a copy: the graph's own output tensor is
        overwritten by the next replay)."""
        bucket = bucket_for(len(lanes))
        if bucket not in self._graphs:
            self._graphs[bucket] = self._capture(bucket)
        static, graph, logits = self._graphs[bucket]
        static.fill(lanes)
        graph.replay()
        rows = [index for index, lane in enumerate(lanes) if len(lane.want) > 0]
        if len(rows) == len(lanes):
            return logits[:len(lanes)].clone()
        if not rows:
            return logits[:0].clone()
        return logits[torch.tensor(rows, device=logits.device)]
