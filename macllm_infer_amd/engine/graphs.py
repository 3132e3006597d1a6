"""Decode steps as captured HIP graphs.

A step whose lanes all hold one token is launch-bound: hundreds of small kernels.  For
each batch-size bucket the forward pass over a ``StaticStep`` is captured once and
replayed; only the index arrays are rewritten between replays.  Buckets are powers of
two; missing lanes are padding on the cache's scratch page and slot.
"""
from __future__ import annotations

from typing import Dict, Sequence

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

    def _capture(self, bucket: int):
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
