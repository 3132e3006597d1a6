"""Steps as captured HIP graphs.

A step whose lanes all hold one token is launch-bound: hundreds of small kernels.  For
each batch-size bucket the forward pass over a ``StaticStep`` is captured once and
replayed; only the index arrays are rewritten between replays.  Buckets are powers of
two; missing lanes are padding on the cache's scratch page and slot.  A graph also fixes how
long a context it can hold (the width of its block tables, the runs of keys its attention is
launched for), so graphs come in buckets of context length as well, powers of two from 2,048
tokens up to the longest the cache can hold: a model that allows 262,144 tokens does not pay
for them while its requests are short.

Steps with prompt portions are launch-bound too once the kernels are fast (a portion of 2,048 tokens is
some 470 launches: launched one by one, the host needs 5 ms for them whatever their length).  Their
graphs are made for a *capacity*, not for a shape: so many tokens in so many lanes with so many wanted
rows, whatever the lanes' lengths.  Every kernel reads where a lane begins and ends from the step's
arrays on the device, and the tables that depend on it (runs of a lane's tokens for the attention
kernel, chunks for the scan) have the size of the worst case; what a step leaves of the capacity is
padding lanes on the scratch page and slot.  A handful of capacities (token counts in steps of a quarter
to a third, lane counts in powers of two) therefore serves every step a scheduler can make, a capacity is
captured when it comes the second time (a single prompt is not worth a capture, which costs two passes of
launches), and ``warm_up`` captures a list of them before the first request.
"""
from __future__ import annotations

from collections import OrderedDict
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import torch

from .context import Lane, LoweredLanes, StaticStep, apply_feeds


def bucket_for(lanes: int) -> int:
    bucket = 1
    while bucket < lanes:
        bucket <<= 1
    return bucket


CONTEXT_BUCKET_FROM = 2048


def token_capacities(most: int) -> List[int]:
    """The token counts that steps with prompt portions are padded to: 16, 32, 48, 64, then steps of a
    quarter of the power of two below (80, 96, 112, 128, 160, ...) and, from 1,024 on, of an eighth (1,152,
    1,280, ...: a scheduler's portion of 2,048 tokens beside a few decoded ones pads to 2,304), up to the first
    one that holds ``most``."""
    out, value = [], 16
    while True:
        out.append(value)
        if value >= most:
            return out
        power = 1 << (value.bit_length() - 1)
        value += max(16, power // (8 if value >= 1024 else 4))


class DecodeGraphs:
    def __init__(self, model, cache, device, max_seq_len: int):
        self.model = model
        self.cache = cache
        self.device = device
        self.max_seq_len = max_seq_len
        self._graphs: Dict[tuple, tuple] = {}
        self._bucket_graphs: "OrderedDict[tuple, tuple]" = OrderedDict()
        self._seen: "OrderedDict[tuple, int]" = OrderedDict()
        self._pool = None
        self.counts = {"decode_replays": 0, "bucket_replays": 0, "bucket_captures": 0, "bucket_eager": 0}

    # captured capacities kept; the least recently used one goes.  A capture costs about as much as thirty replays
    # save, so the graphs of a workload must all fit: 150 requests of 16 to 1,200 prompt tokens through the
    # scheduler meet 31 capacities (portions that end a prompt have any length), and with room for 24 every run
    # of them captured a dozen again (1.06 s a run instead of 0.78).  The graphs share one memory pool: more of them
    # cost their index arrays and nodes, not activations.
    BUCKET_GRAPHS = 96
    BUCKET_SIGHTINGS = 2           # sightings of a capacity before it is captured
    BUCKET_MOST_TOKENS = 16384     # steps beyond this many tokens are launched kernel by kernel

    def context_bucket(self, lowered: LoweredLanes, at_least: int = 0) -> int:
        """The smallest bucket of context length that holds every lane of the step after it ran."""
        longest = max(int((self.cache.lengths_of(lowered.slots) + lowered.lengths).max()), at_least)
        bucket = CONTEXT_BUCKET_FROM
        while bucket < longest:
            bucket <<= 1
        return min(bucket, self.max_seq_len)

    def capacity_for(self, lanes: int, tokens: int, wants: int) -> Optional[Tuple[int, int, int]]:
        """(lanes, tokens, wanted rows) of the smallest capacity that holds such a step, or None."""
        if tokens > self.BUCKET_MOST_TOKENS:
            return None
        lane_cap = bucket_for(lanes)
        for _ in range(2):                                   # the lanes' own bucket, or the next one (room for padding lanes)
            for token_cap in token_capacities(self.BUCKET_MOST_TOKENS):
                if token_cap >= tokens and StaticStep.fits(lane_cap, token_cap, lanes, tokens):
                    return lane_cap, token_cap, lane_cap if wants <= lane_cap else token_cap
            lane_cap <<= 1
        return None

    def token_target(self, lanes: int, tokens: int) -> int:
        """For a scheduler that is free to cut a prompt portion shorter: the largest number of tokens, at most
        ``tokens``, with which a step of ``lanes`` lanes fills a capacity but for one token in each padding
        lane (``tokens`` itself when nothing within an eighth below it does)."""
        if lanes >= tokens or tokens > self.BUCKET_MOST_TOKENS:
            return tokens
        lane_cap = bucket_for(lanes)
        best = 0
        for cap in (lane_cap, lane_cap << 1):
            pads = cap - lanes
            for token_cap in token_capacities(tokens + cap):
                fill = token_cap - pads
                if lanes < fill <= tokens and (pads > 0 or fill == token_cap):
                    best = max(best, fill)
        return best if best >= tokens - tokens // 8 else tokens

    def run_bucket(self, lanes: Sequence[Lane], lowered: LoweredLanes) -> Optional[torch.Tensor]:
        """Logits of a step with prompt portions from the captured graph of its capacity, or None when that
        capacity has no graph (yet): the caller then launches the step kernel by kernel."""
        capacity = self.capacity_for(len(lanes), int(lowered.lengths.sum()), int(lowered.want_counts.sum()))
        if capacity is None:
            self.counts["bucket_eager"] += 1
            return None
        context = self.context_bucket(lowered, at_least=capacity[1])
        if context < capacity[1]:                           # the cache cannot hold a padding lane of that many tokens
            self.counts["bucket_eager"] += 1
            return None
        key = capacity + (context,)
        entry = self._bucket_graphs.get(key)
        if entry is None:
            self._seen[key] = self._seen.get(key, 0) + 1
            self._seen.move_to_end(key)
            while len(self._seen) > 4 * self.BUCKET_GRAPHS:
                self._seen.popitem(last=False)
            if self._seen[key] < self.BUCKET_SIGHTINGS:
                self.counts["bucket_eager"] += 1
                return None
            entry = self._capture_bucket(key)
        else:
            self._bucket_graphs.move_to_end(key)
        static, graph, logits = entry
        static.fill(lowered)
        apply_feeds(static.context.token_ids, lowered.feeds)
        graph.replay()
        self.counts["bucket_replays"] += 1
        return logits[:int(lowered.want_counts.sum())].clone()

    def _capture_bucket(self, key: tuple):
        lane_cap, token_cap, want_cap, context = key
        static = StaticStep(self.cache, lane_cap, context, self.device, tokens=token_cap, wants=want_cap,
                            **self.model.step_layout)
        entry = self._capture(0, static, warm_runs=1)
        self.counts["bucket_captures"] += 1
        while len(self._bucket_graphs) >= self.BUCKET_GRAPHS:
            self._bucket_graphs.popitem(last=False)
        self._bucket_graphs[key] = entry
        return entry

    def warm_up(self, steps: Iterable[Tuple[int, int]], context: int = CONTEXT_BUCKET_FROM) -> List[tuple]:
        """Capture, before the first request, the graphs of steps of (lanes, tokens) with one wanted row a
        lane (steps of single tokens: their decode graphs); returns the keys of what was captured."""
        done = []
        for lanes, tokens in steps:
            if tokens == lanes:
                key = (bucket_for(lanes), min(max(context, CONTEXT_BUCKET_FROM), self.max_seq_len))
                if key not in self._graphs:
                    self._graphs[key] = self._capture(key[0], context=key[1])
                    done.append(key)
                continue
            capacity = self.capacity_for(lanes, tokens, lanes)
            if capacity is None:
                continue
            bucket = CONTEXT_BUCKET_FROM
            while bucket < max(context, capacity[1]):
                bucket <<= 1
            key = capacity + (min(bucket, self.max_seq_len),)
            if key[3] >= capacity[1] and key not in self._bucket_graphs:
                self._capture_bucket(key)
                done.append(key)
        return done

    def measure_split(self, prompt_tokens: int = 1024, singles: int = 16, replays: int = 5) -> Optional[float]:
        """The clock's answer to what a single decoded token costs beside a portion of a prompt, in units of what
        a batch of single tokens of its own costs: (time of ``prompt_tokens`` + ``singles`` single tokens as one
        batch - time of the portion alone) / ``singles`` / time of the ``singles`` alone.  Each of the three is
        a captured step whose lanes are all padding (nothing but the scratch page and slot is touched), replayed
        ``replays`` times; the median counts.  None when the single tokens cost nothing measurable."""
        prompt_tokens = min(prompt_tokens, self.max_seq_len)
        if prompt_tokens < 2:
            return None
        times = []
        for lengths in ([prompt_tokens], [prompt_tokens] + [1] * singles, [1] * singles):
            ends, row = [], 0
            for length in lengths:
                row += length
                ends.append(row - 1)
            static = StaticStep(self.cache, len(lengths), max(prompt_tokens, 64), self.device, lengths=lengths,
                                want_rows=ends, **self.model.step_layout)
            # (a memory pool of its own: the graphs' shared pool ends with the last graph in it)
            _, graph, _ = self._capture(0, static, warm_runs=1, pool=torch.cuda.graph_pool_handle())
            marks = [torch.cuda.Event(enable_timing=True) for _ in range(replays + 1)]
            graph.replay()
            marks[0].record()
            for mark in marks[1:]:
                graph.replay()
                mark.record()
            torch.cuda.synchronize(self.device)
            times.append(sorted(a.elapsed_time(b) for a, b in zip(marks, marks[1:]))[replays // 2])
            del graph, static
        portion, both, alone = times
        if both <= portion or alone <= 0:
            return None
        return (both - portion) / singles / alone

    def measure_halves(self, lanes: int = 128, replays: int = 5) -> Optional[float]:
        """The clock's answer to whether a step of ``lanes`` single tokens is faster as two halves at once, each a
        graph of its own on a stream of its own, than as one graph: the time of the two halves over the time of the
        one.  The halves read every weight twice, which a model whose steps wait for its weights cannot afford
        (the 7B shape: 20.8 ms for 96 single tokens in halves, 15.6 as one graph), while a small model's halves
        go through the skinny kernels and fill each other's waits (the 0.5B shape: 3.9 ms against 4.4).  Every
        lane of the three graphs is padding (nothing but the scratch page and slot is touched: the mixers' kernels
        cost little here, the products what they cost in a step); the median of ``replays`` counts."""
        context = min(CONTEXT_BUCKET_FROM, self.max_seq_len)
        whole = self._capture(bucket_for(lanes), context=context, warm_runs=1, pool=torch.cuda.graph_pool_handle())
        halves = [self._capture(bucket_for((lanes + 1) // 2), context=context, warm_runs=1,
                                pool=torch.cuda.graph_pool_handle()) for _ in range(2)]
        main = torch.cuda.current_stream(self.device)
        beside = torch.cuda.Stream(device=self.device)

        def as_one():
            whole[1].replay()

        def as_halves():
            beside.wait_stream(main)
            with torch.cuda.stream(beside):
                halves[1][1].replay()
            halves[0][1].replay()
            main.wait_stream(beside)

        times = []
        for run in (as_one, as_halves):
            marks = [torch.cuda.Event(enable_timing=True) for _ in range(replays + 1)]
            run()
            marks[0].record()
            for mark in marks[1:]:
                run()
                mark.record()
            torch.cuda.synchronize(self.device)
            times.append(sorted(a.elapsed_time(b) for a, b in zip(marks, marks[1:]))[replays // 2])
        del whole, halves
        return times[1] / times[0] if times[0] > 0 else None

    def _capture(self, bucket: int, static: Optional[StaticStep] = None, warm_runs: int = 2, context: int = 0,
                 pool=None):
        if static is None:
            static = StaticStep(self.cache, bucket, context or self.max_seq_len, self.device,
                                **self.model.step_layout)
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
        # one pool for every graph: replays never overlap, so their intermediate buffers may share memory
        if pool is None:
            if self._pool is None:
                self._pool = torch.cuda.graph_pool_handle()
            pool = self._pool
        with torch.cuda.graph(graph, pool=pool):
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
        apply_feeds(static.context.token_ids, lowered.feeds)
        graph.replay()
        self.counts["decode_replays"] += 1
        if int(lowered.want_counts.min()) > 0:
            return logits[:len(lanes)].clone()
        rows = [index for index, lane in enumerate(lanes) if len(lane.want) > 0]
        if not rows:
            return logits[:0].clone()
        return logits[torch.tensor(rows, device=logits.device)]
