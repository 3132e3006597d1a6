"""The fast paths of a layer whose mixers read the same normed rows and add their outputs (the
``parallel_prenorm`` arrangement, with one mixer or several).  A mixer that hands out its pieces
(``Mixer.projections``: input projection, what lies between, output projection) lets the layer run the
input projections of all its mixers as one matrix [mixer 0 | mixer 1 | ...] and their output projections
as one matrix along the inputs; the parts' own matrices are views of these.  Nothing here names a model:
any registered mixer that offers ``projections`` and ``mix`` takes part, and so does a feed-forward that
offers ``gated_projections`` and a norm that offers ``rms_prologue``; parts that do not run through their
own ``forward``.

Any step in bfloat16 (prompt portions, mixed batches): norm, one input GEMM, the mixers on column views
of its output, one output GEMM, norm, feed-forward: for two mixers, two library GEMMs fewer than part by
part.

Decode steps (every lane holds one token, at most 64 rows) go through the skinny kernels:

    1. residual add + norm + input projection of every mixer                    (fused_gemm)
    2. the mixers, each through its ``mix``, or all of them in one launch where a kernel for that
       set of mixers is registered (``register_mixer_kernel``)
    3. [mixer outputs] . [output projections]^T                                 (fused_gemm)
    4. residual add + norm + gate/up projection + SiLU(g)*u                     (fused_gemm)
    5. down projection                                                          (fused_gemm)

For attention beside Mamba2 such a kernel is registered below: the conv step runs in the epilogue of
launch 1 and both mixers in one launch 2 (``mixer_decode``), five launches a layer instead of fifteen
(seven for batches of more than 16 rows, whose two norms run as kernels of their own).  Where all four
products run through the skinny kernel, 3 and 5 may add to the residual stream themselves and leave the rows
that 4 and the next layer's 1 read, so that no launch and no prologue computes a norm (``FORCE_DEFERRED_NORM``
has the story).

A large weight goes through the BLAS library instead where that is faster (``LIBRARY_MIN_WEIGHT``); the
conv step and SiLU(g)*u then run as kernels of their own.  Which way each product goes is measured per step
size when the layer is built, and the layer's whole plan once more over a chain of layers when the model is
(``CHAIN_LAYERS``).  A second kernel of this engine's own is measured with them, whose waves share the step's
rows (``SHARED_ROWS_FROM``).  Steps of more single tokens than the skinny kernels take rows run
their products through the library around the same ``mixer_decode``, but for 3 and 5 in steps of up to 128 rows
where that second kernel's slabs are faster (``SHARED_ROWS_MOST``).

The fusion belongs to the arrangement (``register_fusion``), which knows its parts; the parts stay as they
are.  It is built only for bfloat16 weights and sizes the kernels cover; otherwise the block runs part by
part.
"""
from __future__ import annotations

import warnings
from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import Residual, ScaledRows
from .block import overlap_pays, register_fusion, side_stream

MAX_ROWS = 64          # rows of a step the skinny kernels take
MAX_NORM_ROWS = 16     # the norm prologue recomputes the normed rows in every workgroup: small batches only
# (and only as many rows as fit LDS at the layer's width, see LayerFusion.norm_rows), and narrow layers only: up to
# MAX_NORM_WIDTH a wave holds a row in registers; beyond, every workgroup reads its rows twice and its LDS fills
# a compute unit (a 3,072-wide layer at 8 rows: 7.84 ms a step with the prologue, 4.96 with the norms as kernels)
MAX_NORM_WIDTH = 2048
# A weight of this many elements or more is measured once, when the first layer of its shape is built, on
# both ways: the skinny kernel, and the BLAS library with the conv step or SiLU(g)*u as a kernel of its own.
# The skinny kernel reads the step's rows once per 16 weight rows and keeps all of K in one workgroup; the
# library tiles the rows and splits a long K, but its choice of tile swings from shape to shape (a 5120 x
# 21504 weight at 8 rows: 115 us against 69; a 3072 x 12288 one: 20 against 25), so the clock decides, per
# shape and per step size (TUNE_ROWS: up to 4, 8, 16, 32, 48 and 64 rows, each measured at its upper edge).  Below
# the limit the skinny kernel wins everywhere.
LIBRARY_MIN_WEIGHT = 2 << 20
LIBRARY_MARGIN = 0.92          # the library has to be this much faster to be taken
FORCE_LIBRARY: Optional[bool] = None      # tests: True or False instead of the clock
TUNE_ROWS = (4, 8, 16, 32, 48, 64)
_library_wins: Dict[tuple, tuple] = {}
# An output or down projection at 32 to 64 rows has a long K and few output features: 64 workgroups of the
# skinny kernel, or whatever tile the library picks (10.7 us for 1,024 x 2,048 at 64 rows).  Split over K into
# float32 slabs that the next norm adds up, the skinny kernel fills the GPU (7.5 us with 2 slabs; at 32 rows 5.2 us against the library's 9.6).  Measured
# at build like the library; the split has to win by SPLIT_MARGIN.
SPLIT_CHOICES = (2, 4, 8)
SPLIT_MARGIN = 0.92
# The slabs can also come from the kernel whose four waves own feature tiles and share the step's rows through
# LDS (in the skinny kernel every wave fetches rows of its own: as many bytes as the weights at 16 rows, four
# times as many at 64): a 5,120 x 21,504 weight at 64 rows in 52 us with 8 slabs, against 93 and the library's 133,
# at 8 rows in 43 against 50; a 3,072 x 12,288 one at 64 rows in 21 against 34 and 35.  Written as a negative
# number of feature tiles (that many a wave).  A slab costs the norm behind it a read, counted at SLAB_READ_RATE
# bytes a microsecond.  The kernel takes any number of rows, but is offered to the measurements from
# SHARED_ROWS_FROM rows on: below, what it gains on a product alone (the second weight above at 16 rows: 16 us in 8
# slabs against 22) a whole step loses again, with the norms as kernels of their own behind the slabs (the 7B shape
# at 8 / 16 rows: 5.01 / 6.46 ms a step with it, 4.96 / 6.25 without; the 34B shape at 8 rows 6.27 against 6.08 for
# 24 layers).
SHARED_ROWS_FROM = 17
# That kernel takes up to 128 rows (6 or 8 tiles of 16 rows a workgroup), the only one of this engine's products
# that does: steps of 65 to 128 single tokens, whose products otherwise all go through the library, take its slabs
# for the output and down projections where a measurement at 128 rows says so (3,072 x 12,288 at 96 / 128 rows: 25
# and 30 us against the library's 54 and 65; 5,120 x 21,504: 62 and 79 against 144 and 153; SiLU(gate) * up from
# it is slower than the library's product there and is not offered).
SHARED_ROWS_MOST = 128
FORCE_SHARED_ROWS: Optional[int] = None   # tests, with FORCE_SPLIT: this many tiles a wave of that kernel
SHARED_SPLIT_CHOICES = (4, 8, 16)
SLAB_READ_RATE = 4.0e6
FORCE_SPLIT: Optional[int] = None         # tests: a number of slabs (0 = never) instead of the clock
_split_wins: Dict[tuple, tuple] = {}
# Beyond 16 rows the skinny kernel's workgroup may own 2 or 4 tiles of 16 output features instead of one: the
# step's rows then cross the caches half or a quarter as often, and fewer workgroups each keep more weight
# fragments in flight (a 5120 x 21504 weight at 32 rows: 135 us with one tile, 86 with two, the library 125).
# Measured with the rest, per shape and step size.
TILE_CHOICES = (1, 2, 4)
TILE_MARGIN = 0.95             # a wider tile has to be this much faster than one tile to be taken
FORCE_TILES: Optional[int] = None         # tests: this many tiles for steps of more than 16 rows instead of the clock
# The library's tile for a prompt portion's input projection depends on the number of output features: 4 120
# of them (0.5B-shaped) take 30.5 us at 2,048 rows, 4 352 (a multiple of 256) take 23.6.  Measured at build in
# the same way, for portions of up to 256, 512, 1,024 and 2,048 tokens and beyond (each at its upper edge, the
# last at 4,096); where padding pays, the prompt path multiplies with zero rows added and ignores their columns.
PAD_FEATURES = 256
PAD_ROWS = (256, 512, 1024, 2048, 4096)
PAD_MARGIN = 0.95
FORCE_PADDING: Optional[bool] = None      # tests: True or False instead of the clock
# The attended heads of a decode step come in runs of keys that a small kernel merges; the output projection
# can merge them in its prologue instead, every workgroup of it again: one launch less, but the projection then
# starts behind a read of the runs.  It pays while a workgroup reads few of them (0.5B-shaped at 2,048-token
# contexts: 1.33 -> 1.26 ms a step at 1 row, 1.39 -> 1.37 at 4, even at 6 to 8, slower from 16; 7B-shaped: faster
# at 1 and 2 rows, slower at 4): up to MERGE_LATER_BYTES of runs a workgroup.
MERGE_LATER_ROWS = 16
MERGE_LATER_BYTES = 96 << 10
FORCE_MERGE_LATER: Optional[bool] = None  # tests: True or False instead of the rule
_padding_wins: Dict[tuple, tuple] = {}
# A projection whose result joins the residual stream can add it there itself (float32, in place) and leave, beside
# the stream, its rows times the next norm's weight in bfloat16 with the partial sums of their squares; the product
# behind that norm then reads those rows and multiplies its float32 sums by 1 / sqrt(mean square + eps): the norm
# costs no pass of its own and no prologue in every workgroup.  Taken for the step sizes at which a layer's four
# projections all run through the skinny kernel unsplit, with one tile in the two that feed the stream.
FORCE_DEFERRED_NORM: Optional[bool] = None  # tests: False = never
# What is fastest for one projection alone need not be fastest for the layer: a down projection that wins by a
# microsecond with two tiles or in slabs keeps the norms as kernels of their own.  So once a model's layers are
# built, a chain of up to CHAIN_LAYERS layers of one shape (their projections and norms, without the mixers) is
# timed per step size with the projections' own choices, with the norms left to them where those choices allow
# it, and with all four through the skinny kernel and the norms left to them; the alternatives have to win by
# CHAIN_MARGIN.  (8 layers of the 34B shape at 1 to 4 rows: 2.95 -> 2.03 ms a step; at 8 rows the projections'
# own choices stay.)
CHAIN_LAYERS = 8
CHAIN_MARGIN = 0.97
# Where the norms are left to the projections, a step of more than 16 rows can have its tiles of 16 rows dealt out
# to several workgroups per tile of features instead of every workgroup taking them all.  The two projections that
# feed the stream have few output features (1,024 of them: 64 workgroups, each of which fetches all of the step's
# rows): with 64 rows over four workgroups 1,024 x 2,048 takes 5.9 us instead of 11.4, at 32 rows 5.7 instead of
# 7.5, and the same bits come out, so this is a fixed rule up to ROW_TILES_FEATURES output features (3,072 x 7,680
# gains at 64 rows only, 35 us against 41, and loses below).  The products behind the norms gain less (4,120 x 1,024
# at 64 rows: 9.4 us against 11.8) and add their rows' partial sums of squares in another order, so for them, and
# beyond the rule, the clock decides over the chain of layers.  A plan's number: 1 = every workgroup all rows,
# 2 = over two workgroups, 4 = one tile of 16 rows each.
ROW_TILES_FEATURES = 2048
FORCE_ROW_TILES: Optional[int] = None     # tests: this number for all four projections instead of the rule and the clock
PLAN_FIELDS = ("library_in", "library_out", "library_gate_up", "library_down", "split_out", "split_down",
               "tiles_in", "tiles_out", "tiles_gate_up", "tiles_down", "deferred",
               "rows_in", "rows_out", "rows_gate_up", "rows_down")
_chain_wins: Dict[tuple, tuple] = {}
_chain_times: list = []     # (rows, microseconds a layer of each candidate, the one taken): what was measured, for whoever asks


def _bucket(rows: int) -> int:
    """The step size a step of ``rows`` rows was measured as: the first of TUNE_ROWS that holds it."""
    for bucket, most in enumerate(TUNE_ROWS):
        if rows <= most:
            return bucket
    return len(TUNE_ROWS) - 1


BUCKETS = len(TUNE_ROWS)
BEYOND = BUCKETS       # the place, behind the measured step sizes, of the plan for steps of more than MAX_ROWS single tokens


def _each(value) -> tuple:
    return (value,) * BUCKETS


def _graph_microseconds(run) -> float:
    """Time of one call of ``run`` on the GPU, replayed from a graph (no launch gaps)."""
    device = torch.cuda.current_device()
    side = torch.cuda.Stream(device=device)
    side.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream(device).wait_stream(side)
    torch.cuda.synchronize(device)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()
    graph.replay()
    torch.cuda.synchronize(device)
    best = float("inf")
    for _ in range(3):                     # the least of three rounds: a round that something else disturbed is left out
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(3):
            graph.replay()
        end.record()
        end.synchronize()
        best = min(best, start.elapsed_time(end) * 1e3 / 3)
    return best


def _padding_pays(weight: torch.Tensor, measure: bool = True) -> tuple:
    """For every portion size of PAD_ROWS: whether rows of zeros up to a multiple of PAD_FEATURES make the
    library's product of a prompt portion faster."""
    N, K = weight.shape
    if N % PAD_FEATURES == 0 or FORCE_PADDING is False or (FORCE_PADDING is None and not measure):
        return (False,) * len(PAD_ROWS)
    if FORCE_PADDING:
        return (True,) * len(PAD_ROWS)
    if weight.numel() < LIBRARY_MIN_WEIGHT:
        return (False,) * len(PAD_ROWS)
    key = (N, K)
    if key not in _padding_wins:
        padded = torch.cat([weight, weight.new_zeros((-N % PAD_FEATURES, K))])
        wins = []
        for rows in PAD_ROWS:
            x = torch.full((rows, K), 0.01, dtype=torch.bfloat16, device=weight.device)

            def plain():
                for _ in range(4):
                    torch.matmul(x, weight.t())

            def wide():
                for _ in range(4):
                    torch.matmul(x, padded.t())

            wins.append(_graph_microseconds(wide) < PAD_MARGIN * _graph_microseconds(plain))
        _padding_wins[key] = tuple(wins)
    return _padding_wins[key]


def _portion_bucket(rows: int) -> int:
    for bucket, most in enumerate(PAD_ROWS):
        if rows <= most:
            return bucket
    return len(PAD_ROWS) - 1


def _measure_split(weight: torch.Tensor, bias, rows: int, library: bool, tiles: int) -> tuple:
    """(slabs, feature tiles): the number of float32 slabs over K with which the skinny kernel, or the kernel that
    shares the rows (negative tiles; the only one beyond MAX_ROWS rows), beats the way this projection would go
    otherwise (the library, or the skinny kernel unsplit) at this many rows, or 0."""
    N, K = weight.shape
    device = weight.device
    copies = max(2, min(64, (512 << 20) // (weight.numel() * 2)))
    weights = [weight] + [weight.clone() for _ in range(copies - 1)]
    fragments = [ops.fragment_order(w) for w in weights]
    x = torch.full((rows, K), 0.01, dtype=torch.bfloat16, device=device)
    out = torch.empty((rows, N), dtype=torch.bfloat16, device=device)

    def whole():
        for w, f in zip(weights, fragments):
            if library:
                ops.linear(x, w, bias)
            else:
                ops.fused_gemm(w, bias, out, x=x, feature_tiles=tiles, fragments=f)

    best, best_time = (0, tiles), SPLIT_MARGIN * _graph_microseconds(whole)
    shared_from = SHARED_ROWS_FROM if K // 32 >= 4 else rows + 1
    for slabs in sorted(set(SPLIT_CHOICES) | (set(SHARED_SPLIT_CHOICES) if rows >= shared_from else set())):
        if K // 32 < slabs:
            continue
        partial = torch.empty((slabs, rows, N), dtype=torch.float32, device=device)
        ways = [tile for tile in TILE_CHOICES[:2] if slabs in SPLIT_CHOICES and rows <= MAX_ROWS]
        ways += [-tile for tile in TILE_CHOICES[:1 if rows > MAX_ROWS else 2]
                 if rows >= shared_from and slabs in SHARED_SPLIT_CHOICES]
        for split_tiles in ways:

            def split():
                for w, f in zip(weights, fragments):
                    ops.fused_gemm_split(w, bias, x, partial, feature_tiles=abs(split_tiles), fragments=f,
                                         shared_rows=split_tiles < 0)

            time = _graph_microseconds(split) + len(weights) * partial.numel() * 4 / SLAB_READ_RATE
            if time < best_time:
                best, best_time = (slabs, split_tiles), time
    return best


def _measure_library(weight: torch.Tensor, bias, rows: int, epilogue: int, tile: int, conv: Optional[dict],
                     wide: bool) -> tuple:
    """(whether the library way is faster for this weight at this many rows, the skinny kernel's best number
    of feature tiles; ``wide``: more than one tile may be taken, i.e. the prologue is the plain one; negative:
    that many a wave of the kernel that shares the rows, which SiLU(gate) * up and the conv step can come from;
    the two that feed the residual stream take its slabs or none).  Copies
    of the weight are cycled through so that the caches do not hold it, as in a model of many layers."""
    N, K = weight.shape
    device = weight.device
    copies = max(2, min(64, (512 << 20) // (weight.numel() * 2)))
    weights = [weight] + [weight.clone() for _ in range(copies - 1)]
    x = torch.full((rows, K), 0.01, dtype=torch.bfloat16, device=device)      # not drawn: the global generator stays as it is
    out = torch.empty((rows, N // 2 if epilogue == ops.EPI_SWIGLU else N), dtype=torch.bfloat16, device=device)
    if conv is not None:
        channels = conv["hi"] - conv["lo"]
        conv = dict(conv, state=torch.zeros((rows, max(conv["taps"] - 1, 0), channels), dtype=torch.bfloat16, device=device),
                    slot_ids=torch.arange(rows, dtype=torch.int32, device=device))

    fragments = [ops.fragment_order(w) for w in weights]

    def skinny(tiles):
        def run():
            for w, f in zip(weights, fragments):
                ops.fused_gemm(w, bias, out, x=x, epilogue=epilogue, conv=conv, feature_tiles=tiles, fragments=f)
        return run

    def library():
        for w in weights:
            product = ops.linear(x, w, bias)
            if epilogue == ops.EPI_SWIGLU:
                ops.swiglu(product, out, tile)
            elif epilogue == ops.EPI_CONV:
                ops.conv_step(product, conv["lo"], conv["hi"] - conv["lo"], conv["weight"], conv["bias"], conv["state"],
                              conv["slot_ids"])

    def shared_rows(tiles):
        def run():
            for w, f in zip(weights, fragments):
                ops.fused_gemm(w, bias, out, x=x, epilogue=epilogue, conv=conv, feature_tiles=tiles, fragments=f,
                               shared_rows=True)
        return run

    times = {tiles: _graph_microseconds(skinny(tiles)) for tiles in (TILE_CHOICES if wide else (1,))}
    if wide and epilogue != ops.EPI_PLAIN and rows >= SHARED_ROWS_FROM and K // 32 >= 4:
        times.update({-tiles: _graph_microseconds(shared_rows(tiles)) for tiles in TILE_CHOICES[:2]})
    tiles = min(times, key=lambda count: times[count] * (1.0 if count == 1 else 1.0 / TILE_MARGIN))
    return _graph_microseconds(library) < LIBRARY_MARGIN * times[tiles], tiles


_MIXER_KERNELS: Dict[tuple, object] = {}


class FastPathDeclined(UserWarning):
    """A layer that could have run its steps of single tokens in one launch runs them through the general kernels
    instead (correct, several times slower): the message says what the fast path misses."""


def _decline(reason: str) -> None:
    warnings.warn(f"no fused decode step for this layer: {reason}", FastPathDeclined, stacklevel=3)


def register_mixer_kernel(*kinds: str):
    """Register ``factory(fusion) -> kernel or None`` for layers whose mixers are of exactly these kinds, in
    this order: a kernel that runs all of them in one launch in steps of single tokens.  The kernel object
    offers ``conv`` (None, or the columns of the input projection that go through a conv step in that
    product's epilogue: {lo, hi, taps, weight, bias}), ``supported(step, caches)``,
    ``conv_state(caches)`` and ``run(u, step, caches, mixed, merge=True)``; a kernel with ``merge_later_bytes(step,
    caches)`` returns, when called with ``merge=False``, the runs of keys of its attended heads (the first columns of
    ``mixed``) unmerged, as ``ops.AttentionRuns``, for the output projection to merge."""
    def decorate(factory):
        _MIXER_KERNELS[tuple(kinds)] = factory
        return factory
    return decorate


@register_fusion("parallel_prenorm")
def build_layer_fusion(block, build) -> Optional["LayerFusion"]:
    return LayerFusion.build(block, build)


def _run_chain(chain, rows: int, bucket: int, h: torch.Tensor, mixed: torch.Tensor, tails=None) -> None:
    """The projections and norms of the layers of ``chain`` one after the other, as a decode step of ``rows``
    rows runs them (the mixers left out: the same rows stand for what they would write).  ``tails``: (conv state
    of ``rows`` slots, their ids), where the input projection runs a conv step in its epilogue."""
    residual = Residual(h)
    for index, fusion in enumerate(chain):
        residual.next_norm = chain[(index + 1) % len(chain)].mixer_scale
        conv = None
        if tails is not None and fusion.kernel is not None and fusion.kernel.conv is not None:
            conv = dict(fusion.kernel.conv, state=tails[0], slot_ids=tails[1])
        fusion._project_in(residual, rows, bucket, conv)
        fusion._after_the_mixers(residual, mixed, None, rows, bucket)


def _measure_chain(chain, bucket: int) -> dict:
    """The fastest plan (a value for each of PLAN_FIELDS) for steps of TUNE_ROWS[bucket] rows through the layers
    of ``chain``, which are of one shape; the layers are left as they were."""
    first = chain[0]
    rows = TUNE_ROWS[bucket]
    current = first._plan(bucket)
    candidates = [dict(current, deferred=False)]
    if first._may_defer(current):
        candidates.append(dict(current, deferred=True))
    skinny = dict(current, library_in=False, library_out=False, library_gate_up=False, library_down=False,
                  split_out=0, split_down=0, tiles_out=1, tiles_down=1, deferred=True)
    if (skinny not in candidates and first._may_defer(skinny)
            and all(f is not None for fusion in chain for f in (fusion.f_in, fusion.f_out, fusion.f_gate_up, fusion.f_down))):
        candidates.append(skinny)
    device = first.w_in.device
    h = torch.full((rows, first.hidden), 0.01, dtype=torch.float32, device=device)
    mixed = torch.full((rows, first.mixed_width), 0.01, dtype=torch.bfloat16, device=device)
    tails = None
    conv = first.kernel.conv if first.kernel is not None else None
    if conv is not None:            # the conv step is part of the input projection's time (4 of its 14 us at 64 rows of 4,120 features)
        tails = (torch.zeros((rows, max(conv["taps"] - 1, 0), conv["hi"] - conv["lo"]), dtype=torch.bfloat16, device=device),
                 torch.arange(rows, dtype=torch.int32, device=device))
    times = []

    def clock(plan):
        for fusion in chain:
            fusion._apply(bucket, plan)
        times.append(_graph_microseconds(lambda: _run_chain(chain, rows, bucket, h, mixed, tails)))

    def fastest():
        return min(range(len(candidates)), key=lambda index: times[index] / (1.0 if index == 0 else CHAIN_MARGIN))

    for plan in candidates:
        clock(plan)
    base = candidates[fastest()]
    if rows > 16 and base["deferred"]:          # the winner with its rows dealt out otherwise: (into the stream, behind the norms)
        for stream, behind in ((1, 1), (4, 1), (2, 1), (4, 4), (4, 2)):
            variant = dict(base, rows_out=stream, rows_down=stream, rows_in=behind, rows_gate_up=behind)
            if behind > 1:
                variant.update(tiles_in=1, tiles_gate_up=1)
            if variant not in candidates:
                candidates.append(variant)
                clock(variant)
    for fusion in chain:
        fusion._apply(bucket, current)
    best = fastest()
    _chain_times.append((rows, [round(time / len(chain), 2) for time in times], best))
    return candidates[best]


class LayerFusion:
    @staticmethod
    def build(block, build) -> Optional["LayerFusion"]:
        if build.dtype != torch.bfloat16 or build.device.type != "cuda":
            return None
        pieces = [mixer.projections() if hasattr(mixer, "projections") else None for _, mixer in block.mixers]
        if not pieces or any(piece is None for piece in pieces):
            return None
        linears = [linear for piece in pieces for linear in piece[:2]]
        if any(linear.weight.dtype != torch.bfloat16 for linear in linears):
            return None
        fusion = LayerFusion(block, pieces, build)
        return fusion if fusion.general or fusion.decode_ok else None

    def __init__(self, block, pieces, build):
        self.block = block
        device = build.device
        self.hidden = build.hidden_size
        self.measure = bool(getattr(build, "measure_paths", True))
        self.names = [name for name, _ in block.mixers]
        self.mixers = [mixer for _, mixer in block.mixers]
        in_linears, out_linears = [piece[0] for piece in pieces], [piece[1] for piece in pieces]
        # columns of each mixer in the input projection's output and in the rows the output projection reads
        self.in_cols, self.mixed_cols, first_in, first_mixed = [], [], 0, 0
        for in_linear, _, width in pieces:
            self.in_cols.append((first_in, first_in + in_linear.out_features))
            self.mixed_cols.append((first_mixed, first_mixed + width))
            first_in += in_linear.out_features
            first_mixed += width
        # 1: [mixer 0 | mixer 1 | ...]
        self.w_in = torch.cat([linear.weight for linear in in_linears], dim=0).contiguous()
        self.b_in = _cat_bias(in_linears, device)
        # prompt portions may multiply with rows of zeros added (the decode kernels take the rows that count)
        self.w_in_wide, self.b_in_wide = self.w_in, self.b_in
        self.padding_pays = _padding_pays(self.w_in, self.measure)          # by portion size
        if any(self.padding_pays):
            extra = -self.w_in.shape[0] % PAD_FEATURES
            self.w_in_wide = torch.cat([self.w_in, self.w_in.new_zeros((extra, self.w_in.shape[1]))])
            self.w_in = self.w_in_wide[:self.w_in.shape[0]]
            if self.b_in is not None:
                self.b_in_wide = torch.cat([self.b_in, self.b_in.new_zeros(extra)])
        self.in_width = self.w_in.shape[0]
        self.in_ld = -(-self.in_width // 8) * 8
        # 3: [mixer outputs] . [output projections]^T
        self.w_out = torch.cat([linear.weight for linear in out_linears], dim=1).contiguous()
        biases = [linear.bias for linear in out_linears if linear.bias is not None]
        self.b_out = sum(biases[1:], biases[0]).contiguous() if biases else None
        self.mixed_width = first_mixed
        for in_linear, out_linear, (lo, hi), (mixed_lo, mixed_hi) in zip(in_linears, out_linears, self.in_cols,
                                                                         self.mixed_cols):
            in_linear.weight = self.w_in[lo:hi]                       # the parts' matrices: views of the fused ones
            out_linear.weight = self.w_out[:, mixed_lo:mixed_hi]
        # the column views the mixers get must start at 16 bytes and rows must be multiples of 8 elements
        self.aligned = self.mixed_width % 8 == 0 and all(lo % 8 == 0 for lo, _ in self.in_cols + self.mixed_cols)
        self.general = self.aligned and self.in_width % 8 == 0
        # 4 and 5: a gated feed-forward whose gate and up rows are interleaved in tiles of 8 (the part stores them
        # so) runs through the skinny kernels as well; any other runs through its own forward
        gated = block.ffn.gated_projections() if hasattr(block.ffn, "gated_projections") else None
        self.gate_up, self.down, self.inner = None, None, 0
        if gated is not None and gated[2] == 8 and gated[0].weight.dtype == torch.bfloat16 \
                and gated[1].weight.dtype == torch.bfloat16 and gated[1].in_features % 32 == 0:
            self.gate_up, self.down, _ = gated
            self.inner = self.down.in_features
        # the skinny kernels take K in chunks of 32
        self.decode_ok = (self.hidden % 32 == 0 and self.mixed_width % 32 == 0
                          and ops.fused_gemm_supported(False, 1, self.hidden)
                          and ops.fused_gemm_supported(False, 1, self.mixed_width)
                          and (self.gate_up is None or ops.fused_gemm_supported(False, 1, self.inner)))
        # norms that the skinny kernel computes in its prologue (a wide model's rows do not fit its LDS, and another
        # kind of norm is not what it computes: those run as kernels of their own)
        # (the largest step size of TUNE_ROWS, up to MAX_NORM_ROWS, whose rows fit LDS at this width; steps of more
        # rows, the "wide" step sizes, run their norms as kernels of their own)
        self.norm_rows = max([rows for rows in TUNE_ROWS if rows <= MAX_NORM_ROWS and self.decode_ok
                              and self.hidden <= MAX_NORM_WIDTH and ops.fused_gemm_supported(True, rows, self.hidden)],
                             default=0)
        self.wide_buckets = tuple(bucket for bucket, rows in enumerate(TUNE_ROWS) if rows > self.norm_rows)
        self.mixer_rms = _rms_prologue(block.mixer_norm) if self.norm_rows else None
        self.ffn_rms = _rms_prologue(block.ffn_norm) if self.norm_rows else None
        self.norm_fits = self.mixer_rms is not None and self.ffn_rms is not None
        # the same two norms for the products that take them as a row scale (any width)
        self.mixer_scale = _rms_prologue(block.mixer_norm) if self.decode_ok else None
        self.ffn_scale = _rms_prologue(block.ffn_norm) if self.decode_ok else None
        # a kernel for this set of mixers, if one is registered and takes these sizes
        factory = _MIXER_KERNELS.get(tuple(getattr(mixer, "kind", None) for mixer in self.mixers))
        self.kernel = factory(self) if factory is not None and self.decode_ok else None
        if self.kernel is None and not self.aligned:          # no view of its columns for a mixer's own ``mix``
            self.decode_ok = False
        conv = self.kernel.conv if self.kernel is not None else None
        # which projections go through the library, by step size
        # (and how many tiles of 16 output features a workgroup of the skinny kernel owns where it is taken)
        self.library_in, self.tiles_in = self._tune(self.w_in, self.b_in, ops.EPI_CONV if conv else ops.EPI_PLAIN, conv,
                                                    self.mixer_rms is not None)
        self.library_out, self.tiles_out = self._tune(self.w_out, self.b_out, ops.EPI_PLAIN)
        # and which of the two that feed the residual stream are split over K instead (steps of more than norm_rows rows)
        self.split_out, self.tiles_out = self._tune_split(self.w_out, self.b_out, self.library_out, self.tiles_out)
        beyond_out, beyond_down = self._tune_split_beyond(self.w_out, self.b_out), (0, 1)
        # what the skinny kernel reads: a second copy of each matrix in the order of its waves' fragments (one run
        # of 1 KiB a load instead of 64 bytes of each of 16 rows: 15 to 25 % faster); the row-major ones stay for
        # the library and for prompt portions.  A projection that always goes through the library has none.

        def fragments(weight, library, split):
            if not self.decode_ok or (all(library) and not any(split)):
                return None
            return ops.fragment_order(weight)

        self.f_in = fragments(self.w_in, self.library_in, ())
        self.f_out = fragments(self.w_out, self.library_out, self.split_out + beyond_out[:1])
        if self.gate_up is not None:
            self.library_gate_up, self.tiles_gate_up = self._tune(self.gate_up.weight, self.gate_up.bias, ops.EPI_SWIGLU,
                                                                  None, self.ffn_rms is not None)
            self.library_down, self.tiles_down = self._tune(self.down.weight, self.down.bias, ops.EPI_PLAIN)
            self.split_down, self.tiles_down = self._tune_split(self.down.weight, self.down.bias, self.library_down,
                                                                self.tiles_down)
            beyond_down = self._tune_split_beyond(self.down.weight, self.down.bias)
            self.f_gate_up = fragments(self.gate_up.weight, self.library_gate_up, ())
            self.f_down = fragments(self.down.weight, self.library_down, self.split_down + beyond_down[:1])
        # how the rows of a step are dealt out where the norms are left to the projections
        self.rows_in = self.rows_gate_up = _each(1 if FORCE_ROW_TILES is None else FORCE_ROW_TILES)
        self.rows_out = self._row_tiles(self.w_out)
        self.rows_down = self._row_tiles(self.down.weight) if self.down is not None else _each(1)
        # step sizes at which the norms are left to the projections around them
        self.deferred = _each(False)
        self.deferred = tuple(self._may_defer(self._plan(bucket)) for bucket in range(BUCKETS))
        # and behind the measured step sizes the plan of steps of more than MAX_ROWS single tokens: every projection
        # through the library, with the mixers' decode kernel between them; for up to SHARED_ROWS_MOST of them the two
        # that feed the stream in slabs from the kernel that shares the rows, where that is faster
        beyond = dict(library_in=True, library_out=True, library_gate_up=True, library_down=True,
                      split_out=beyond_out[0], split_down=beyond_down[0], tiles_in=1, tiles_out=beyond_out[1],
                      tiles_gate_up=1, tiles_down=beyond_down[1], deferred=False, rows_in=1, rows_out=1, rows_gate_up=1,
                      rows_down=1)
        for name, value in beyond.items():
            if hasattr(self, name):
                setattr(self, name, getattr(self, name) + (value,))

    def _row_tiles(self, weight: torch.Tensor) -> tuple:
        """The fixed rule for a projection into the stream: one tile of 16 rows a workgroup where it has few output
        features and the step more than 16 rows."""
        if FORCE_ROW_TILES is not None:
            return _each(FORCE_ROW_TILES)
        return tuple(4 if rows > 16 and weight.shape[0] <= ROW_TILES_FEATURES else 1 for rows in TUNE_ROWS)

    def _plan(self, bucket: int) -> dict:
        """How steps of TUNE_ROWS[bucket] rows go through the layer's projections."""
        if self.gate_up is None:
            return {}
        return {name: getattr(self, name)[bucket] for name in PLAN_FIELDS}

    def _apply(self, bucket: int, plan: dict) -> None:
        for name, value in plan.items():
            values = list(getattr(self, name))
            values[bucket] = value
            setattr(self, name, tuple(values))

    def _may_defer(self, plan: dict) -> bool:
        """Whether the norms can be left to the projections under ``plan``: all four through the skinny kernel,
        the two that feed the stream whole and with one tile."""
        if (FORCE_DEFERRED_NORM is False or self.gate_up is None or not self.decode_ok or self.ffn_scale is None
                or self.hidden % 16 != 0):
            return False
        return not (plan["library_in"] or plan["library_out"] or plan["library_gate_up"] or plan["library_down"]
                    or plan["split_out"] or plan["split_down"] or plan["tiles_out"] != 1 or plan["tiles_down"] != 1)

    def _shape_key(self) -> tuple:
        return (tuple(self.w_in.shape), tuple(self.w_out.shape), self.inner, self.b_in is None, self.b_out is None,
                self.gate_up is not None and self.gate_up.bias is None, self.down is not None and self.down.bias is None,
                self.norm_rows, self.mixer_scale is None, self.ffn_scale is None)

    def tune_chain(self, peers) -> None:
        """Called once the model's layers are built, with the fusions of all of them: the plan of each step size
        by the clock over a chain of layers of this one's shape (measured once per shape)."""
        if (not self.measure or not self.decode_ok or self.gate_up is None or self.ffn_scale is None
                or self.mixer_scale is None
                or any(force is not None for force in (FORCE_DEFERRED_NORM, FORCE_LIBRARY, FORCE_SPLIT, FORCE_TILES,
                                                      FORCE_SHARED_ROWS, FORCE_ROW_TILES))
                or self.w_in.numel() + self.w_out.numel() + self.gate_up.weight.numel() + self.down.weight.numel()
                < LIBRARY_MIN_WEIGHT):
            return
        key = self._shape_key()
        if key not in _chain_wins:
            chain = [peer for peer in peers if isinstance(peer, LayerFusion) and peer._shape_key() == key][:CHAIN_LAYERS]
            _chain_wins[key] = tuple(_measure_chain(chain, bucket) for bucket in range(BUCKETS))
        for bucket, plan in enumerate(_chain_wins[key]):
            self._apply(bucket, plan)

    def path_choices(self) -> dict:
        """Which way each projection goes for steps of up to TUNE_ROWS rows, as short strings (S: the skinny
        kernel, L: the library, a number: that many slabs over K), the feature tiles of the skinny kernel (with
        an r: a wave's, of the kernel that shares the rows), for portions of up to PAD_ROWS tokens whether
        the input projection is padded (P), and how the output and down projections of steps of more than
        MAX_ROWS single tokens go (up to SHARED_ROWS_MOST of them: slabs, or L)."""
        if not self.decode_ok:
            return {}

        def way(library, split=None):
            library = library[:BUCKETS]
            split = split or (0,) * len(library)
            return "/".join(str(slabs) if slabs else ("L" if lib else "S") for lib, slabs in zip(library, split))

        def tiled(tiles):
            return "/".join(str(tile) if tile > 0 else f"{-tile}r" for tile in tiles[:BUCKETS])

        def beyond(split):
            return str(split[BEYOND]) if split[BEYOND] else "L"

        out = {"in": way(self.library_in), "out": way(self.library_out, self.split_out),
               "tiles_in": tiled(self.tiles_in), "tiles_out": tiled(self.tiles_out),
               "padded_in": "/".join("P" if pays else "-" for pays in self.padding_pays)}
        if self.gate_up is not None:
            out.update({"gate_up": way(self.library_gate_up), "down": way(self.library_down, self.split_down),
                        "tiles_gate_up": tiled(self.tiles_gate_up), "tiles_down": tiled(self.tiles_down),
                        "norms": "/".join("D" if deferred else "-" for deferred in self.deferred[:BUCKETS]),
                        "rows": "/".join("".join(str(rows[bucket]) for rows in (self.rows_in, self.rows_out, self.rows_gate_up,
                                                                                self.rows_down)) if self.deferred[bucket] else "-"
                                         for bucket in range(BUCKETS)),
                        "beyond_out_down": f"{beyond(self.split_out)}/{beyond(self.split_down)}"})
        return out

    def decode_supported(self, step, caches) -> bool:
        """Whether the step's rows go through the decode path: steps of up to MAX_ROWS single tokens through the
        skinny products (or the library, as measured) around the mixers' decode kernel; steps of as few tokens in
        portions of prompts (a short prompt, the tail of a long one, beside decoded tokens), whose mixers then
        run their own kernels between those products; and steps of more single tokens than that, whose products
        all go through the library, when there is a decode kernel for the mixers (the prompt kernels would take a
        step of 96 single tokens as 96 prompts of one token: 9.1 ms on the 0.5B shape against 3.3 for 64)."""
        if not self.decode_ok:
            return False
        if step.num_tokens > MAX_ROWS:
            return (self.general and step.max_query_len == 1 and self.kernel is not None
                    and self.kernel.supported(step, caches))
        if step.max_query_len != 1:
            return self.aligned
        return self.aligned or self.kernel.supported(step, caches)

    def forward(self, residual: Residual, step, caches) -> bool:
        """Runs the layer and returns True, or returns False with nothing done (the block then
        runs part by part)."""
        if self.decode_supported(step, caches):
            self.forward_decode(residual, step, caches)
            return True
        if self.general:
            self.forward_general(residual, step, caches)
            return True
        return False

    def _mix_each(self, u: torch.Tensor, step, caches, mixed: torch.Tensor, order=None) -> None:
        for index in (range(len(self.mixers)) if order is None else order):
            (lo, hi), (mixed_lo, mixed_hi) = self.in_cols[index], self.mixed_cols[index]
            self.mixers[index].mix(u[:, lo:hi], step, caches[self.names[index]], mixed[:, mixed_lo:mixed_hi])

    def forward_general(self, residual: Residual, step, caches) -> None:
        block = self.block
        normed = block.mixer_norm.forward(residual)
        if self.padding_pays[_portion_bucket(normed.shape[0])]:
            u = ops.linear(normed, self.w_in_wide, self.b_in_wide)
        else:
            u = ops.linear(normed, self.w_in, self.b_in)
        mixed = torch.empty((u.shape[0], self.mixed_width), dtype=u.dtype, device=u.device)
        if overlap_pays(self.mixers, u.shape[0], u.device):
            # two mixers read the same rows and write different columns: the first runs on a second stream
            # beside the second (in a captured graph only: launched one by one the step waits for the host,
            # which the second stream costs more).  The mixer on the main stream is recorded first: the graph
            # keeps the branch it meets first on the queue of the projections before and after it, and the
            # other branch pays the hops between queues.  (Attention beside a state-space mixer, whose kernels
            # are many and small: the state-space chain is the longer one and stays on the main queue.)
            main = torch.cuda.current_stream(u.device)
            side = side_stream(u.device, main)
            side.wait_stream(main)
            self._mix_each(u, step, caches, mixed, order=(1,))
            with torch.cuda.stream(side):
                self._mix_each(u, step, caches, mixed, order=(0,))
            main.wait_stream(side)
        else:
            self._mix_each(u, step, caches, mixed)
        residual.pending = [ops.linear(mixed, self.w_out, self.b_out)]
        normed = block.ffn_norm.forward(residual)
        residual.pending = [block.ffn.forward(normed)]

    def _tune(self, weight: torch.Tensor, bias, epilogue: int, conv: Optional[dict] = None,
              normed: bool = False) -> tuple:
        """For every step size of TUNE_ROWS: whether this projection goes through the library, and the feature
        tiles of the skinny kernel.  (``normed``: the norm before it runs in the skinny kernel's prologue in steps
        of up to ``norm_rows`` rows; those stay with the skinny kernel and one tile.)"""
        if not self.decode_ok:
            return _each(True), _each(1)
        choices, tiles = self._tune_all(weight, bias, epilogue, conv, normed)
        if normed:
            choices = tuple(choice and bucket in self.wide_buckets for bucket, choice in enumerate(choices))
        return choices, tiles

    def _tune_split(self, weight: torch.Tensor, bias, library: tuple, tiles: tuple) -> tuple:
        """For every step size of TUNE_ROWS: the number of slabs over K, or 0 for the whole product, and the
        feature tiles that go with it.  Steps of up to ``norm_rows`` rows feed the next kernel's norm prologue,
        which takes whole rows."""
        if self.hidden % 4 != 0 or FORCE_SPLIT == 0:
            return _each(0), tiles
        if FORCE_SPLIT:
            slabs = FORCE_SPLIT if weight.shape[1] // 32 >= FORCE_SPLIT else 0
            if FORCE_SHARED_ROWS and slabs and weight.shape[1] // 32 >= 4:
                tiles = tuple(-FORCE_SHARED_ROWS if bucket in self.wide_buckets else tile for bucket, tile in enumerate(tiles))
            return tuple(slabs if bucket in self.wide_buckets else 0 for bucket in range(BUCKETS)), tiles
        if weight.numel() < LIBRARY_MIN_WEIGHT or not self.measure:
            return _each(0), tiles
        slabs, split_tiles = [], []
        for bucket in range(BUCKETS):
            if bucket not in self.wide_buckets:
                slabs.append(0)
                split_tiles.append(tiles[bucket])
                continue
            key = (tuple(weight.shape), bias is None, bucket, library[bucket], tiles[bucket])
            if key not in _split_wins:
                _split_wins[key] = _measure_split(weight, bias, TUNE_ROWS[bucket], library[bucket], tiles[bucket])
            slabs.append(_split_wins[key][0])
            split_tiles.append(_split_wins[key][1])
        return tuple(slabs), tuple(split_tiles)

    def _tune_split_beyond(self, weight: torch.Tensor, bias) -> tuple:
        """(slabs, feature tiles) for steps of more than MAX_ROWS and up to SHARED_ROWS_MOST single tokens: slabs
        from the kernel that shares the rows (one tile a wave: -1), or (0, 1) for the library."""
        chunks = weight.shape[1] // 32
        if not self.decode_ok or self.hidden % 4 != 0 or FORCE_SPLIT == 0 or chunks < 4:
            return 0, 1
        if FORCE_SPLIT:
            return (FORCE_SPLIT, -1) if FORCE_SHARED_ROWS and chunks >= FORCE_SPLIT else (0, 1)
        if weight.numel() < LIBRARY_MIN_WEIGHT or not self.measure or FORCE_LIBRARY is not None:
            return 0, 1
        key = (tuple(weight.shape), bias is None, BEYOND, True, 1)
        if key not in _split_wins:
            _split_wins[key] = _measure_split(weight, bias, SHARED_ROWS_MOST, True, 1)
        return _split_wins[key]

    def _tune_all(self, weight: torch.Tensor, bias, epilogue: int, conv: Optional[dict], normed: bool) -> tuple:
        forced = 1 if FORCE_TILES is None else FORCE_TILES
        if FORCE_SHARED_ROWS and epilogue != ops.EPI_PLAIN and weight.shape[1] // 32 >= 4:
            forced = -FORCE_SHARED_ROWS
        fixed_tiles = tuple(forced if bucket in self.wide_buckets else 1 for bucket in range(BUCKETS))
        if (not self.general or FORCE_LIBRARY is False
                or (FORCE_LIBRARY is None and (weight.numel() < LIBRARY_MIN_WEIGHT or not self.measure))):
            return _each(False), fixed_tiles
        if FORCE_LIBRARY:
            return _each(True), fixed_tiles
        choices, tiles = [], []
        for bucket, rows in enumerate(TUNE_ROWS):
            wide = bucket in self.wide_buckets or not normed          # the plain prologue: a workgroup may own several tiles
            key = (tuple(weight.shape), epilogue, bias is None, bucket, wide)
            if key not in _library_wins:
                _library_wins[key] = _measure_library(weight, bias, rows, epilogue, 8, conv, wide)
            choices.append(_library_wins[key][0])
            tiles.append(_library_wins[key][1] if FORCE_TILES is None or bucket not in self.wide_buckets else FORCE_TILES)
        return tuple(choices), tuple(tiles)

    def forward_decode(self, residual: Residual, step, caches) -> None:
        M = step.num_tokens
        bucket = _bucket(M) if M <= MAX_ROWS else BEYOND
        kernel = self.kernel if (self.kernel is not None and step.max_query_len == 1
                                 and self.kernel.supported(step, caches)) else None
        conv = None
        if kernel is not None and kernel.conv is not None:
            conv = dict(kernel.conv, state=kernel.conv_state(caches), slot_ids=step.slot_ids)
        u = self._project_in(residual, M, bucket, conv)
        mixed = torch.empty((M, self.mixed_width), dtype=torch.bfloat16, device=u.device)
        attended = None
        if kernel is not None:
            later = (not self.library_out[bucket] and not self.split_out[bucket]
                     and self._merges_later(kernel, step, caches))
            attended = kernel.run(u, step, caches, mixed, merge=not later)
        else:
            self._mix_each(u, step, caches, mixed)
        self._after_the_mixers(residual, mixed, attended, M, bucket)

    def _norm_prologue(self, residual: Residual, M: int, norm, rms):
        """The input of a projection: the norm in the kernel's prologue, or its own kernel before."""
        if M > self.norm_rows or rms is None:
            return dict(x=norm.forward(residual)), None          # adds the pending deltas in place
        pending = residual.pending
        if len(pending) > 2 or any(delta.dtype != torch.bfloat16 for delta in pending):
            return dict(x=norm.forward(residual)), None
        h_out = torch.empty_like(residual.h) if pending else None
        arguments = dict(h_in=residual.h, deltas=pending, h_out=h_out, norm_weight=rms[0], eps=rms[1])
        return arguments, h_out

    def _add_to_the_stream(self, residual: Residual, x, weight, bias, fragments, next_weight, attended=None,
                           row_tiles: int = 1) -> None:
        """h += the projection, with the rows that the product behind the norm of ``next_weight`` reads."""
        M, device = x.shape[0], x.device
        rows = torch.empty((M, self.hidden), dtype=torch.bfloat16, device=device)
        ssq = ops.residual_workspace(M, self.hidden, device)
        if attended is not None:
            ops.fused_gemm_merge(weight, bias, None, x, attended, fragments, residual=(residual.h, rows, next_weight, ssq))
        else:
            ops.fused_gemm_residual(weight, bias, x, residual.h, rows, next_weight, ssq, fragments, row_tiles=row_tiles)
        residual.scaled = ScaledRows(rows, ssq, next_weight)

    def _behind_the_norm(self, scaled: ScaledRows, rms) -> dict:
        return dict(x=scaled.rows, row_scale=ops.RowScale(scaled.ssq, self.hidden, rms[1]))

    def _project_in(self, residual: Residual, M: int, bucket: int, conv: Optional[dict]) -> torch.Tensor:
        """1: the mixers' input projection of the normed rows (with the conv step of ``conv``'s columns)."""
        block = self.block
        device = residual.h.device
        epilogue = ops.EPI_CONV if conv is not None else ops.EPI_PLAIN
        scaled = residual.scaled
        if (scaled is not None and not self.library_in[bucket] and self.mixer_scale is not None
                and scaled.weight is self.mixer_scale[0] and not residual.pending):
            # the layer before left the stream prepared for this norm
            u = torch.empty((M, self.in_ld), dtype=torch.bfloat16, device=device)
            ops.fused_gemm(self.w_in, self.b_in, u[:, :self.in_width], epilogue=epilogue, conv=conv,
                           fragments=self.f_in, **_tiles(self.tiles_in[bucket], self.rows_in[bucket]),
                           **self._behind_the_norm(scaled, self.mixer_scale))
        elif self.library_in[bucket]:
            u = ops.linear(block.mixer_norm.forward(residual), self.w_in, self.b_in)
            if conv is not None:
                ops.conv_step(u, conv["lo"], conv["hi"] - conv["lo"], conv["weight"], conv["bias"], conv["state"],
                              conv["slot_ids"])
        else:
            u = torch.empty((M, self.in_ld), dtype=torch.bfloat16, device=device)
            arguments, h_out = self._norm_prologue(residual, M, block.mixer_norm, self.mixer_rms)
            ops.fused_gemm(self.w_in, self.b_in, u[:, :self.in_width], epilogue=epilogue, conv=conv,
                           fragments=self.f_in, **(_tiles(self.tiles_in[bucket]) if "x" in arguments else {}),
                           **arguments)
            if h_out is not None:
                residual.h, residual.pending = h_out, []
        return u

    def _after_the_mixers(self, residual: Residual, mixed: torch.Tensor, attended, M: int, bucket: int) -> None:
        """3 to 5: the output projection, the norm, the feed-forward.  (Whatever ran in 1 has added what was
        pending to the stream.)"""
        block = self.block
        # 3
        if self.deferred[bucket] and not residual.pending:
            self._add_to_the_stream(residual, mixed, self.w_out, self.b_out, self.f_out, self.ffn_scale[0], attended,
                                    self.rows_out[bucket])
        else:
            residual.pending = self._to_the_stream(mixed, self.w_out, self.b_out, self.library_out[bucket],
                                                   self.split_out[bucket], self.tiles_out[bucket], self.f_out, attended)
        # 4
        if self.gate_up is None:
            residual.pending = [block.ffn.forward(block.ffn_norm.forward(residual))]
            return
        activated = torch.empty((M, self.inner), dtype=torch.bfloat16, device=mixed.device)
        scaled = residual.scaled
        if scaled is not None and (self.ffn_scale is None or scaled.weight is not self.ffn_scale[0]):
            scaled = None
        if scaled is not None:
            ops.fused_gemm(self.gate_up.weight, self.gate_up.bias, activated, epilogue=ops.EPI_SWIGLU,
                           fragments=self.f_gate_up, **_tiles(self.tiles_gate_up[bucket], self.rows_gate_up[bucket]),
                           **self._behind_the_norm(scaled, self.ffn_scale))
        elif self.library_gate_up[bucket]:
            ops.swiglu(ops.linear(block.ffn_norm.forward(residual), self.gate_up.weight, self.gate_up.bias), activated, 8)
        else:
            arguments, h_out = self._norm_prologue(residual, M, block.ffn_norm, self.ffn_rms)
            ops.fused_gemm(self.gate_up.weight, self.gate_up.bias, activated, epilogue=ops.EPI_SWIGLU,
                           fragments=self.f_gate_up, **(_tiles(self.tiles_gate_up[bucket]) if "x" in arguments else {}),
                           **arguments)
            if h_out is not None:
                residual.h, residual.pending = h_out, []
        # 5
        if scaled is not None and residual.next_norm is not None:
            self._add_to_the_stream(residual, activated, self.down.weight, self.down.bias, self.f_down,
                                    residual.next_norm[0], row_tiles=self.rows_down[bucket])
            return
        residual.pending = self._to_the_stream(activated, self.down.weight, self.down.bias, self.library_down[bucket],
                                               self.split_down[bucket], self.tiles_down[bucket], self.f_down)

    def _merges_later(self, kernel, step, caches) -> bool:
        """Whether the output projection merges the runs of keys of this step's attended heads itself."""
        estimate = getattr(kernel, "merge_later_bytes", None)
        rows = step.num_tokens
        if estimate is None or rows > MERGE_LATER_ROWS or FORCE_MERGE_LATER is False:
            return False
        merged = estimate(step, caches)                  # (merged columns, bytes of runs one workgroup reads)
        if merged is None or not ops.fused_gemm_merge_supported(rows, self.w_out.shape[1], 1, merged[0]):
            return False
        if FORCE_MERGE_LATER:
            return True
        return merged[1] <= MERGE_LATER_BYTES

    def _to_the_stream(self, x: torch.Tensor, weight: torch.Tensor, bias, library: bool, slabs: int, tiles: int,
                       fragments, attended=None) -> list:
        """A projection whose result is added to the residual stream: what the next norm will add, as one
        bfloat16 branch or as float32 partial sums over runs of K (views of one tensor, in order).
        ``attended``: the first columns of x are to be merged from these runs of keys."""
        M = x.shape[0]
        if attended is not None:
            delta = torch.empty((M, self.hidden), dtype=torch.bfloat16, device=x.device)
            ops.fused_gemm_merge(weight, bias, delta, x, attended, fragments)
            return [delta]
        if slabs and (M <= MAX_ROWS or (tiles < 0 and M <= SHARED_ROWS_MOST)):
            partial = torch.empty((slabs, M, self.hidden), dtype=torch.float32, device=x.device)
            ops.fused_gemm_split(weight, bias, x, partial, fragments=fragments, feature_tiles=abs(tiles),
                                 shared_rows=tiles < 0)
            return list(partial.unbind(0))
        if library or M > MAX_ROWS:
            return [ops.linear(x, weight, bias)]
        delta = torch.empty((M, self.hidden), dtype=torch.bfloat16, device=x.device)
        ops.fused_gemm(weight, bias, delta, x=x, feature_tiles=abs(tiles), fragments=fragments)
        return [delta]


def _tiles(tiles: int, rows: int = 1) -> dict:
    """A plan's number of feature tiles as the products' arguments: negative, that many a wave of the kernel that
    shares the rows.  ``rows``: over how many workgroups the step's rows are dealt out (the skinny kernel with one
    tile of features only)."""
    return dict(feature_tiles=abs(tiles), shared_rows=tiles < 0, row_tiles=rows if tiles == 1 else 1)


def _rms_prologue(norm):
    prologue = getattr(norm, "rms_prologue", None)
    return prologue() if prologue is not None else None


@register_mixer_kernel("attention", "mamba2")
def attention_mamba2_step(fusion: "LayerFusion") -> Optional["AttentionMamba2Step"]:
    attention, mamba = fusion.mixers
    a, s = attention.spec, mamba.spec
    fused_rotation = getattr(attention.position, "fused_rotation", None)
    if fused_rotation is None or fused_rotation() is None or attention.position.score_slopes is not None:
        _decline(f"the position encoding {type(attention.position).__name__} declares no rotation the decode kernel "
                 "applies (fused_rotation)")
        return None
    if a.head_dim not in (64, 128) or a.num_heads // a.num_kv_heads > 8 or s.state_size > 512:
        _decline(f"the decode kernel takes heads of 64 or 128 dimensions in groups of up to 8 and states of up to 512 "
                 f"columns, not {a.head_dim}, {a.num_heads // a.num_kv_heads} and {s.state_size}")
        return None
    return AttentionMamba2Step(fusion)


class AttentionMamba2Step:
    """Attention beside Mamba2 in steps of single tokens: the conv step of the state-space columns runs in the
    epilogue of the input product, and one launch (``mixer_decode``) rotates q and the new key, writes the new
    key and value into their cache cell, attends over the request's pages in runs that a small kernel merges,
    and advances the state-space state by one step with the gate on the way out."""

    def __init__(self, fusion: "LayerFusion"):
        self.attention, self.mamba = fusion.mixers
        self.attention_name, self.mamba_name = fusion.names
        a, s = self.attention.spec, self.mamba.spec
        q_width, kv_width = a.num_heads * a.head_dim, a.num_kv_heads * a.head_dim
        first, second = fusion.in_cols[0][0], fusion.in_cols[1][0]
        self.q_col, self.k_col, self.v_col = first, first + q_width, first + q_width + kv_width
        self.z_col = second
        self.x_col = second + s.inner_size
        self.dt_col = self.x_col + s.conv_width
        self.attended_width = q_width
        self.inv_freq, self.rotary_dim = self.attention.position.fused_rotation()
        self.conv = dict(lo=self.x_col, hi=self.dt_col, taps=s.conv_kernel, weight=self.mamba.conv_weight,
                         bias=self.mamba.conv_bias)

    def conv_state(self, caches) -> torch.Tensor:
        return caches[self.mamba_name].states["conv"]

    def supported(self, step, caches) -> bool:
        a = self.attention.spec
        cache = caches[self.attention_name]
        return (cache.owns_kv
                and ops.mixer_decode_supported(a.num_heads, a.num_kv_heads, a.head_dim, cache.k_cache.shape[2],
                                               self.mamba.spec.state_size, step.max_seq_len, a.window, self.rotary_dim))

    def merge_later_bytes(self, step, caches):
        """(columns of the attended heads, bytes of runs of keys a workgroup reads to merge them), or None."""
        a = self.attention.spec
        rows, page_size = step.num_tokens, caches[self.attention_name].k_cache.shape[2]
        span = max(1, int(step.max_seq_len)) if not a.window else a.window + page_size
        runs = ops.mixer_runs(rows, a.num_kv_heads, page_size, span)[1]
        return a.num_heads * a.head_dim, rows * a.num_heads * min(runs, ops.MERGE_AT_ONCE) * (a.head_dim + 2) * 4

    def run(self, u: torch.Tensor, step, caches, mixed: torch.Tensor, merge: bool = True):
        a, s = self.attention.spec, self.mamba.spec
        kv, state = caches[self.attention_name], caches[self.mamba_name]
        gated_norm = self.mamba.norm_weight is not None
        y = torch.empty((u.shape[0], s.inner_size), dtype=torch.float32, device=u.device) if gated_norm else None
        attended = ops.mixer_decode(
            u, num_heads=a.num_heads, num_kv_heads=a.num_kv_heads, head_dim=a.head_dim, q_col=self.q_col,
            k_col=self.k_col, v_col=self.v_col, inv_freq=self.inv_freq,
            rotary_dim=self.rotary_dim, k_cache=kv.k_cache, v_cache=kv.v_cache,
            block_tables=step.block_tables[kv.group], positions=step.positions,
            slot_mapping=step.slot_mappings[kv.group], scale=a.scale, window=a.window, max_seq_len=step.max_seq_len,
            ssm_heads=s.num_heads, ssm_head_dim=s.head_dim, state_size=s.state_size,
            num_groups=s.num_groups, z_col=self.z_col, x_col=self.x_col, dt_col=self.dt_col,
            dt_bias=self.mamba.dt_bias, A=self.mamba.A, D=self.mamba.D, ssm_state=state.states["ssm"],
            slot_ids=step.slot_ids, out=mixed, ssm_y=y, merge=merge)
        if gated_norm:
            ops.gate_norm(y, u[:, self.z_col:self.z_col + s.inner_size], self.mamba.norm_weight, s.num_groups,
                          s.norm_eps, mixed[:, self.attended_width:])
        return attended


def _cat_bias(linears, device):
    if all(linear.bias is None for linear in linears):
        return None
    return torch.cat([torch.zeros(linear.out_features, dtype=torch.float32, device=device)
                      if linear.bias is None else linear.bias for linear in linears]).contiguous()
