"""The fast paths of a layer made of RMSNorm, attention, Mamba2 and SwiGLU.  The two mixers read
the same normed rows and their outputs are added, so their input projections are one matrix
[q|k|v|z|x B C|dt] and their output projections one matrix [Wo | W_out] along the inputs; the
parts' own matrices are views of these.

Any step in bfloat16 (prompt portions, mixed batches): norm, one input GEMM, the two mixers on
column views of its output, one output GEMM, norm, feed-forward: two library GEMMs fewer than
part by part.

Decode steps (every lane holds one token, at most 64 rows): five launches instead of fifteen
(seven for batches of more than 16 rows, whose two norms run as kernels of their own)

    1. residual add + norm + [q|k|v|z|x B C|dt] projection + conv step        (fused_gemm)
    2. attention (rotation, cache write, split context) and SSM step           (mixer_decode)
    3. [attention | ssm] . [Wo | W_out]^T                                       (fused_gemm)
    4. residual add + norm + gate/up projection + SiLU(g)*u                     (fused_gemm)
    5. down projection                                                          (fused_gemm)

A large weight goes through the BLAS library instead where that is faster (``LIBRARY_MIN_WEIGHT``); the
conv step and SiLU(g)*u then run as kernels of their own.

The fusion belongs to the arrangement, which knows its parts; the parts stay as they are.  It
is built only for bfloat16 weights and sizes the kernels cover; otherwise the block runs part
by part.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .attention import Attention
from .base import Residual
from .ffn import SwiGLU
from .mamba2 import Mamba2
from .norm import RmsNorm
from .position import NoPosition, Rope

MAX_ROWS = 64          # rows of a step the skinny kernels take
MAX_NORM_ROWS = 16     # the norm prologue recomputes the normed rows in every workgroup: small batches only
# A weight of this many elements or more is measured once, when the first layer of its shape is built, on
# both ways: the skinny kernel, and the BLAS library with the conv step or SiLU(g)*u as a kernel of its own.
# The skinny kernel reads the step's rows once per 16 weight rows and keeps all of K in one workgroup; the
# library tiles the rows and splits a long K, but its choice of tile swings from shape to shape (a 5120 x
# 21504 weight at 8 rows: 115 us against 69; a 3072 x 12288 one: 20 against 25), so the clock decides, per
# shape and per step size (up to 16, 32, 64 rows).  Below the limit the skinny kernel wins everywhere.
LIBRARY_MIN_WEIGHT = 2 << 20
LIBRARY_MARGIN = 0.92          # the library has to be this much faster to be taken
FORCE_LIBRARY: Optional[bool] = None      # tests: True or False instead of the clock
TUNE_ROWS = (8, 32, 64)
_library_wins: Dict[tuple, tuple] = {}
# An output or down projection at 32 to 64 rows has a long K and few output features: 64 workgroups of the
# skinny kernel, or whatever tile the library picks (10.7 us for 1,024 x 2,048 at 64 rows).  Split over K into
# float32 slabs that the next norm adds up, the skinny kernel fills the GPU (7.5 us with 2 slabs; at 32 rows 5.2 us against the library's 9.6).  Measured
# at build like the library; the split has to win by SPLIT_MARGIN, for the norm reads the slabs.
SPLIT_CHOICES = (2, 4, 8)
SPLIT_MARGIN = 0.85
FORCE_SPLIT: Optional[int] = None         # tests: a number of slabs (0 = never) instead of the clock
_split_wins: Dict[tuple, tuple] = {}
# Beyond 16 rows the skinny kernel's workgroup may own 2 or 4 tiles of 16 output features instead of one: the
# step's rows then cross the caches half or a quarter as often, and fewer workgroups each keep more weight
# fragments in flight (a 5120 x 21504 weight at 32 rows: 135 us with one tile, 86 with two, the library 125).
# Measured with the rest, per shape and step size.
TILE_CHOICES = (1, 2, 4)
FORCE_TILES: Optional[int] = None         # tests: this many tiles for steps of more than 16 rows instead of the clock
# The library's tile for a prompt portion's input projection depends on the number of output features: 4 120
# of them (0.5B-shaped) take 30.5 us at 2,048 rows, 4 352 (a multiple of 256) take 23.6.  Measured at build in
# the same way; where padding pays, the prompt path multiplies with zero rows added and ignores their columns.
PAD_FEATURES = 256
PAD_ROWS = 2048
PAD_MARGIN = 0.95
FORCE_PADDING: Optional[bool] = None      # tests: True or False instead of the clock
_padding_wins: Dict[tuple, bool] = {}


OVERLAP_MIN_TOKENS = 256       # prompt portions from this size on run their two mixers on two streams
_side_streams: Dict[int, "torch.cuda.Stream"] = {}


def _side_stream(device: torch.device) -> "torch.cuda.Stream":
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index not in _side_streams:
        _side_streams[index] = torch.cuda.Stream(device=device)       # default priority
    return _side_streams[index]


def _bucket(rows: int) -> int:
    return 0 if rows <= MAX_NORM_ROWS else 1 if rows <= 32 else 2


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


def _padding_pays(weight: torch.Tensor) -> bool:
    """Whether rows of zeros up to a multiple of PAD_FEATURES make the library's product of a prompt portion faster."""
    N, K = weight.shape
    if N % PAD_FEATURES == 0 or FORCE_PADDING is False:
        return False
    if FORCE_PADDING:
        return True
    if weight.numel() < LIBRARY_MIN_WEIGHT:
        return False
    key = (N, K)
    if key not in _padding_wins:
        x = torch.full((PAD_ROWS, K), 0.01, dtype=torch.bfloat16, device=weight.device)
        padded = torch.cat([weight, weight.new_zeros((-N % PAD_FEATURES, K))])

        def plain():
            for _ in range(4):
                torch.matmul(x, weight.t())

        def wide():
            for _ in range(4):
                torch.matmul(x, padded.t())

        _padding_wins[key] = _graph_microseconds(wide) < PAD_MARGIN * _graph_microseconds(plain)
    return _padding_wins[key]


def _measure_split(weight: torch.Tensor, bias, rows: int, library: bool, tiles: int) -> tuple:
    """(slabs, feature tiles): the number of float32 slabs over K with which the skinny kernel beats the way this
    projection would go otherwise (the library, or the skinny kernel unsplit) at this many rows, or 0."""
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
    for slabs in SPLIT_CHOICES:
        if K // 32 < slabs:
            continue
        partial = torch.empty((slabs, rows, N), dtype=torch.float32, device=device)
        for split_tiles in TILE_CHOICES[:2]:

            def split():
                for w, f in zip(weights, fragments):
                    ops.fused_gemm_split(w, bias, x, partial, feature_tiles=split_tiles, fragments=f)

            time = _graph_microseconds(split)
            if time < best_time:
                best, best_time = (slabs, split_tiles), time
    return best


def _measure_library(weight: torch.Tensor, bias, rows: int, epilogue: int, tile: int, conv: Optional[dict]) -> tuple:
    """(whether the library way is faster for this weight at this many rows, the skinny kernel's best number
    of feature tiles).  Copies of the weight are cycled through so that the caches do not hold it, as in a
    model of many layers."""
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

    times = {tiles: _graph_microseconds(skinny(tiles)) for tiles in (TILE_CHOICES if rows > MAX_NORM_ROWS else (1,))}
    tiles = min(times, key=times.get)
    return _graph_microseconds(library) < LIBRARY_MARGIN * times[tiles], tiles


class ParallelFusion:
    @staticmethod
    def build(block, build) -> Optional["ParallelFusion"]:
        if build.dtype != torch.bfloat16 or build.device.type != "cuda":
            return None
        mixers = dict(block.mixers)
        if len(mixers) != 2:
            return None
        attention = next((m for m in mixers.values() if type(m) is Attention), None)
        mamba = next((m for m in mixers.values() if type(m) is Mamba2), None)
        if attention is None or mamba is None or type(block.ffn) is not SwiGLU:
            return None
        if type(block.mixer_norm) is not RmsNorm or type(block.ffn_norm) is not RmsNorm:
            return None
        if type(attention.position) not in (Rope, NoPosition):
            return None
        linears = [attention.qkv, attention.out, mamba.in_proj, mamba.out_proj, block.ffn.gate_up, block.ffn.down]
        if any(linear.weight.dtype != torch.bfloat16 for linear in linears):
            return None
        a, s = attention.spec, mamba.spec
        hidden = build.hidden_size
        inner = block.ffn.spec.intermediate_size
        mixed_width = a.num_heads * a.head_dim + s.inner_size
        if a.head_dim not in (64, 128) or a.num_heads // a.num_kv_heads > 8 or s.state_size > 512:
            return None
        if block.ffn.tile != 8 or hidden % 32 != 0 or mixed_width % 32 != 0 or inner % 32 != 0:
            return None
        if not (ops.fused_gemm_supported(False, 1, hidden) and ops.fused_gemm_supported(False, 1, mixed_width)
                and ops.fused_gemm_supported(False, 1, inner)):
            return None
        return ParallelFusion(block, attention, mamba, build)

    def __init__(self, block, attention: Attention, mamba: Mamba2, build):
        self.block = block
        self.attention = attention
        self.mamba = mamba
        self.attention_name = next(name for name, mixer in block.mixers if mixer is attention)
        self.mamba_name = next(name for name, mixer in block.mixers if mixer is mamba)
        device = build.device
        a, s = attention.spec, mamba.spec
        self.hidden = build.hidden_size
        q_width, kv_width = a.num_heads * a.head_dim, a.num_kv_heads * a.head_dim
        E, C = s.inner_size, s.conv_width
        # 1: [q | k | v | z | x B C | dt]
        self.w_in = torch.cat([attention.qkv.weight, mamba.in_proj.weight], dim=0).contiguous()
        self.b_in = _cat_bias([attention.qkv, mamba.in_proj], device)
        # prompt portions may multiply with rows of zeros added (the decode kernels take the rows that count)
        self.w_in_wide, self.b_in_wide = self.w_in, self.b_in
        if _padding_pays(self.w_in):
            extra = -self.w_in.shape[0] % PAD_FEATURES
            self.w_in_wide = torch.cat([self.w_in, self.w_in.new_zeros((extra, self.w_in.shape[1]))])
            self.w_in = self.w_in_wide[:self.w_in.shape[0]]
            if self.b_in is not None:
                self.b_in_wide = torch.cat([self.b_in, self.b_in.new_zeros(extra)])
        self.q_col, self.k_col, self.v_col = 0, q_width, q_width + kv_width
        self.z_col = q_width + 2 * kv_width
        self.x_col = self.z_col + E
        self.dt_col = self.x_col + C
        self.in_width = self.w_in.shape[0]
        self.in_ld = -(-self.in_width // 8) * 8
        self.qkv_width = q_width + 2 * kv_width
        attention.qkv.weight = self.w_in[:self.qkv_width]             # the parts' matrices: views of the fused ones
        mamba.in_proj.weight = self.w_in[self.qkv_width:]
        # 3: [attention | ssm] . [Wo | W_out]^T
        self.w_out = torch.cat([attention.out.weight, mamba.out_proj.weight], dim=1).contiguous()
        biases = [linear.bias for linear in (attention.out, mamba.out_proj) if linear.bias is not None]
        self.b_out = sum(biases[1:], biases[0]).contiguous() if biases else None
        self.mixed_width = q_width + E
        self.q_width = q_width
        attention.out.weight = self.w_out[:, :q_width]
        mamba.out_proj.weight = self.w_out[:, q_width:]
        # the column views the mixers get must start at 16 bytes and rows must be multiples of 8 elements
        self.general = (self.in_width % 8 == 0 and self.qkv_width % 8 == 0 and q_width % 8 == 0
                        and self.mixed_width % 8 == 0)
        # 4: gate and up rows interleaved in tiles of 8: the feed-forward part stores them so
        ffn = block.ffn
        inner = ffn.spec.intermediate_size
        self.w_gate_up = ffn.gate_up.weight
        self.b_gate_up = ffn.gate_up.bias
        self.inner = inner
        self.position = attention.position
        # a wide model's normed rows do not fit the norm prologue's LDS: its norms then run as kernels of their own
        self.norm_fits = ops.fused_gemm_supported(True, 1, self.hidden)
        # which projections go through the library, by step size
        conv = dict(lo=self.x_col, hi=self.dt_col, taps=s.conv_kernel, weight=mamba.conv_weight, bias=mamba.conv_bias)
        # (and how many tiles of 16 output features a workgroup of the skinny kernel owns where it is taken)
        self.library_in, self.tiles_in = self._tune(self.w_in, self.b_in, ops.EPI_CONV, conv)
        self.library_out, self.tiles_out = self._tune(self.w_out, self.b_out, ops.EPI_PLAIN)
        self.library_gate_up, self.tiles_gate_up = self._tune(self.w_gate_up, self.b_gate_up, ops.EPI_SWIGLU)
        self.library_down, self.tiles_down = self._tune(ffn.down.weight, ffn.down.bias, ops.EPI_PLAIN)
        # and which of the two that feed the residual stream are split over K instead (steps of more than 16 rows)
        self.split_out, self.tiles_out = self._tune_split(self.w_out, self.b_out, self.library_out, self.tiles_out)
        self.split_down, self.tiles_down = self._tune_split(ffn.down.weight, ffn.down.bias, self.library_down,
                                                            self.tiles_down)
        # what the skinny kernel reads: a second copy of each matrix in the order of its waves' fragments (one run
        # of 1 KiB a load instead of 64 bytes of each of 16 rows: 15 to 25 % faster); the row-major ones stay for
        # the library and for prompt portions.  A projection that always goes through the library has none.

        def fragments(weight, library, split):
            return None if all(library) and not any(split) else ops.fragment_order(weight)

        self.f_in = fragments(self.w_in, self.library_in, ())
        self.f_out = fragments(self.w_out, self.library_out, self.split_out)
        self.f_gate_up = fragments(self.w_gate_up, self.library_gate_up, ())
        self.f_down = fragments(ffn.down.weight, self.library_down, self.split_down)

    def decode_supported(self, step, cache) -> bool:
        a = self.attention.spec
        rotary = self.position.rotary_dim if isinstance(self.position, Rope) else 0
        return (step.max_query_len == 1 and step.num_tokens <= MAX_ROWS and cache.owns_kv
                and ops.mixer_decode_supported(a.num_heads, a.num_kv_heads, a.head_dim, cache.k_cache.shape[2],
                                               self.mamba.spec.state_size, step.max_seq_len, a.window, rotary))

    def forward(self, residual: Residual, step, caches) -> bool:
        """Runs the layer and returns True, or returns False with nothing done (the block then
        runs part by part)."""
        if self.decode_supported(step, caches[self.attention_name]):
            self.forward_decode(residual, step, caches)
            return True
        if self.general:
            self.forward_general(residual, step, caches)
            return True
        return False

    def forward_general(self, residual: Residual, step, caches) -> None:
        block = self.block
        normed = block.mixer_norm.forward(residual)
        u = ops.linear(normed, self.w_in_wide, self.b_in_wide)
        mixed = torch.empty((u.shape[0], self.mixed_width), dtype=u.dtype, device=u.device)
        if u.shape[0] >= OVERLAP_MIN_TOKENS and torch.cuda.is_current_stream_capturing():
            # the two mixers read the same rows and write different columns: attention runs on a second
            # stream beside the state-space chain, whose kernels are many and small (in a captured graph
            # only: launched one by one the step waits for the host, which the second stream costs more).
            # The chain is recorded first: the graph keeps the branch it meets first on the queue of the
            # projections before and after it, and the other branch pays the hops between queues
            main = torch.cuda.current_stream(u.device)
            side = _side_stream(u.device)
            side.wait_stream(main)
            self.mamba.mix(u[:, self.qkv_width:self.in_width], step, caches[self.mamba_name], mixed[:, self.q_width:])
            with torch.cuda.stream(side):
                self.attention.mix(u[:, :self.qkv_width], step, caches[self.attention_name], mixed[:, :self.q_width])
            main.wait_stream(side)
        else:
            self.attention.mix(u[:, :self.qkv_width], step, caches[self.attention_name], mixed[:, :self.q_width])
            self.mamba.mix(u[:, self.qkv_width:self.in_width], step, caches[self.mamba_name], mixed[:, self.q_width:])
        residual.pending = [ops.linear(mixed, self.w_out, self.b_out)]
        normed = block.ffn_norm.forward(residual)
        residual.pending = [block.ffn.forward(normed)]

    def _tune(self, weight: torch.Tensor, bias, epilogue: int, conv: Optional[dict] = None) -> tuple:
        """For step sizes of up to 16, 32 and 64 rows: whether this projection goes through the library, and
        the feature tiles of the skinny kernel.  (Where the norm runs in the skinny kernel's prologue, small
        steps stay with it.)"""
        choices, tiles = self._tune_all(weight, bias, epilogue, conv)
        if epilogue != ops.EPI_PLAIN and self.norm_fits:
            choices = (False,) + choices[1:]
        return choices, tiles

    def _tune_split(self, weight: torch.Tensor, bias, library: tuple, tiles: tuple) -> tuple:
        """For step sizes of up to 16, 32 and 64 rows: the number of slabs over K, or 0 for the whole product,
        and the feature tiles that go with it.  Steps of up to 16 rows feed the next kernel's norm prologue,
        which takes whole rows."""
        if self.hidden % 4 != 0 or FORCE_SPLIT == 0:
            return (0, 0, 0), tiles
        if FORCE_SPLIT:
            slabs = FORCE_SPLIT if weight.shape[1] // 32 >= FORCE_SPLIT else 0
            return (0, slabs, slabs), tiles
        if weight.numel() < LIBRARY_MIN_WEIGHT:
            return (0, 0, 0), tiles
        slabs, split_tiles = [0], [tiles[0]]
        for bucket in (1, 2):
            key = (tuple(weight.shape), bias is None, bucket, library[bucket], tiles[bucket])
            if key not in _split_wins:
                _split_wins[key] = _measure_split(weight, bias, TUNE_ROWS[bucket], library[bucket], tiles[bucket])
            slabs.append(_split_wins[key][0])
            split_tiles.append(_split_wins[key][1])
        return tuple(slabs), tuple(split_tiles)

    def _tune_all(self, weight: torch.Tensor, bias, epilogue: int, conv: Optional[dict]) -> tuple:
        forced = 1 if FORCE_TILES is None else FORCE_TILES
        fixed_tiles = (1, forced, forced)
        if not self.general or FORCE_LIBRARY is False or (FORCE_LIBRARY is None and weight.numel() < LIBRARY_MIN_WEIGHT):
            return (False, False, False), fixed_tiles
        if FORCE_LIBRARY:
            return (True, True, True), fixed_tiles
        choices, tiles = [], []
        for bucket, rows in enumerate(TUNE_ROWS):
            key = (tuple(weight.shape), epilogue, bias is None, bucket)
            if key not in _library_wins:
                _library_wins[key] = _measure_library(weight, bias, rows, epilogue, self.block.ffn.tile, conv)
            choices.append(_library_wins[key][0])
            tiles.append(_library_wins[key][1] if FORCE_TILES is None or bucket == 0 else FORCE_TILES)
        return tuple(choices), tuple(tiles)

    def forward_decode(self, residual: Residual, step, caches) -> None:
        block, a, s = self.block, self.attention.spec, self.mamba.spec
        kv, state = caches[self.attention_name], caches[self.mamba_name]
        M = step.num_tokens
        bucket = _bucket(M)
        device = residual.h.device
        bf16 = torch.bfloat16

        def norm_prologue(norm):
            """The input of a projection: the norm in the kernel's prologue, or its own kernel before."""
            if M > MAX_NORM_ROWS or not self.norm_fits:
                return dict(x=norm.forward(residual)), None          # adds the pending deltas in place
            pending = residual.pending
            h_out = torch.empty_like(residual.h) if pending else None
            arguments = dict(h_in=residual.h, deltas=pending, h_out=h_out, norm_weight=norm.weight, eps=norm.eps)
            return arguments, h_out

        # 1
        if self.library_in[bucket]:
            u = ops.linear(block.mixer_norm.forward(residual), self.w_in, self.b_in)
            ops.conv_step(u, self.x_col, self.dt_col - self.x_col, self.mamba.conv_weight, self.mamba.conv_bias,
                          state.states["conv"], step.slot_ids)
        else:
            u = torch.empty((M, self.in_ld), dtype=bf16, device=device)
            arguments, h_out = norm_prologue(block.mixer_norm)
            ops.fused_gemm(self.w_in, self.b_in, u[:, :self.in_width], epilogue=ops.EPI_CONV,
                           conv=dict(lo=self.x_col, hi=self.dt_col, taps=s.conv_kernel, weight=self.mamba.conv_weight,
                                     bias=self.mamba.conv_bias, state=state.states["conv"], slot_ids=step.slot_ids),
                           feature_tiles=self.tiles_in[bucket] if "x" in arguments else 1, fragments=self.f_in,
                           **arguments)
            if h_out is not None:
                residual.h, residual.pending = h_out, []
        # 2
        mixed = torch.empty((M, self.mixed_width), dtype=bf16, device=device)
        gated_norm = self.mamba.norm_weight is not None
        y = torch.empty((M, s.inner_size), dtype=torch.float32, device=device) if gated_norm else None
        rope = isinstance(self.position, Rope)
        ops.mixer_decode(
            u, num_heads=a.num_heads, num_kv_heads=a.num_kv_heads, head_dim=a.head_dim, q_col=self.q_col,
            k_col=self.k_col, v_col=self.v_col, inv_freq=self.position.inv_freq if rope else None,
            rotary_dim=self.position.rotary_dim if rope else 0, k_cache=kv.k_cache, v_cache=kv.v_cache,
            block_tables=step.block_tables[kv.group], positions=step.positions,
            slot_mapping=step.slot_mappings[kv.group], scale=a.scale, window=a.window, max_seq_len=step.max_seq_len,
            ssm_heads=s.num_heads, ssm_head_dim=s.head_dim, state_size=s.state_size,
            num_groups=s.num_groups, z_col=self.z_col, x_col=self.x_col, dt_col=self.dt_col,
            dt_bias=self.mamba.dt_bias, A=self.mamba.A, D=self.mamba.D, ssm_state=state.states["ssm"],
            slot_ids=step.slot_ids, out=mixed, ssm_y=y)
        if gated_norm:
            ops.gate_norm(y, u[:, self.z_col:self.z_col + s.inner_size], self.mamba.norm_weight, s.num_groups,
                          s.norm_eps, mixed[:, a.num_heads * a.head_dim:])
        # 3
        residual.pending = self._to_the_stream(mixed, self.w_out, self.b_out, self.library_out[bucket],
                                               self.split_out[bucket], self.tiles_out[bucket], self.f_out)
        # 4
        activated = torch.empty((M, self.inner), dtype=bf16, device=device)
        if self.library_gate_up[bucket]:
            ops.swiglu(ops.linear(block.ffn_norm.forward(residual), self.w_gate_up, self.b_gate_up), activated,
                       block.ffn.tile)
        else:
            arguments, h_out = norm_prologue(block.ffn_norm)
            ops.fused_gemm(self.w_gate_up, self.b_gate_up, activated, epilogue=ops.EPI_SWIGLU,
                           feature_tiles=self.tiles_gate_up[bucket] if "x" in arguments else 1,
                           fragments=self.f_gate_up, **arguments)
            if h_out is not None:
                residual.h, residual.pending = h_out, []
        # 5
        down = block.ffn.down
        residual.pending = self._to_the_stream(activated, down.weight, down.bias, self.library_down[bucket],
                                               self.split_down[bucket], self.tiles_down[bucket], self.f_down)

    def _to_the_stream(self, x: torch.Tensor, weight: torch.Tensor, bias, library: bool, slabs: int, tiles: int,
                       fragments) -> list:
        """A projection whose result is added to the residual stream: what the next norm will add, as one
        bfloat16 branch or as float32 partial sums over runs of K (views of one tensor, in order)."""
        M = x.shape[0]
        if slabs:
            partial = torch.empty((slabs, M, self.hidden), dtype=torch.float32, device=x.device)
            ops.fused_gemm_split(weight, bias, x, partial, feature_tiles=tiles, fragments=fragments)
            return list(partial.unbind(0))
        if library:
            return [ops.linear(x, weight, bias)]
        delta = torch.empty((M, self.hidden), dtype=torch.bfloat16, device=x.device)
        ops.fused_gemm(weight, bias, delta, x=x, feature_tiles=tiles, fragments=fragments)
        return [delta]


def _cat_bias(linears, device):
    if all(linear.bias is None for linear in linears):
        return None
    return torch.cat([torch.zeros(linear.out_features, dtype=torch.float32, device=device)
                      if linear.bias is None else linear.bias for linear in linears]).contiguous()
