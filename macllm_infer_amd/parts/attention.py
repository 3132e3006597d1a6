"""Grouped-query causal attention over the paged cache."""
from __future__ import annotations

import torch

from ..cache.manager import KVNeed
from ..kernels import ops
from ..kernels.limits import ATTENTION_MAX_HEAD_DIM, GRID_MOST, beyond
from ..weights.loader import Expect
from .base import BuildContext, Mixer, part_class, register_part
from .linear import Linear


@register_part("attention")
class Attention(Mixer):
    """q, k, v projections (one fused product) -> position encoding of q and k -> K (encoded)
    and V written to the request's pages -> softmax(q.k * scale) . v over every visible
    cached key -> output projection.
    (reference: src/decoder.rs:1099-1161 projections, :953-962 RoPE and cache write,
    :4580-4670 scores with float32 softmax, :923-931 output; GQA pairing :4641-4647.)

    Multipliers: ``in_multiplier`` scales the input of q/k/v (folded into their weights),
    ``key_multiplier`` the k projection's output (weights and bias), ``out_multiplier``
    the output projection's output."""
    graph_safe = True
    kernel_modules = ("common", "attention", "gemm")
    query_tile = 64          # tokens of one lane that a workgroup of the prompt attention kernels takes

    @classmethod
    def expected_tensors(cls, spec, prefix: str, hidden_size: int):
        q_rows = spec.num_heads * spec.head_dim
        kv_rows = spec.num_kv_heads * spec.head_dim
        out = [Expect(f"{prefix}.q_proj.weight", ((q_rows, hidden_size),)),
               Expect(f"{prefix}.k_proj.weight", ((kv_rows, hidden_size),)),
               Expect(f"{prefix}.v_proj.weight", ((kv_rows, hidden_size),)),
               Expect(f"{prefix}.o_proj.weight", ((hidden_size, q_rows),))]
        if spec.qkv_bias:
            out += [Expect(f"{prefix}.q_proj.bias", ((q_rows,),), init="bias"),
                    Expect(f"{prefix}.k_proj.bias", ((kv_rows,),), init="bias"),
                    Expect(f"{prefix}.v_proj.bias", ((kv_rows,),), init="bias")]
        if spec.out_bias:
            out.append(Expect(f"{prefix}.o_proj.bias", ((hidden_size,),), init="bias"))
        return out

    @classmethod
    def limits(cls, spec, hidden_size: int):
        return (beyond("attention", "head_dim", spec.head_dim, ATTENTION_MAX_HEAD_DIM,
                       "a query row and its sums are kept in LDS and registers")
                + beyond("attention", "num_heads", spec.num_heads, GRID_MOST, "heads index a dimension of the launch")
                + part_class(spec.position).limits(spec.position, spec.head_dim))

    @classmethod
    def cache_needs(cls, spec):
        return [KVNeed(spec.num_kv_heads, spec.head_dim, spec.window)]

    def __init__(self, spec, prefix: str, tensors, build: BuildContext):
        self.spec = spec
        self.build = build
        q_rows = spec.num_heads * spec.head_dim
        kv_rows = spec.num_kv_heads * spec.head_dim
        get = lambda name: tensors.get(f"{prefix}.{name}")
        weight_scale = torch.cat([torch.full((q_rows,), spec.in_multiplier),
                                  torch.full((kv_rows,), spec.in_multiplier * spec.key_multiplier),
                                  torch.full((kv_rows,), spec.in_multiplier)])
        bias_scale = torch.cat([torch.ones(q_rows), torch.full((kv_rows,), spec.key_multiplier),
                                torch.ones(kv_rows)])
        self.qkv = Linear([get("q_proj.weight"), get("k_proj.weight"), get("v_proj.weight")],
                          [get("q_proj.bias"), get("k_proj.bias"), get("v_proj.bias")], build,
                          weight_scale=weight_scale, bias_scale=bias_scale)
        self.out = Linear([get("o_proj.weight")], [get("o_proj.bias")], build,
                          weight_scale=spec.out_multiplier, bias_scale=spec.out_multiplier)
        self.position = part_class(spec.position)(spec.position, spec.head_dim, build)
        self.graph_safe = bool(getattr(self.position, "graph_safe", False))

    def projections(self):
        return self.qkv, self.out, self.spec.num_heads * self.spec.head_dim

    def forward(self, x: torch.Tensor, step, cache) -> torch.Tensor:
        spec = self.spec
        attended = torch.empty((x.shape[0], spec.num_heads * spec.head_dim), dtype=x.dtype, device=x.device)
        self.mix(self.qkv(x), step, cache, attended)
        return self.out(attended)

    def mix(self, qkv: torch.Tensor, step, cache, attended: torch.Tensor) -> None:
        """From the projected rows [q | k | v] (rotated and stored in place) to the attended rows
        ``attended`` [T, Hq * dh]; both may be column views of wider matrices."""
        spec = self.spec
        self.position.rotate_and_store(qkv, spec.num_heads, spec.num_kv_heads, spec.head_dim, step, cache)
        geometry = (spec.num_heads, spec.num_kv_heads, spec.head_dim)
        slopes = self.position.score_slopes
        # lanes of several tokens: the general kernel shares a run of keys among the queries of a tile of the step's
        # table of runs (when the step was packed with one)
        tiles = {}
        if step.max_query_len > 1 and 0 < getattr(step, "query_tile", 0) < (1 << 20):
            tiles = dict(query_tiles=step.query_tiles, tile_tokens=step.query_tile, cu_seqlens=step.cu_seqlens)
        if slopes is not None:                           # a bias on the scores: the general kernel knows it
            ops.paged_attention(qkv, *geometry, cache.k_cache, cache.v_cache, step.block_tables[cache.group],
                                step.lane_of_token, step.positions, spec.scale, spec.window, attended,
                                step.max_seq_len, slopes, **tiles)
        elif step.max_query_len == 1 and ops.decode_attention_supported(qkv.dtype, *geometry, cache.k_cache.shape[2]):
            ops.decode_attention(qkv, *geometry, cache.k_cache, cache.v_cache, step.block_tables[cache.group],
                                 step.lane_of_token, step.positions, spec.scale, spec.window, step.max_seq_len,
                                 attended)
        elif ops.prefill_attention_supported(qkv.dtype, *geometry, cache.k_cache.shape[2]):
            ops.prefill_attention(qkv, *geometry, cache.k_cache, cache.v_cache, step.block_tables[cache.group],
                                  step.query_tiles, step.cu_seqlens, step.start_pos, spec.scale, spec.window,
                                  attended, step.max_seq_len)
        else:
            ops.paged_attention(qkv, *geometry, cache.k_cache, cache.v_cache, step.block_tables[cache.group],
                                step.lane_of_token, step.positions, spec.scale, spec.window, attended,
                                step.max_seq_len, **tiles)
