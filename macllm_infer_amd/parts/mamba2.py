"""Mamba2 state-space mixer with its per-request conv tail and SSM state."""
from __future__ import annotations

import torch

from ..cache.manager import StateNeed
from ..kernels import ops
from ..kernels.limits import CONV_MAX_TAPS, GRID_MOST, SCAN_MAX_STATE, beyond
from ..weights.loader import Expect
from .base import BuildContext, Mixer, register_part
from .linear import Linear


@register_part("mamba2")
class Mamba2(Mixer):
    """in_proj -> [z | x | B | C | dt] -> causal depthwise conv + SiLU over [x|B|C] (tail from
    the request's slot) -> selective scan from and into the slot's float32 state, D skip
    -> * SiLU(z) -> optional grouped RMSNorm -> out_proj.
    (reference: src/decoder.rs:2175 in_proj, :2203-2209 split, :2211-2253 conv,
    :2295-2349 scan, :2350-2367 gate and norm, :2368-2371 out_proj, :2373-2399 state.)

    The decay is stored as ``A_log`` and used as A = -exp(A_log).  ``multipliers`` scale the
    five segments of in_proj's output (after its bias), ``in_multiplier`` its input,
    ``out_multiplier`` out_proj's output; all are folded into the weights."""
    graph_safe = True
    CHUNKED_FROM = 8        # the longest lane of a step has at least this many tokens
    kernel_modules = ("common", "mamba2", "ssd", "gemm")

    @classmethod
    def expected_tensors(cls, spec, prefix: str, hidden_size: int):
        out = [Expect(f"{prefix}.in_proj.weight", ((spec.projection_width, hidden_size),)),
               Expect(f"{prefix}.conv1d.weight", ((spec.conv_width, spec.conv_kernel),
                                                  (spec.conv_width, 1, spec.conv_kernel)), init="conv"),
               Expect(f"{prefix}.dt_bias", ((spec.num_heads,),), init="dt_bias"),
               Expect(f"{prefix}.A_log", ((spec.num_heads,), (spec.num_heads, 1)), init="A_log"),
               Expect(f"{prefix}.D", ((spec.num_heads,), (spec.num_heads, 1)), init="D"),
               Expect(f"{prefix}.out_proj.weight", ((hidden_size, spec.inner_size),))]
        if spec.conv_bias:
            out.append(Expect(f"{prefix}.conv1d.bias", ((spec.conv_width,),), init="bias"))
        if spec.proj_bias:
            out += [Expect(f"{prefix}.in_proj.bias", ((spec.projection_width,),), init="bias"),
                    Expect(f"{prefix}.out_proj.bias", ((hidden_size,),), init="bias")]
        if spec.gated_norm:
            out.append(Expect(f"{prefix}.norm.weight",
                              ((spec.num_groups, spec.inner_size // spec.num_groups), (spec.inner_size,)),
                              init="norm"))
        return out

    @classmethod
    def limits(cls, spec, hidden_size: int):
        return (beyond("mamba2", "conv_kernel", spec.conv_kernel, CONV_MAX_TAPS, "the taps of a channel are kept in registers")
                + beyond("mamba2", "state_size", spec.state_size, SCAN_MAX_STATE, "a state row is spread over one wave")
                + beyond("mamba2", "num_heads", spec.num_heads, GRID_MOST, "heads index a dimension of the launch")
                + beyond("mamba2", "num_groups", spec.num_groups, GRID_MOST, "groups index a dimension of the launch"))

    @classmethod
    def cache_needs(cls, spec):
        return [StateNeed("conv", (spec.conv_kernel - 1, spec.conv_width), "activation"),
                StateNeed("ssm", (spec.num_heads, spec.head_dim, spec.state_size), "float32")]

    def __init__(self, spec, prefix: str, tensors, build: BuildContext):
        self.spec = spec
        self.build = build
        device = build.device
        get = lambda name: tensors.get(f"{prefix}.{name}")
        E, GN, H = spec.inner_size, spec.num_groups * spec.state_size, spec.num_heads
        m = spec.multipliers
        segment = torch.cat([torch.full((E,), m[0]), torch.full((E,), m[1]), torch.full((GN,), m[2]),
                             torch.full((GN,), m[3]), torch.full((H,), m[4])])
        self.in_proj = Linear([get("in_proj.weight")], [get("in_proj.bias")], build,
                              weight_scale=segment * spec.in_multiplier, bias_scale=segment)
        self.out_proj = Linear([get("out_proj.weight")], [get("out_proj.bias")], build,
                               weight_scale=spec.out_multiplier, bias_scale=spec.out_multiplier)
        f32 = lambda tensor: tensor.to(torch.float32).contiguous().to(device)
        self.conv_weight = f32(get("conv1d.weight").reshape(spec.conv_width, spec.conv_kernel))
        self.conv_bias = f32(get("conv1d.bias")) if spec.conv_bias else None
        self.dt_bias = f32(get("dt_bias"))
        self.A = f32(-torch.exp(get("A_log").to(torch.float32).reshape(H)))
        self.D = f32(get("D").reshape(H))
        self.norm_weight = f32(get("norm.weight").reshape(E)) if spec.gated_norm else None
        self._chunks_supported = None
        self.chunk_tokens = spec.chunk_size          # the step's chunk table that the chunked scan reads

    def _chunked(self, u: torch.Tensor, step) -> bool:
        """Prompt portions in bfloat16 scan in chunks on the matrix cores; single tokens, float32
        and sizes the chunked kernels do not take scan token by token."""
        spec = self.spec
        if u.dtype != torch.bfloat16 or step.max_query_len < self.CHUNKED_FROM:
            return False
        if self._chunks_supported is None:
            self._chunks_supported = ops.ssd_supported(spec.chunk_size, spec.head_dim, spec.state_size,
                                                       spec.num_groups, spec.inner_size)
        return self._chunks_supported

    def _chunk_table(self, step):
        """The step's own table of chunks, or (a step that was packed without one) one made from its lanes."""
        table = step.chunk_tables.get(self.spec.chunk_size)
        if table is not None:
            return table
        key = ("ssd_chunks", self.spec.chunk_size)
        if key not in step.derived:
            step.derived[key] = ops.SsdChunks(step.lane_lengths, self.spec.chunk_size, step.token_ids.device)
        return step.derived[key]

    def projections(self):
        return self.in_proj, self.out_proj, self.spec.inner_size

    def forward(self, x: torch.Tensor, step, cache) -> torch.Tensor:
        u = self.in_proj(x)                                               # [T, E + C + H]
        gated = torch.empty((x.shape[0], self.spec.inner_size), dtype=u.dtype, device=u.device)
        self.mix(u, step, cache, gated)
        return self.out_proj(gated)

    def mix(self, u: torch.Tensor, step, cache, gated: torch.Tensor) -> None:
        """From the projected rows [z | x B C | dt] to the gated (and normed) scan output
        ``gated`` [T, E]; both may be column views of wider matrices."""
        spec = self.spec
        E, C = spec.inner_size, spec.conv_width
        T = u.shape[0]
        conv_state, ssm_state = cache.states["conv"], cache.states["ssm"]
        chunked = self._chunked(u, step)
        raw = u[:, E:E + C]
        xbc = raw if step.max_query_len == 1 and not chunked else torch.empty((T, C), dtype=u.dtype, device=u.device)
        conv = None
        if chunked and ops.ssd_conv_supported(spec.conv_kernel, C, raw):
            # the chunked scan runs the conv and the tail update in its own launches
            conv = dict(u=raw, weight=self.conv_weight, bias=self.conv_bias, state=conv_state)
        elif step.max_query_len == 1:
            # single tokens: the conv step in place and the tail rolled by one, in one launch (the same products in
            # the same order as the two kernels below give for a lane of one token)
            ops.conv_step(u, E, C, self.conv_weight, self.conv_bias, conv_state, step.slot_ids)
            xbc = raw
        else:
            ops.conv1d_silu(u, E, C, self.conv_weight, self.conv_bias, conv_state, step.lane_of_token,
                            step.cu_seqlens, step.slot_ids, xbc)
            ops.conv_state_update(u, E, C, spec.conv_kernel, conv_state, step.cu_seqlens, step.slot_ids)
        if chunked:
            arguments = (xbc, u[:, E + C:], self.dt_bias, self.A, self.D, ssm_state, self._chunk_table(step),
                         step.slot_ids, spec.num_groups)
            if self.norm_weight is None and u.stride(0) % 4 == 0 and gated.stride(0) % 4 == 0:
                ops.ssd_prefill(*arguments, None, z=u[:, :E], gated=gated, conv=conv)      # the gate on the scan's way out
                return
            y = torch.empty((T, E), dtype=torch.float32, device=u.device)
            ops.ssd_prefill(*arguments, y, conv=conv)
        else:
            y = torch.empty((T, E), dtype=torch.float32, device=u.device)
            ops.ssm_scan(xbc, u[:, E + C:], self.dt_bias, self.A, self.D, ssm_state, step.cu_seqlens,
                         step.slot_ids, spec.num_groups, y, step.max_query_len)
        ops.gate_norm(y, u[:, :E], self.norm_weight, spec.num_groups, spec.norm_eps, gated)
