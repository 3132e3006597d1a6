"""Dense feed-forward parts."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import Expect
from .base import BuildContext, FeedForward, register_part
from .linear import Linear


@register_part("swiglu")
class SwiGLU(FeedForward):
    """down(SiLU(gate(x)) * up(x)); gate and up are one fused product
    (reference: src/decoder.rs:261-306).  ``gate_multiplier`` scales gate's output,
    ``down_multiplier`` down's output; both are folded into the weights.  When the width is a
    multiple of 8 the rows of the fused matrix are stored in tiles of 8 gate rows and 8 up rows
    (``tile``), the order the fused decode kernel wants, so that one matrix serves every path."""
    graph_safe = True
    kernel_modules = ("common", "gemm")

    @classmethod
    def expected_tensors(cls, spec, prefix: str, hidden_size: int):
        inner = spec.intermediate_size
        out = [Expect(f"{prefix}.gate_proj.weight", ((inner, hidden_size),)),
               Expect(f"{prefix}.up_proj.weight", ((inner, hidden_size),)),
               Expect(f"{prefix}.down_proj.weight", ((hidden_size, inner),))]
        if spec.bias:
            out += [Expect(f"{prefix}.gate_proj.bias", ((inner,),), init="bias"),
                    Expect(f"{prefix}.up_proj.bias", ((inner,),), init="bias"),
                    Expect(f"{prefix}.down_proj.bias", ((hidden_size,),), init="bias")]
        return out

    def __init__(self, spec, prefix: str, tensors, build: BuildContext):
        self.spec = spec
        inner = spec.intermediate_size
        get = lambda name: tensors.get(f"{prefix}.{name}")
        scale = torch.cat([torch.full((inner,), spec.gate_multiplier), torch.ones(inner)])
        self.gate_up = Linear([get("gate_proj.weight"), get("up_proj.weight")],
                              [get("gate_proj.bias"), get("up_proj.bias")], build,
                              weight_scale=scale, bias_scale=scale)
        self.down = Linear([get("down_proj.weight")], [get("down_proj.bias")], build,
                           weight_scale=spec.down_multiplier, bias_scale=spec.down_multiplier)
        self.tile = 8 if inner % 8 == 0 else 0
        if self.tile:
            order = torch.arange(2 * inner).view(2, inner // 8, 8).permute(1, 0, 2).reshape(-1).to(build.device)
            self.gate_up.weight = self.gate_up.weight[order].contiguous()
            if self.gate_up.bias is not None:
                self.gate_up.bias = self.gate_up.bias[order].contiguous()

    def gated_projections(self):
        return self.gate_up, self.down, self.tile

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        gate_up = self.gate_up(x)
        activated = torch.empty((x.shape[0], self.spec.intermediate_size), dtype=gate_up.dtype, device=x.device)
        ops.swiglu(gate_up, activated, self.tile)
        return self.down(activated)
