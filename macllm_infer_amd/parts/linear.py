"""A projection y = x . W^T (+ b) with W [out, in] (reference: src/model_weights.rs:530-545).

Matrices keep the dtype they were stored in unless the whole model runs in float32:
a bfloat16 matrix feeds the bfloat16 product, a matrix stored in 32-bit keeps its
32 bits and its product runs in float32.  Multipliers that are linear in the weights
are folded in at build time, in float32, and the result is rounded once.
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch

from ..kernels import ops
from .base import BuildContext


def _as_rows(scale, rows: int) -> Optional[torch.Tensor]:
    if scale is None:
        return None
    if isinstance(scale, (int, float)):
        return None if float(scale) == 1.0 else torch.full((rows, 1), float(scale), dtype=torch.float32)
    scale = torch.as_tensor(scale, dtype=torch.float32).reshape(rows, 1)
    return None if bool((scale == 1.0).all()) else scale


class Linear:
    def __init__(self, weights: Sequence[torch.Tensor], biases: Sequence[Optional[torch.Tensor]],
                 build: BuildContext, weight_scale=None, bias_scale=None):
        """``weights``: matrices [out_i, in] stacked along the output dimension (fused
        projections); ``biases``: one per matrix or None.  ``weight_scale`` / ``bias_scale``:
        a scalar or one value per output row, folded into the weights / biases."""
        stored = {w.dtype for w in weights}
        keep = torch.float32 if (build.dtype == torch.float32 or stored != {torch.bfloat16}) else torch.bfloat16
        weight = torch.cat([w.to(torch.float32) for w in weights], dim=0)
        rows = weight.shape[0]
        scale = _as_rows(weight_scale, rows)
        if scale is not None:
            weight = weight * scale.to(weight.device)
        self.weight = weight.to(keep).contiguous().to(build.device)
        self.bias = None
        if any(b is not None for b in biases):
            parts = [torch.zeros(w.shape[0], device=w.device) if b is None else b.to(torch.float32).reshape(-1)
                     for w, b in zip(weights, biases)]
            bias = torch.cat(parts)
            scale = _as_rows(bias_scale, rows)
            if scale is not None:
                bias = bias * scale.reshape(-1).to(bias.device)
            self.bias = bias.contiguous().to(build.device)
        self.out_features, self.in_features = self.weight.shape

    def __call__(self, x: torch.Tensor, rows: Optional[int] = None) -> torch.Tensor:
        """``rows``: use only the first ``rows`` output rows."""
        if rows is None:
            return ops.linear(x, self.weight, self.bias)
        return ops.linear(x, self.weight[:rows], None if self.bias is None else self.bias[:rows])
