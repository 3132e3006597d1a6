"""RMSNorm fused with the residual add that precedes it."""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from ..kernels.limits import NORM_MAX_WIDTH, beyond
from ..weights.loader import Expect
from .base import BuildContext, Part, Residual, register_part


def partial_slab(pending) -> Optional[torch.Tensor]:
    """The float32 [S, T, d] tensor whose slabs, in order, ``pending`` lists (a branch that arrives as
    partial sums of a product split over K), or None."""
    if len(pending) < 2:
        return None
    base = pending[0]._base
    if (base is None or base.dim() != 3 or base.dtype != torch.float32 or base.shape[0] != len(pending)
            or not base.is_contiguous()):
        return None
    for index, slab in enumerate(pending):
        if slab._base is not base or slab.shape != base.shape[1:] or slab.data_ptr() != base[index].data_ptr():
            return None
    return base


@register_part("rmsnorm")
class RmsNorm(Part):
    """y = x / sqrt(mean(x^2) + eps) * w, statistics in float32
    (reference: src/model_weights.rs:563-565, golden src/decoder.rs:10331-10334)."""
    graph_safe = True
    kernel_modules = ("common",)

    @classmethod
    def expected_tensors(cls, spec, prefix: str, hidden_size: int):
        return [Expect(f"{prefix}.weight", ((hidden_size,),), init="norm")]

    @classmethod
    def limits(cls, spec, hidden_size: int):
        return beyond("rmsnorm", "hidden_size", hidden_size, NORM_MAX_WIDTH, "the norm stages a float32 row in 64 KiB of LDS")

    def __init__(self, spec, prefix: str, tensors, build: BuildContext):
        self.eps = spec.eps
        self.build = build
        self.weight = tensors[f"{prefix}.weight"].to(torch.float32).contiguous().to(build.device)

    def rms_prologue(self):
        return self.weight, self.eps

    def forward(self, residual: Residual, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Add the pending branch outputs to the residual stream and return its normed rows
        (all of them, or only ``rows``; with ``rows`` the stream itself is left unchanged)."""
        pending = residual.pending
        slab = partial_slab(pending)
        if slab is not None and slab.shape[0] <= 16 and residual.h.shape[1] % 4 == 0:
            # partial sums of one branch: added and normed in one launch (with a gather: added here,
            # the gather below then norms the rows of the stream itself)
            out = None
            if rows is None:
                out = torch.empty(residual.h.shape, dtype=self.build.dtype, device=residual.h.device)
            ops.add_partials_rmsnorm(residual.h, slab, self.weight, self.eps, out)
            residual.pending = pending = []
            if rows is None:
                return out
        while len(pending) > 2:                    # more than two branches: add the extra ones first
            ops.add_rmsnorm(residual.h, pending[:2], self.weight, self.eps, None)
            pending = pending[2:]
        count = residual.h.shape[0] if rows is None else rows.numel()
        out = torch.empty((count, residual.h.shape[1]), dtype=self.build.dtype, device=residual.h.device)
        ops.add_rmsnorm(residual.h, pending, self.weight, self.eps, out, rows)
        if rows is None:
            residual.pending = []
        return out
