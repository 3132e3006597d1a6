"""What a step has to move and to compute, from the model's sizes: bytes read and written and flops, per
group of kernels.  ``bench.py`` takes its roofline figures from here and ``kernel_trace`` sets them against
the measured times of each group's kernels.

The figures are the least a step can do: every weight it uses read once, the cache and the state of the live
requests read once, what it has to write written once; activations between kernels (a few rows in a decode
step) are left out of a decode step and counted once per kernel boundary in a prompt step.
(The reference sizes the same quantities for its cache: src/architecture.rs:677-795.)
"""
from __future__ import annotations

import re
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

PEAK_HBM_BYTES = 8.0e12                                   # MI355X, published: 8 TB/s
PEAK_FLOPS = {"bf16": 2.5e15, "f32": 157.3e12}            # dense matrix cores, published


@dataclass
class Cost:
    read: float = 0.0        # bytes
    written: float = 0.0     # bytes
    flops: float = 0.0

    def __add__(self, other: "Cost") -> "Cost":
        return Cost(self.read + other.read, self.written + other.written, self.flops + other.flops)

    def times(self, factor: float) -> "Cost":
        return Cost(self.read * factor, self.written * factor, self.flops * factor)


def model_sizes(spec) -> dict:
    """Sums over the scheduled layers of a ``ModelSpec``: matrix elements by projection, K/V elements per
    token, state elements (float32) and conv tail elements (activation dtype) per request."""
    d = spec.hidden_size
    total = dict(in_weights=0, out_weights=0, gate_up=0, down=0, kv_per_token=0, state=0, conv_tail=0,
                 attention=0, scan=0, layers=len(spec.schedule), head=spec.vocab_size * d, hidden=d,
                 mixed=0, inner=0, in_width=0)
    for entry in spec.schedule:
        layer = spec.layers[entry.layer]
        for slot in layer.mixers:
            part = slot.spec
            if part.kind == "attention":
                q, kv = part.num_heads * part.head_dim, part.num_kv_heads * part.head_dim
                total["in_weights"] += (q + 2 * kv) * d
                total["out_weights"] += d * q
                total["kv_per_token"] += 2 * kv if entry.kv_from is None else 0
                total["attention"] += part.num_heads * part.head_dim      # x 2 T^2 flops (causal: half of 4 T^2)
                total["mixed"] += q
                total["in_width"] += q + 2 * kv
            elif part.kind == "mamba2":
                total["in_weights"] += part.projection_width * d
                total["out_weights"] += d * part.inner_size
                total["state"] += part.num_heads * part.head_dim * part.state_size
                total["conv_tail"] += max(part.conv_kernel - 1, 0) * part.conv_width
                total["scan"] += part.num_heads * part.head_dim * part.state_size      # x 6 T flops
                total["mixed"] += part.inner_size
                total["in_width"] += part.projection_width
        if layer.ffn.kind == "swiglu":
            total["gate_up"] += 2 * layer.ffn.intermediate_size * d
            total["down"] += d * layer.ffn.intermediate_size
            total["inner"] += layer.ffn.intermediate_size
    return total


def decode_step_costs(spec, batch: int, context: float, element: int = 2) -> Dict[str, Cost]:
    """A step of ``batch`` single tokens whose requests hold ``context`` tokens each."""
    s = model_sizes(spec)
    rows = batch
    return {
        "input projections": Cost(s["in_weights"] * element, 0, 2.0 * rows * s["in_weights"]),
        "mixers": Cost(batch * (s["kv_per_token"] * context * element + s["state"] * 4 + s["conv_tail"] * element),
                       batch * (s["kv_per_token"] * element + s["state"] * 4 + s["conv_tail"] * element),
                       batch * (2.0 * s["attention"] * 2 * context + 6.0 * s["scan"])),
        "output projections": Cost(s["out_weights"] * element, 0, 2.0 * rows * s["out_weights"]),
        "gate and up projections": Cost(s["gate_up"] * element, 0, 2.0 * rows * s["gate_up"]),
        "down projections": Cost(s["down"] * element, 0, 2.0 * rows * s["down"]),
        "output head": Cost(s["head"] * element, batch * spec.vocab_size * 4, 2.0 * rows * s["head"]),
    }


def prefill_costs(spec, tokens: int, element: int = 2) -> Dict[str, Cost]:
    """One prompt of ``tokens`` tokens in one step (its last position's logits wanted)."""
    s = model_sizes(spec)
    T = tokens
    weights = s["in_weights"] + s["out_weights"] + s["gate_up"] + s["down"]
    rows_moved = T * element * (s["hidden"] * 4 * s["layers"] + s["in_width"] + s["mixed"] + 3 * s["inner"])
    return {
        "matrix products": Cost(weights * element + rows_moved, 0, 2.0 * T * weights + 2.0 * s["head"]),
        "attention": Cost(T * s["kv_per_token"] * element, T * s["kv_per_token"] * element, 2.0 * s["attention"] * T * T),
        "state-space scan": Cost(s["state"] * 4, s["state"] * 4, 6.0 * s["scan"] * T),
    }


def total(costs: Dict[str, Cost]) -> Cost:
    out = Cost()
    for cost in costs.values():
        out = out + cost
    return out


# Which kernels do the work of which group (name patterns of this package's kernels and of the BLAS library's).
# fused_gemm_kernel<row tiles, prologue (0 norm, 1 plain, 2 merge of the attention runs), epilogue (0 plain,
# 1 SiLU(g)*u, 2 conv, 3 add to the residual stream), ...>; shared_rows_gemm_kernel<row tiles, feature tiles a
# wave, epilogue (0 float32 slabs, 1 SiLU(g)*u, 2 conv or plain rows)>.  A product with the plain epilogue that is
# launched once a step is the output head; launched more often, an output or down projection (the library's
# products carry no such mark and stay with the other kernels).
DECODE_GROUPS: List[Tuple[str, str]] = [
    (r"mixer_decode_kernel|mixer_merge_kernel|decode_attention_kernel|decode_merge_kernel|ssm_scan_kernel|conv_step_kernel|"
     r"gate_norm_kernel|rope_kv_store_kernel|paged_attention_kernel|paged_attention_tile_kernel|"
     r"paged_attention_merge_kernel", "mixers"),
    (r"fused_gemm_kernel<\d+, \d+, 2|shared_rows_gemm_kernel<\d+, \d+, 2", "input projections"),
    (r"fused_gemm_kernel<\d+, \d+, 1|shared_rows_gemm_kernel<\d+, \d+, 1", "gate and up projections"),
    (r"fused_gemm_kernel<\d+, \d+, 3|fused_gemm_kernel<\d+, 2, 0|shared_rows_gemm_kernel<\d+, \d+, 0|fused_gemm_split_kernel",
     "output projections + down projections"),
]
PLAIN_PRODUCT = r"fused_gemm_kernel<\d+, [01], 0"
PREFILL_GROUPS: List[Tuple[str, str]] = [
    (r"^Cijk_|gemm_f32_kernel", "matrix products"),
    (r"prefill_attention|paged_attention_kernel|paged_attention_tile_kernel|paged_attention_merge_kernel|"
     r"rope_kv_store_kernel", "attention"),
    (r"ssd_|ssm_scan_kernel|conv1d_silu|conv_state_update|gate_norm_kernel", "state-space scan"),
]


def group_of(kernel: str, groups: List[Tuple[str, str]], calls: int = 2) -> Optional[str]:
    """The group of a kernel by its name and, for the products that carry no other mark, by how often a step
    launches it (``calls``)."""
    for pattern, name in groups:
        if re.search(pattern, kernel):
            return name
    if groups is DECODE_GROUPS and re.search(PLAIN_PRODUCT, kernel):
        return "output head" if calls == 1 else "output projections + down projections"
    return None


def merged(costs: Dict[str, Cost], name: str) -> Cost:
    """The cost of a group whose name joins several of ``costs`` with " + "."""
    out = Cost()
    for piece in name.split(" + "):
        out = out + costs.get(piece, Cost())
    return out
