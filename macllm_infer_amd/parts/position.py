"""Position encodings: transforms of q and k before the cache write, and biases on the attention scores."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import BuildContext, Part, register_part


class PositionEncoding(Part):
    """Interface: ``rotate_and_store`` encodes the absolute positions ``step.positions`` into
    the q and k heads of ``qkv`` (q in place) and, if ``cache.owns_kv``, writes the encoded
    k and the raw v of every token into the cache cell ``step.slot_mappings[cache.group]``.
    A subclass may implement only ``rotate`` (in place on ``qkv``); the store is then done
    by the cache-write kernel without rotation.

    An encoding that (also) biases the scores by distance sets ``score_slopes``: a float32 tensor [query heads]
    on the device, with score(head, query at s, key at p) -= score_slopes[head] * (s - p).  The attention part
    then takes its general kernel, which knows the term; the matrix-core and fused decode kernels do not."""
    kernel_modules = ("attention",)
    score_slopes = None

    def fused_rotation(self):
        """What a kernel that rotates q and the new key itself has to apply in place of ``rotate_and_store``:
        ``(inv_freq, rotary_dim)`` of a half-split rotation by position * inv_freq[j] of the first ``rotary_dim``
        dimensions of every head (``(None, 0)``: nothing), or None when the encoding is no such rotation; the
        layer then runs this part's own ``rotate_and_store`` and the general kernels."""
        return None

    def rotate(self, qkv, num_heads, num_kv_heads, head_dim, step) -> None:
        return None

    def rotate_and_store(self, qkv, num_heads, num_kv_heads, head_dim, step, cache) -> None:
        self.rotate(qkv, num_heads, num_kv_heads, head_dim, step)
        if cache.owns_kv:
            ops.rope_kv_store(qkv, num_heads, num_kv_heads, head_dim, step.positions, None, 0,
                              step.slot_mappings[cache.group], cache.k_cache, cache.v_cache)


@register_part("none")
class NoPosition(PositionEncoding):
    graph_safe = True

    def __init__(self, spec, head_dim: int, build: BuildContext):
        pass

    def fused_rotation(self):
        return None, 0


@register_part("rope")
class Rope(PositionEncoding):
    """Half-split rotary encoding: f_j = theta^(-2j/rotary_dim) formed in float64 and rounded
    to float32; angle = position * f_j, cos and sin in float32
    (reference: src/decoder.rs:136-144, 186-195, 226-229)."""
    graph_safe = True

    def __init__(self, spec, head_dim: int, build: BuildContext):
        self.rotary_dim = spec.rotary_dim
        frequencies = [1.0 / (spec.theta ** (index / spec.rotary_dim)) for index in range(0, spec.rotary_dim, 2)]
        self.inv_freq = torch.tensor(frequencies, dtype=torch.float64).to(torch.float32).to(build.device)

    def fused_rotation(self):
        return self.inv_freq, self.rotary_dim

    def rotate_and_store(self, qkv, num_heads, num_kv_heads, head_dim, step, cache) -> None:
        owns = cache.owns_kv
        ops.rope_kv_store(qkv, num_heads, num_kv_heads, head_dim, step.positions, self.inv_freq,
                          self.rotary_dim, step.slot_mappings[cache.group] if owns else None,
                          cache.k_cache if owns else None, cache.v_cache if owns else None)
