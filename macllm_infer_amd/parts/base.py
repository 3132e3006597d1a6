"""What every part of a layer looks like from outside, and the registry of part kinds.

A part is built from its spec (sizes and constants as fields), the path of its
tensors, the tensors themselves and a ``BuildContext``; it never learns which model it
is in.  ``register_part(kind)`` maps the ``kind`` string of a spec dataclass to the class
that runs it, so a new mixer, feed-forward, norm or position encoding is added by
registering a class, without a change to this package.

Interfaces
----------
every part      ``expected_tensors(spec, prefix, hidden_size) -> [Expect]`` (classmethod),
                ``kernel_modules`` (names of the HIP modules it launches),
                ``__init__(spec, prefix, tensors, build)``
mixer           ``cache_needs(spec) -> [KVNeed | StateNeed]`` (classmethod);
                ``forward(x [T, d], step, cache: EntryCache) -> [T, d]``;
                optional ``step_tables() -> [StepTable]``: index tables of its own in every step;
                optional ``projections()`` + ``mix(...)``: see ``Mixer.projections``
feed-forward    ``forward(x [T, d]) -> [T, d]``; optional ``gated_projections()``
norm            ``forward(residual, rows=None) -> normed activations``; optional ``rms_prologue() ->
                (weight, eps)``: the norm is y = x / sqrt(mean(x^2) + eps) * weight, which the skinny
                kernels compute in their prologue, or take over altogether (``Residual.scaled``)
position        ``rotate_and_store(qkv, heads, kv_heads, head_dim, step, cache)``; optional
                ``fused_rotation() -> (inv_freq or None, rotary_dim) | None``: what the fused decode kernel
                applies in its place
every part      ``graph_safe = True`` if its forward may be captured in a HIP graph;
                ``limits(spec, hidden_size) -> [Limit]`` (classmethod): sizes its kernels refuse
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

_PARTS: Dict[str, type] = {}


def register_part(kind: str):
    def decorate(cls):
        _PARTS[kind] = cls
        cls.kind = kind
        return cls
    return decorate


def part_class(spec) -> type:
    kind = getattr(spec, "kind", None)
    if kind not in _PARTS:
        raise KeyError(f"no part is registered for kind {kind!r}; registered: {sorted(_PARTS)}")
    return _PARTS[kind]


@dataclass
class BuildContext:
    hidden_size: int
    dtype: torch.dtype            # activation dtype: torch.float32 or torch.bfloat16
    device: torch.device
    max_context: int
    # Where two kernels can serve a product, a fast path may time both when the model is built and take the
    # faster one; False: fixed rules only, so that which kernel runs (and with it the last bits of bfloat16
    # results) is the same in every process.
    measure_paths: bool = True


@dataclass
class ScaledRows:
    """The residual stream's rows as the product behind a norm wants them, but for the division by the root mean
    square: ``rows`` bfloat16 [T, d] = h * weight, with the partial sums of squares of h (``ssq``, float32
    [workgroups, rows rounded up to 16]) that give it.  ``weight`` is the norm's weight they were made for."""
    rows: torch.Tensor
    ssq: torch.Tensor
    weight: torch.Tensor


class Residual:
    """The float32 residual stream [T, d] plus the branch outputs not yet added to it.
    The next norm adds them and normalizes in one kernel.

    ``next_norm``: (weight, eps) of the norm that the layer after the one running starts with (the final norm
    after the last), if that norm is a root-mean-square norm, set by whoever runs the layers; a layer whose last
    projection adds to the stream itself may then leave ``scaled`` rows for it.  ``scaled`` is dropped whenever
    ``h`` or ``pending`` is assigned: whoever changes the stream without knowing of it makes it stale."""

    def __init__(self, h: torch.Tensor):
        self._h = h
        self._pending: List[torch.Tensor] = []
        self.scaled: Optional[ScaledRows] = None
        self.next_norm: Optional[tuple] = None

    @property
    def h(self) -> torch.Tensor:
        return self._h

    @h.setter
    def h(self, value: torch.Tensor) -> None:
        self._h, self.scaled = value, None

    @property
    def pending(self) -> List[torch.Tensor]:
        return self._pending

    @pending.setter
    def pending(self, value: List[torch.Tensor]) -> None:
        self._pending, self.scaled = value, None


class Part:
    kernel_modules = ()
    # True when ``forward`` only enqueues work on the current stream (no host read-back, no
    # data-dependent launch shapes), so that a decode step containing the part can be captured
    # as a HIP graph.  Parts that do not say so run eagerly.
    graph_safe = False

    @classmethod
    def expected_tensors(cls, spec, prefix: str, hidden_size: int):
        return []

    @classmethod
    def limits(cls, spec, hidden_size: int):
        """The sizes of ``spec`` that no kernel of this part takes, as ``kernels.limits.Limit``s: asked when a
        model is built, before its weights are read.  A part whose kernels take every size reports none."""
        return []


class Mixer(Part):
    # rows of one lane that one workgroup of the mixer's prompt kernel takes: the step's table of such runs
    # is cut to the largest tile any mixer of the model names (0: the mixer reads no such table)
    query_tile = 0
    # tokens of a chunk: the step then carries every lane cut from its first token into chunks of that many
    # (``step.chunk_tables[chunk_tokens]``); 0: the mixer reads no such table
    chunk_tokens = 0

    @classmethod
    def cache_needs(cls, spec):
        return []

    def step_tables(self):
        """Index tables of its own that the mixer wants in every step, as ``engine.context.StepTable``s: each is
        written on the host from the step's lanes by the function the mixer gives, uploaded with the step's
        other arrays, and found in ``step.tables[name]`` (int32, on the device); in a step that a captured graph
        reads it has the size of the step's capacity and a fixed address.  Mixers that declare the same name
        share one table."""
        return ()

    def forward(self, x: torch.Tensor, step, cache) -> torch.Tensor:
        raise NotImplementedError

    def projections(self):
        """A mixer that is "input projection of the normed rows, something in between, output projection"
        may hand out the three pieces: ``(in Linear, out Linear, width of what lies between)``, with
        ``mix(projected [T, in.out_features], step, cache, out [T, width])`` doing the part in between on
        column views of wider matrices.  A layer can then run the projections of all its mixers as one
        product each (and, for steps of single tokens, through the skinny kernels).  None: the mixer is
        only ever run through ``forward``."""
        return None


class FeedForward(Part):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def gated_projections(self):
        """A feed-forward that is down(SiLU(gate(x)) * up(x)) may hand out ``(gate_up Linear, down Linear,
        tile)``: gate and up rows of the first interleaved in tiles of ``tile`` rows.  None: it is only
        ever run through ``forward``."""
        return None
