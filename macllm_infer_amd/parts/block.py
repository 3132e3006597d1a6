"""Arrangements of parts in a layer."""
from __future__ import annotations

from typing import Dict

import torch

from .base import BuildContext, Residual, part_class

_ARRANGEMENTS: Dict[str, type] = {}
_FUSIONS: Dict[str, object] = {}

OVERLAP_MIN_TOKENS = 256       # prompt portions from this size on run their two mixers on two streams
_side_streams: Dict[int, list] = {}


def side_stream(device: torch.device, beside: "torch.cuda.Stream") -> "torch.cuda.Stream":
    """A second stream of the device (default priority) that is not ``beside``.  Streams come from a pool of a
    few dozen that hands them out in turn, so the one drawn may be the very stream a graph is being captured on:
    work recorded "beside" it would queue behind (a 2,048-token prompt of the 0.5B shape: 7.2 ms instead of 6.3)."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    streams = _side_streams.setdefault(index, [])
    for stream in streams:
        if stream != beside:
            return stream
    while True:
        streams.append(torch.cuda.Stream(device=device))
        if streams[-1] != beside:
            return streams[-1]


def overlap_pays(mixers, rows: int, device: torch.device) -> bool:
    """Whether two mixers of a layer that read the same rows should run beside each other on two streams: in a
    captured graph only (launched one by one the step waits for the host, which the second stream costs more),
    for portions long enough to be worth the hops between the queues, and if both only queue work."""
    return (len(mixers) == 2 and rows >= OVERLAP_MIN_TOKENS and device.type == "cuda"
            and torch.cuda.is_current_stream_capturing()
            and all(getattr(mixer, "graph_safe", False) for mixer in mixers))


def register_fusion(arrangement: str):
    """Register ``factory(block, build) -> fusion or None`` for layers of ``arrangement``: a fusion runs the
    whole layer through fewer launches where its parts and sizes allow
    (``forward(residual, step, caches) -> bool``: True when it ran the layer)."""
    def decorate(factory):
        _FUSIONS[arrangement] = factory
        return factory
    return decorate


def register_arrangement(name: str):
    def decorate(cls):
        _ARRANGEMENTS[name] = cls
        return cls
    return decorate


def arrangement_class(name: str) -> type:
    if name not in _ARRANGEMENTS:
        raise KeyError(f"no arrangement named {name!r}; registered: {sorted(_ARRANGEMENTS)}")
    return _ARRANGEMENTS[name]


@register_arrangement("parallel_prenorm")
class ParallelPreNormBlock:
    """n = norm(h); h += sum over mixers of mixer(n); h += ffn(norm(h)).
    All mixers read the same normed input and their outputs are summed into the residual
    (reference: src/decoder.rs:2658-2682, 2684-2699).  With one mixer this is the ordinary
    sequential pre-norm layer."""

    @classmethod
    def expected_tensors(cls, layer, hidden_size: int):
        out = []
        out += part_class(layer.mixer_norm).expected_tensors(
            layer.mixer_norm, f"{layer.prefix}.{layer.mixer_norm_name}", hidden_size)
        for slot in layer.mixers:
            out += part_class(slot.spec).expected_tensors(slot.spec, f"{layer.prefix}.{slot.name}", hidden_size)
        out += part_class(layer.ffn_norm).expected_tensors(
            layer.ffn_norm, f"{layer.prefix}.{layer.ffn_norm_name}", hidden_size)
        out += part_class(layer.ffn).expected_tensors(layer.ffn, f"{layer.prefix}.{layer.ffn_name}", hidden_size)
        return out

    @classmethod
    def limits(cls, layer, hidden_size: int):
        """What the kernels of this layer's parts refuse (see ``Part.limits``)."""
        out = []
        for spec in [layer.mixer_norm, layer.ffn_norm, layer.ffn] + [slot.spec for slot in layer.mixers]:
            out += part_class(spec).limits(spec, hidden_size)
        return out

    @classmethod
    def kernel_modules(cls, layer):
        modules = []
        for spec in [layer.mixer_norm, layer.ffn_norm, layer.ffn] + [slot.spec for slot in layer.mixers]:
            modules += list(part_class(spec).kernel_modules)
        return modules

    def __init__(self, layer, tensors, build: BuildContext):
        self.layer = layer
        self.mixer_norm = part_class(layer.mixer_norm)(
            layer.mixer_norm, f"{layer.prefix}.{layer.mixer_norm_name}", tensors, build)
        self.mixers = [(slot.name, part_class(slot.spec)(slot.spec, f"{layer.prefix}.{slot.name}", tensors, build))
                       for slot in layer.mixers]
        self.ffn_norm = part_class(layer.ffn_norm)(
            layer.ffn_norm, f"{layer.prefix}.{layer.ffn_norm_name}", tensors, build)
        self.ffn = part_class(layer.ffn)(layer.ffn, f"{layer.prefix}.{layer.ffn_name}", tensors, build)
        factory = _FUSIONS.get(layer.arrangement)
        self.fusion = factory(self, build) if factory is not None else None      # None when parts or sizes do not fit

    @property
    def graph_safe(self) -> bool:
        parts = [self.mixer_norm, self.ffn_norm, self.ffn] + [mixer for _, mixer in self.mixers]
        return all(getattr(part, "graph_safe", False) for part in parts)

    def tune(self, peers) -> None:
        """Called once every layer of the model is built, with all of them: what a layer can only decide by
        timing itself among the others."""
        tune = getattr(self.fusion, "tune_chain", None)
        if tune is not None:
            tune([getattr(peer, "fusion", None) for peer in peers])

    @property
    def first_norm(self):
        """The norm this arrangement starts with: what a layer before it may prepare the stream for."""
        return self.mixer_norm

    def forward(self, residual: Residual, step, caches) -> None:
        """``caches``: mixer name -> EntryCache of this run of the layer."""
        fusion = self.fusion
        if fusion is not None and fusion.forward(residual, step, caches):
            return
        normed = self.mixer_norm.forward(residual)
        if overlap_pays([mixer for _, mixer in self.mixers], normed.shape[0], normed.device):
            # the second mixer is recorded first and stays on the queue of the kernels around it (see the fast
            # path's ``forward_general``); what either allocates is its own stream's until the join
            (first_name, first), (second_name, second) = self.mixers
            main = torch.cuda.current_stream(normed.device)
            side = side_stream(normed.device, main)
            side.wait_stream(main)
            second_out = second.forward(normed, step, caches[second_name])
            with torch.cuda.stream(side):
                first_out = first.forward(normed, step, caches[first_name])
            main.wait_stream(side)
            residual.pending = [first_out, second_out]
        else:
            residual.pending = [mixer.forward(normed, step, caches[name]) for name, mixer in self.mixers]
        normed = self.ffn_norm.forward(residual)
        residual.pending = [self.ffn.forward(normed)]
