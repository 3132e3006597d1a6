"""Arrangements of parts in a layer."""
from __future__ import annotations

from typing import Dict

from .base import BuildContext, Residual, part_class

_ARRANGEMENTS: Dict[str, type] = {}
_FUSIONS: Dict[str, object] = {}


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
        residual.pending = [mixer.forward(normed, step, caches[name]) for name, mixer in self.mixers]
        normed = self.ffn_norm.forward(residual)
        residual.pending = [self.ffn.forward(normed)]
