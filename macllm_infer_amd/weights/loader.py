"""Weights by tensor name, with one error that says everything that is wrong with a file.

Every part declares the tensors it needs (``Expect``: name, the shapes it accepts,
how to draw it at random).  ``bind`` compares the whole list with the file before any
tensor is handed out: missing names, names nobody asked for and wrong shapes are
collected into a single ``WeightError``.  The reference asks for each tensor by exact
name with an expected shape (src/model_weights.rs:36-77, ``UnexpectedShape``
:229-238) and rejects unknown tensors (src/gguf_model.rs:687-744).

Tensors keep the dtype they were stored in: a bfloat16 checkpoint stays bfloat16, a
tensor stored in 32-bit stays 32-bit, integer tables become int32.  What a part does
with them (upcasting small vectors to float32, fusing matrices) is the part's business.
"""
from __future__ import annotations

import json
import os
import warnings
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .safetensors_io import SafetensorsFile


class Float16Narrowed(UserWarning):
    """Tensors stored in float16 were kept in bfloat16, which drops 3 bits of their mantissas."""


class WeightError(ValueError):
    """Lists every missing tensor, unexpected tensor and wrong shape of a checkpoint."""

    def __init__(self, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)
        lines = ["the checkpoint does not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, expected, got in self.wrong_shape:
            wanted = " or ".join(str(list(shape)) for shape in expected)
            lines.append(f"  wrong shape: {name} expected {wanted}, got {list(got)}")
        for name, got in self.wrong_dtype:
            lines.append(f"  wrong dtype: {name} is {got}, expected a floating-point tensor")
        super().__init__("\n".join(lines))


@dataclass(frozen=True)
class Expect:
    """One tensor a part needs.  ``shapes[0]`` is the canonical shape (the one written by
    the random-weights mode); the others are accepted on disk and reshaped to it.
    ``init`` names the distribution used by the random-weights mode."""
    name: str
    shapes: Tuple[Tuple[int, ...], ...]
    init: str = "linear"
    integer: bool = False


class WeightSource:
    """Name -> tensor over one ``model.safetensors`` or the shards listed by
    ``model.safetensors.index.json`` (discovery as src/weights.rs:380-404)."""

    def __init__(self, files: Sequence[SafetensorsFile]):
        self._files = list(files)
        self._where: Dict[str, SafetensorsFile] = {}
        self._stored: Dict[str, str] = {}                 # name as asked for -> name in the file
        self.clashes: List[Tuple[str, str]] = []          # (stored name, the stored name it doubles)
        for handle in self._files:
            for name in handle.names():
                self._where[name] = handle
                self._stored[name] = name

    def apply_aliases(self, aliases: Sequence[Tuple[str, str]], root_prefix: str = "") -> None:
        """Let tensors stored under another spelling answer to the model's names.  ``aliases``:
        (other spelling, the model's spelling) of a piece of a name, e.g. (".feed_forward.",
        ".mlp.") (the alias table idea of src/gguf.rs:1786-1813).  ``root_prefix``: if no stored
        name starts with it, every stored name but the output head's gets it in front: a
        checkpoint saved from the inner model has ``layers.0...`` for ``model.layers.0...``
        (namespace choice of src/decoder.rs:2987-2995).  A tensor stored under two spellings is
        reported by ``bind`` as unexpected."""
        rooted = bool(root_prefix) and not any(name.startswith(root_prefix) for name in self._where)
        renamed: Dict[str, str] = {}
        for stored in sorted(self._where):
            name = stored
            if rooted and not name.startswith("lm_head"):
                name = root_prefix + name
            for other, ours in aliases:
                if other in name:
                    name = name.replace(other, ours)
            if name in renamed:
                self.clashes.append((stored, renamed[name]))
            else:
                renamed[name] = stored
        self._stored = renamed

    @classmethod
    def from_dir(cls, model_dir: str) -> "WeightSource":
        single = os.path.join(model_dir, "model.safetensors")
        index = os.path.join(model_dir, "model.safetensors.index.json")
        if os.path.isfile(single):
            return cls([SafetensorsFile(single)])
        if os.path.isfile(index):
            with open(index) as handle:
                shards = sorted(set(json.load(handle)["weight_map"].values()))
            return cls([SafetensorsFile(os.path.join(model_dir, shard)) for shard in shards])
        raise FileNotFoundError(f"{model_dir} holds neither model.safetensors nor model.safetensors.index.json")

    @classmethod
    def from_tensors(cls, tensors: Dict[str, torch.Tensor]) -> "WeightSource":
        return cls([_MemoryFile(tensors)])

    def names(self):
        return self._stored.keys()

    def stored_name(self, name: str) -> str:
        return self._stored[name]

    def shape(self, name: str):
        stored = self._stored[name]
        return self._where[stored].shape(stored)

    def dtype(self, name: str):
        stored = self._stored[name]
        return self._where[stored].dtype(stored)

    def tensor(self, name: str) -> torch.Tensor:
        stored = self._stored[name]
        return self._where[stored].tensor(stored)

    def close(self) -> None:
        for handle in self._files:
            handle.close()


class _MemoryFile:
    def __init__(self, tensors):
        self._tensors = dict(tensors)

    def names(self):
        return self._tensors.keys()

    def shape(self, name):
        return tuple(self._tensors[name].shape)

    def dtype(self, name):
        return self._tensors[name].dtype

    def tensor(self, name):
        return self._tensors[name].detach().cpu().clone()

    def close(self):
        return None


def bind(source: WeightSource, expectations: Sequence[Expect],
         copies: Optional[Dict[str, str]] = None) -> Dict[str, torch.Tensor]:
    """Check the whole checkpoint against ``expectations`` and return name -> CPU tensor
    (canonical shape, stored dtype; integer tables as int32).  ``copies``: name of a tensor the model
    does not bind -> the bound tensor it may repeat (a tied output head saved beside the embedding);
    it is accepted when both hold the same values and reported as unexpected otherwise."""
    wanted = {}
    for expect in expectations:
        wanted[expect.name] = expect                      # a name asked for twice (tied weights) is one tensor
    present = set(source.names())
    missing = sorted(name for name in wanted if name not in present)
    unexpected = []
    for name in sorted(present - set(wanted)):
        original = (copies or {}).get(name)
        if original in wanted and original in present:
            if (tuple(source.shape(name)) == tuple(source.shape(original))
                    and torch.equal(source.tensor(name), source.tensor(original))):
                continue
            unexpected.append(f"{source.stored_name(name)} (the model shares {original}, and this tensor differs from it)")
        else:
            unexpected.append(source.stored_name(name))
    unexpected.sort()
    unexpected += [f"{stored} (the same tensor as {other})" for stored, other in source.clashes]
    wrong_shape: List[Tuple[str, Tuple, Tuple]] = []
    wrong_dtype: List[Tuple[str, str]] = []
    for name, expect in wanted.items():
        if name not in present:
            continue
        if tuple(source.shape(name)) not in expect.shapes:
            wrong_shape.append((name, expect.shapes, tuple(source.shape(name))))
        if not expect.integer and not source.dtype(name).is_floating_point:
            wrong_dtype.append((name, str(source.dtype(name))))
    if missing or unexpected or wrong_shape or wrong_dtype:
        raise WeightError(missing, unexpected, sorted(wrong_shape), sorted(wrong_dtype))
    out: Dict[str, torch.Tensor] = {}
    narrowed: List[str] = []
    for name, expect in wanted.items():
        tensor = source.tensor(name).reshape(expect.shapes[0])
        if expect.integer:
            tensor = tensor.to(torch.int32)
        elif tensor.dtype == torch.float64:
            tensor = tensor.to(torch.float32)
        elif tensor.dtype == torch.float16:
            tensor = tensor.to(torch.bfloat16)            # the 16-bit serving dtype is bfloat16
            narrowed.append(name)
        out[name] = tensor
    if narrowed:
        warnings.warn(f"{len(narrowed)} tensors stored in float16 (the first: {narrowed[0]}) are kept in bfloat16: "
                      "3 of their 10 mantissa bits are dropped and values beyond bfloat16's 8 bits are rounded; "
                      "store the checkpoint in bfloat16 or float32 to choose the rounding yourself",
                      Float16Narrowed, stacklevel=2)
    return out
