"""Random-weights mode: a model folder (config.json, model.safetensors) from a
configuration and a seed.

Tensor names and shapes are the ones the model's parts declare, so any registered
architecture can be written.  Distributions ("baseline" preset): projections and
embeddings N(0, 0.02); norm weights 1 + N(0, 0.1); A_log = log U[1, 16]; D = 1 + N(0, 0.1);
dt_bias = softplus^-1 of a log-uniform step in [1e-3, 0.1]; biases N(0, 0.02).
The "unit" preset keeps activations of order one through every branch (projections
N(0, 1/sqrt(fan_in)), embeddings N(0, 1/sqrt(width)), conv taps N(0, 1/sqrt(K)), biases N(0, 0.1)),
so that a fault in any part shows in the logits of a tiny model.
Values are drawn in float32 on the CPU in declaration order, then rounded to the
storage dtype; vectors of the state-space recurrence (A_log, D, dt_bias) stay float32.
With ``device`` they are drawn on that device instead (another stream of numbers for the
same seed): the way to get the billions of weights of a large shape in seconds.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict

import torch

from ..engine.model import DecoderModel
from .safetensors_io import write_safetensors

_KEEP_F32 = ("A_log", "D", "dt_bias")


def random_tensors(config, seed: int, storage_dtype: torch.dtype = torch.bfloat16,
                   preset: str = "baseline", device="cpu") -> Dict[str, torch.Tensor]:
    if preset not in ("baseline", "unit"):
        raise ValueError(f"unknown init preset {preset!r}")
    device = torch.device(device)
    generator = torch.Generator(device=device).manual_seed(int(seed))
    unit = preset == "unit"

    def normal(shape, std, mean=0.0):
        return torch.randn(shape, generator=generator, dtype=torch.float32, device=device) * std + mean

    def uniform(shape, low, high):
        return torch.rand(shape, generator=generator, dtype=torch.float32, device=device) * (high - low) + low

    out: Dict[str, torch.Tensor] = {}
    for expect in DecoderModel.expected_tensors(config.to_model_spec()):
        shape = expect.shapes[0]
        kind = expect.init
        if kind == "linear":
            tensor = normal(shape, 1.0 / math.sqrt(shape[-1]) if unit else 0.02)
        elif kind == "embedding":
            tensor = normal(shape, 1.0 / math.sqrt(shape[-1]) if unit else 0.02)
        elif kind == "norm":
            tensor = normal(shape, 0.1, 1.0)
        elif kind == "bias":
            tensor = normal(shape, 0.1 if unit else 0.02)
        elif kind == "conv":
            tensor = normal(shape, 1.0 / math.sqrt(shape[-1]) if unit else 0.02)
        elif kind == "A_log":
            tensor = torch.log(uniform(shape, 1.0, 16.0))
        elif kind == "D":
            tensor = normal(shape, 0.1, 1.0)
        elif kind == "dt_bias":
            step = torch.exp(uniform(shape, math.log(1e-3), math.log(0.1)))
            tensor = step + torch.log(-torch.expm1(-step))          # inverse softplus
        else:
            raise ValueError(f"tensor {expect.name} asks for unknown init {kind!r}")
        leaf = expect.name.rsplit(".", 1)[-1]
        out[expect.name] = tensor if leaf in _KEEP_F32 else tensor.to(storage_dtype)
    return out


def write_random_model(config, seed: int, folder: str, storage_dtype: torch.dtype = torch.bfloat16,
                       preset: str = "baseline") -> str:
    """Write ``folder/config.json`` and ``folder/model.safetensors``; returns ``folder``."""
    os.makedirs(folder, exist_ok=True)
    raw = config.to_dict()
    raw["torch_dtype"] = "bfloat16" if storage_dtype == torch.bfloat16 else "float32"
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(raw, handle, indent=1)
    write_safetensors(os.path.join(folder, "model.safetensors"), random_tensors(config, seed, storage_dtype, preset))
    return folder
