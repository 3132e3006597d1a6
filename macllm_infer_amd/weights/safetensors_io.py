"""Reading and writing the safetensors container: an 8-byte little-endian header length,
a JSON header ``{name: {dtype, shape, data_offsets}}``, then the raw little-endian bytes.

Tensors are read lazily by name from a memory map, in the dtype they were stored in
(the reference maps its safetensors files the same way, src/weights.rs:255-260).
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, Tuple

import numpy as np
import torch

# stored name -> (torch dtype, numpy carrier dtype, bytes per element)
_DTYPES = {
    "F64": (torch.float64, np.float64, 8),
    "F32": (torch.float32, np.float32, 4),
    "F16": (torch.float16, np.float16, 2),
    "BF16": (torch.bfloat16, np.uint16, 2),
    "I64": (torch.int64, np.int64, 8),
    "I32": (torch.int32, np.int32, 4),
    "I16": (torch.int16, np.int16, 2),
    "I8": (torch.int8, np.int8, 1),
    "U8": (torch.uint8, np.uint8, 1),
    "BOOL": (torch.bool, np.bool_, 1),
}
_NAMES = {entry[0]: name for name, entry in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One mapped file: ``names()``, ``shape(name)``, ``dtype(name)``, ``tensor(name)``."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: too short to be a safetensors file")
        self._file = open(path, "rb")
        header_len = struct.unpack("<Q", self._file.read(8))[0]
        if header_len > size - 8:
            raise SafetensorsError(f"{path}: header length {header_len} exceeds the file")
        try:
            header = json.loads(self._file.read(header_len).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as error:
            raise SafetensorsError(f"{path}: header is not valid JSON: {error}") from error
        header.pop("__metadata__", None)
        self._data_start = 8 + header_len
        self._entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        for name, entry in header.items():
            dtype = entry["dtype"]
            if dtype not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name} has unsupported dtype {dtype}")
            shape = tuple(int(d) for d in entry["shape"])
            begin, end = (int(v) for v in entry["data_offsets"])
            count = int(np.prod(shape, dtype=np.int64)) if shape else 1
            if end - begin != count * _DTYPES[dtype][2] or self._data_start + end > size:
                raise SafetensorsError(f"{path}: tensor {name} has inconsistent offsets")
            self._entries[name] = (dtype, shape, begin, end)
        self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    def names(self) -> Iterable[str]:
        return self._entries.keys()

    def __contains__(self, name: str) -> bool:
        return name in self._entries

    def shape(self, name: str) -> Tuple[int, ...]:
        return self._entries[name][1]

    def dtype(self, name: str) -> torch.dtype:
        return _DTYPES[self._entries[name][0]][0]

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor that owns its memory, in the stored dtype."""
        dtype, shape, begin, end = self._entries[name]
        torch_dtype, carrier, width = _DTYPES[dtype]
        count = (end - begin) // width
        array = np.frombuffer(self._map, dtype=carrier, count=count, offset=self._data_start + begin)
        tensor = torch.from_numpy(array.copy())
        if torch_dtype == torch.bfloat16:
            tensor = tensor.view(torch.bfloat16)
        return tensor.reshape(shape)

    def close(self) -> None:
        if self._map is not None:
            self._map.close()
            self._map = None
        self._file.close()


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor]) -> None:
    header = {}
    blobs = []
    offset = 0
    for name, tensor in tensors.items():
        tensor = tensor.detach().cpu().contiguous()
        if tensor.dtype not in _NAMES:
            raise SafetensorsError(f"tensor {name} has dtype {tensor.dtype}, which safetensors cannot hold")
        carrier = tensor.view(torch.uint16) if tensor.dtype == torch.bfloat16 else tensor
        raw = carrier.numpy().tobytes()
        header[name] = {"dtype": _NAMES[tensor.dtype], "shape": list(tensor.shape),
                        "data_offsets": [offset, offset + len(raw)]}
        blobs.append(raw)
        offset += len(raw)
    encoded = json.dumps(header, separators=(",", ":")).encode("utf-8")
    encoded += b" " * ((8 - len(encoded) % 8) % 8)
    with open(path, "wb") as handle:
        handle.write(struct.pack("<Q", len(encoded)))
        handle.write(encoded)
        for raw in blobs:
            handle.write(raw)
