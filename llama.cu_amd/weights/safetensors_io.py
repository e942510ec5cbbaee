"""The safetensors container: 8 bytes little-endian header length, a JSON header
``{name: {"dtype", "shape", "data_offsets"}}``, then the tensors' bytes.  Files are
memory-mapped, so a tensor costs memory only when it is copied to the GPU.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, List, Tuple

import torch


class SafetensorsError(ValueError):
    pass


DTYPES = {"F32": torch.float32, "BF16": torch.bfloat16, "F16": torch.float16, "F64": torch.float64,
          "I32": torch.int32, "I64": torch.int64, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
          "BOOL": torch.bool}
NAMES = {v: k for k, v in DTYPES.items()}


def read_safetensors_header(path: str) -> Tuple[Dict[str, dict], int]:
    """(header without ``__metadata__``, offset of the data) after checking every entry
    against the file's size."""
    size = os.path.getsize(path)
    with open(path, "rb") as f:
        first = f.read(8)
        if len(first) < 8:
            raise SafetensorsError(f"{path}: too short for a safetensors file")
        (hlen,) = struct.unpack("<Q", first)
        if hlen > size - 8:
            raise SafetensorsError(f"{path}: header length {hlen} exceeds the file ({size} bytes)")
        try:
            header = json.loads(f.read(hlen))
        except (json.JSONDecodeError, UnicodeDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON: {e}") from None
    if not isinstance(header, dict):
        raise SafetensorsError(f"{path}: the header is no JSON object")
    header.pop("__metadata__", None)
    base = 8 + hlen
    for name, info in header.items():
        if not isinstance(info, dict):
            raise SafetensorsError(f"{path}: the header's entry for tensor {name!r} is no object")
        dt = DTYPES.get(info.get("dtype"))
        if dt is None:
            raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {info.get('dtype')!r}")
        shape, offsets = info.get("shape"), info.get("data_offsets")
        if not isinstance(shape, list) or not all(isinstance(x, int) and x >= 0 for x in shape):
            raise SafetensorsError(f"{path}: tensor {name!r}: 'shape' is missing or no list of sizes")
        if not isinstance(offsets, list) or len(offsets) != 2 or not all(isinstance(x, int) for x in offsets):
            raise SafetensorsError(f"{path}: tensor {name!r}: 'data_offsets' is missing or no pair of offsets")
        a, b = offsets
        n = 1
        for s in shape:
            n *= s
        if b - a != n * torch.empty(0, dtype=dt).element_size():
            raise SafetensorsError(f"{path}: tensor {name!r}: {b - a} bytes do not hold shape {info['shape']} of {info['dtype']}")
        if a < 0 or base + b > size:
            raise SafetensorsError(f"{path}: tensor {name!r} lies outside the file (truncated?)")
    return header, base


class SafetensorsFile:
    """A memory-mapped safetensors file; ``tensor(name)`` is a CPU view (no copy)."""

    def __init__(self, path: str):
        self.path = path
        self.header, self.base = read_safetensors_header(path)
        self._f = open(path, "rb")
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if os.path.getsize(path) else None

    def names(self) -> List[str]:
        return list(self.header)

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(self.header[name]["shape"])

    def dtype(self, name: str) -> torch.dtype:
        return DTYPES[self.header[name]["dtype"]]

    def tensor(self, name: str) -> torch.Tensor:
        info = self.header[name]
        a, b = info["data_offsets"]
        dt = DTYPES[info["dtype"]]
        if b == a:
            return torch.empty(tuple(info["shape"]), dtype=dt)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")     # the map is read-only; nothing writes through the view
            t = torch.frombuffer(self._mm, dtype=dt, count=(b - a) // torch.empty(0, dtype=dt).element_size(),
                                 offset=self.base + a)
        return t.view(tuple(info["shape"]))

    def close(self) -> None:
        # views may still point into the map: it is closed when they are gone
        self._f.close()


def open_safetensors(folder: str) -> List[SafetensorsFile]:
    """The weight files of a model folder: ``model.safetensors``, or the shards that
    ``model.safetensors.index.json`` names."""
    single = os.path.join(folder, "model.safetensors")
    index = os.path.join(folder, "model.safetensors.index.json")
    if os.path.isfile(single):
        return [SafetensorsFile(single)]
    if os.path.isfile(index):
        try:
            with open(index) as f:
                weight_map = json.load(f)["weight_map"]
            shards = sorted(set(weight_map.values()))
        except (json.JSONDecodeError, UnicodeDecodeError, KeyError, TypeError, AttributeError) as e:
            raise SafetensorsError(f"{index}: no JSON object with a 'weight_map' from tensor names to files ({type(e).__name__}: {e})") from None
        absent = [s for s in shards if not os.path.isfile(os.path.join(folder, str(s)))]
        if absent:
            raise SafetensorsError(f"{index} names files that are not in {folder!r}: {', '.join(map(str, absent))}")
        return [SafetensorsFile(os.path.join(folder, s)) for s in shards]
    raise SafetensorsError(f"no model.safetensors (or model.safetensors.index.json) in {folder!r}")


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor]) -> None:
    header = {}
    offset = 0
    items = []
    for name in sorted(tensors):
        t = tensors[name].detach().cpu().contiguous()
        if t.dtype not in NAMES:
            raise SafetensorsError(f"tensor {name!r}: dtype {t.dtype} cannot be written")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
        items.append(t)
    blob = json.dumps(header, separators=(",", ":")).encode()
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for t in items:
            f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
