"""Random weights from a configuration and a seed: matrices N(0, std), norm weights
1 + N(0, std), each tensor from its own stream (seed and tensor name), so a tensor's
values do not depend on which other tensors the model has.  The reference has no such
mode; it exists so that the engine can be tested and measured without any file."""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict

import torch

from ..parts.base import TensorSpec
from .safetensors_io import write_safetensors


def _stream_seed(seed: int, name: str) -> int:
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & 0x7FFFFFFFFFFFFFFF


def random_tensors(expected: Dict[str, TensorSpec], seed: int, dtype: torch.dtype = torch.bfloat16,
                   std: float = 0.02, device="cpu", vector_dtype=None) -> Dict[str, torch.Tensor]:
    """A tensor for every expected name that the random mode makes (a tied model gets no
    output matrix).  ``vector_dtype`` (default: ``dtype``)
    is the type of 1-d tensors (norm weights)."""
    out = {}
    dev = torch.device(device)
    for name, spec in expected.items():
        if not spec.random:
            continue
        g = torch.Generator(device=dev).manual_seed(_stream_seed(seed, name))
        if spec.integer:
            out[name] = torch.zeros(spec.shape, dtype=torch.int32, device=dev)
            continue
        t = torch.randn(spec.shape, generator=g, dtype=torch.float32, device=dev) * std
        if spec.init == "one_plus_normal":
            t = t + 1.0
        dt = (vector_dtype or dtype) if len(spec.shape) == 1 else dtype
        out[name] = t.to(dt)
    return out


def write_random_model(folder: str, config, seed: int, dtype: torch.dtype = torch.bfloat16, std: float = 0.02,
                       vector_dtype=None) -> str:
    """Write ``config.json`` and ``model.safetensors`` for ``config`` (a typed
    configuration of a registered architecture) with random weights from ``seed``."""
    from ..config import architecture_of
    from ..parts import DecoderModel
    data = config.to_dict()
    arch = architecture_of(data)
    model = DecoderModel(arch.build_spec(config))
    os.makedirs(folder, exist_ok=True)
    data["torch_dtype"] = {torch.bfloat16: "bfloat16", torch.float32: "float32", torch.float16: "float16"}[dtype]
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(data, f, indent=1)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      random_tensors(model.tensors(), seed, dtype=dtype, std=std, vector_dtype=vector_dtype))
    return folder
