"""Random weights from a configuration and a seed: matrices N(0, std), norm weights
1 + N(0, std).  The reference has no such mode; it exists so that the engine can be tested
against a plain implementation and measured without any file.

One generator for the host and the GPU (csrc/shared/random_normal.h, compiled into the host
library and into the kernel of csrc/kernels/random_fill.hip): element ``i`` of a tensor is a
function of (seed, tensor name, i) alone, so a model that is made on the GPU from a seed is,
bit for bit, the model that ``write_random_model`` writes to a folder from the same seed, and a
tensor's values do not depend on which other tensors the model has.  Tensors are made under the
names that files use, before anything is fused.
"""
from __future__ import annotations

import ctypes
import json
import os
from typing import Callable, Dict, List

import torch

from ..parts.base import TensorSpec
from .safetensors_io import write_safetensors

_MASK = (1 << 64) - 1
_GOLDEN = 0x9E3779B97F4A7C15


def _mix64(z: int) -> int:
    z &= _MASK
    z ^= z >> 30
    z = (z * 0xBF58476D1CE4E5B9) & _MASK
    z ^= z >> 27
    z = (z * 0x94D049BB133111EB) & _MASK
    z ^= z >> 31
    return z


def _fnv1a64(text: str) -> int:
    h = 0xCBF29CE484222325
    for b in text.encode():
        h = ((h ^ b) * 0x100000001B3) & _MASK
    return h


def stream_key(seed: int, name: str) -> int:
    """The key of the stream of tensor ``name`` under ``seed``."""
    return _mix64(_mix64(int(seed) & _MASK) ^ _fnv1a64(name))


def fill_normal(out: torch.Tensor, key: int, std: float, shift: float = 0.0) -> torch.Tensor:
    """``out[i] = normal(key, i) * std + shift`` over the flattened, contiguous tensor ``out``
    (float32 or bfloat16), on the host or on the GPU: the same bits on both."""
    if out.dtype not in (torch.float32, torch.bfloat16) or not out.is_contiguous():
        raise ValueError("fill_normal: a contiguous float32 or bfloat16 tensor is needed")
    if out.is_cuda:
        from ..kernels import ops
        return ops.random_fill(out, key, std, shift)
    from ..kernels import build
    lib = build.load(build.HOST_LIBRARY)
    st = lib.lcu_random_fill_host(ctypes.c_void_p(out.data_ptr()), 0 if out.dtype == torch.float32 else 1,
                                  ctypes.c_longlong(out.numel()), ctypes.c_ulonglong(key), ctypes.c_longlong(0),
                                  ctypes.c_float(std), ctypes.c_float(shift), min(8, os.cpu_count() or 1))
    if st:
        raise ValueError(f"fill_normal: the host library refused its arguments ({st})")
    return out


# How the random mode fills a tensor, by the name that ``TensorSpec.init`` holds: ``fill(out, key, std)`` fills the
# contiguous float32 or bfloat16 tensor ``out`` (on the host or on the GPU) in place; ``key`` is the tensor's stream
# (``fill_normal(out, key, ...)`` gives the same bits on both sides), ``std`` the scale that the caller asked for.
_INITIALISERS: Dict[str, Callable[[torch.Tensor, int, float], None]] = {}


def register_initialiser(name: str, fill: Callable[[torch.Tensor, int, float], None], replace: bool = False) -> None:
    """Make ``name`` known as a value of ``TensorSpec.init``: a part whose tensors need another start than a
    normal distribution (zeros, a decay in some range, a bias) registers its own and names it in ``tensors()``."""
    if name in _INITIALISERS and not replace:
        raise ValueError(f"initialiser {name!r} is already registered")
    _INITIALISERS[name] = fill


def registered_initialisers() -> List[str]:
    return sorted(_INITIALISERS)


register_initialiser("normal", lambda out, key, std: fill_normal(out, key, std))                   # N(0, std): matrices
register_initialiser("one_plus_normal", lambda out, key, std: fill_normal(out, key, std, 1.0))    # 1 + N(0, std): norm weights
register_initialiser("zeros", lambda out, key, std: out.zero_())
register_initialiser("ones", lambda out, key, std: out.fill_(1.0))


def random_tensors(expected: Dict[str, TensorSpec], seed: int, dtype: torch.dtype = torch.bfloat16,
                   std: float = 0.02, device="cpu", vector_dtype=None) -> Dict[str, torch.Tensor]:
    """A tensor for every expected name that the random mode makes (a tied model gets no
    output matrix).  ``vector_dtype`` (default: ``dtype``) is the type of 1-d tensors (norm
    weights).  Values are made in 32-bit and rounded once to the tensor's type."""
    out = {}
    dev = torch.device(device)
    for name, spec in expected.items():
        if not spec.random:
            continue
        if spec.integer:
            out[name] = torch.zeros(spec.shape, dtype=torch.int32, device=dev)
            continue
        dt = (vector_dtype or dtype) if len(spec.shape) == 1 else dtype
        made = dt if dt in (torch.float32, torch.bfloat16) else torch.float32
        fill = _INITIALISERS.get(spec.init)
        if fill is None:
            raise ValueError(f"tensor {name!r}: no initialiser {spec.init!r}; registered: {registered_initialisers()}")
        t = torch.empty(spec.shape, dtype=made, device=dev)
        fill(t, stream_key(seed, name), std)
        out[name] = t if made == dt else t.to(dt)
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
