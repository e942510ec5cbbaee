"""Binding the tensors of a model folder to the model's parts.

The model says which tensors it expects, by full name with their shapes
(``DecoderModel.tensors()``).  The files are checked against that list as a whole: one
error names every missing tensor, every unexpected one and every wrong shape.  (The
reference looks tensors up one by one and panics at the first miss,
llama.cu/src/model/mod.rs:80-88.)

Types: with the bfloat16 compute type, floating tensors are kept in bfloat16, except
that a tensor its file stores in 32-bit stays 32-bit (the kernels take a 32-bit norm
weight, table or matrix beside bfloat16 activations); integer tables become int32.
With the float32 compute type every floating tensor becomes float32, which is exact
for bfloat16 and float16 files.
"""
from __future__ import annotations

import re
from typing import Dict, List, Tuple

import torch

from ..parts.base import TensorSpec
from .safetensors_io import SafetensorsFile

# tensors that files of this ecosystem may carry and that hold no weights
IGNORED = [re.compile(r".*\.rotary_emb\.inv_freq$")]


class WeightError(ValueError):
    """The weight files do not fit the model; the message lists every problem."""


def check_tensors(expected: Dict[str, TensorSpec], found: Dict[str, Tuple[int, ...]]) -> None:
    """Raise one WeightError that lists missing and unexpected tensors and wrong shapes."""
    missing = sorted(n for n, s in expected.items() if n not in found and not s.optional)
    unexpected = sorted(n for n in found if n not in expected and not any(p.match(n) for p in IGNORED))
    wrong = sorted((n, tuple(found[n]), tuple(s.shape)) for n, s in expected.items()
                   if n in found and tuple(found[n]) != tuple(s.shape))
    if not (missing or unexpected or wrong):
        return
    lines = ["the weight files do not fit the model:"]
    if missing:
        lines.append(f"  missing tensors ({len(missing)}):")
        lines += [f"    {n}  expected shape {list(expected[n].shape)}" for n in missing]
    if unexpected:
        lines.append(f"  unexpected tensors ({len(unexpected)}):")
        lines += [f"    {n}  shape {list(found[n])}" for n in unexpected]
    if wrong:
        lines.append(f"  wrong shapes ({len(wrong)}):")
        lines += [f"    {n}  found {list(f)}, expected {list(e)}" for n, f, e in wrong]
    raise WeightError("\n".join(lines))


def convert(t: torch.Tensor, spec: TensorSpec, compute: torch.dtype) -> torch.Tensor:
    if spec.integer:
        if t.is_floating_point():
            raise WeightError(f"an integer table is stored as {t.dtype}")
        return t.to(torch.int32)
    if not t.is_floating_point():
        raise WeightError(f"a floating tensor is stored as {t.dtype}")
    if compute == torch.float32:
        return t.to(torch.float32)
    if t.dtype in (torch.float32, torch.float64):
        return t.to(torch.float32)           # stored in 32-bit (or more): stays 32-bit
    return t.to(torch.bfloat16)


def load_weights(files: List[SafetensorsFile], expected: Dict[str, TensorSpec], compute: torch.dtype,
                 device: torch.device) -> Dict[str, torch.Tensor]:
    """All expected tensors, checked, converted and on ``device``."""
    where: Dict[str, SafetensorsFile] = {}
    dup = []
    for f in files:
        for n in f.names():
            if n in where:
                dup.append(n)
            where[n] = f
    if dup:
        raise WeightError("tensors that more than one file holds: " + ", ".join(sorted(dup)))
    check_tensors(expected, {n: f.shape(n) for n, f in where.items()})
    out: Dict[str, torch.Tensor] = {}
    for n, spec in expected.items():
        if n not in where:
            continue
        try:
            t = where[n].tensor(n)
            out[n] = convert(t.to(device, non_blocking=False), spec, compute)
        except WeightError as e:
            raise WeightError(f"tensor {n!r}: {e}") from None
    return out
