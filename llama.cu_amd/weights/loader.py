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
from dataclasses import dataclass
from typing import Dict, List, Sequence, Tuple

import torch

from ..parts.base import TensorSpec
from .safetensors_io import SafetensorsFile


class WeightError(ValueError):
    """The weight files do not fit the model; the message lists every problem."""


def check_tensors(expected: Dict[str, TensorSpec], found: Dict[str, Tuple[int, ...]], ignored: Sequence[str] = ()) -> None:
    """Raise one WeightError that lists missing and unexpected tensors and wrong shapes.  ``ignored``: regular
    expressions for tensors that the files may hold beside the weights (the architecture's registry entry names
    them); they are passed over."""
    patterns = [re.compile(p) for p in ignored]
    missing = sorted(n for n, s in expected.items() if n not in found and not s.optional)
    unexpected = sorted(n for n in found if n not in expected and not any(p.match(n) for p in patterns))
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


def final_dtype(stored: torch.dtype, spec: TensorSpec, compute: torch.dtype) -> torch.dtype:
    """The type ``convert`` gives a tensor that its file stores as ``stored``."""
    return convert(torch.empty(0, dtype=stored), spec, compute).dtype


ALIGN = 256               # every tensor (or group of fused tensors) starts at a multiple of this in the arena
STAGE_BYTES = 64 << 20    # size of each of the two pinned host buffers that the copies go through


@dataclass(frozen=True)
class FusedGroup:
    """Tensors that a part multiplies as one matrix (rows of the first, then of the second, ...):
    the loader lays them out one after the other, so that ``fused_rows`` finds the fused matrix in
    place and nothing is concatenated.  ``pad_rows_to``: every member is followed by rows of zeros up
    to this many rows (0: none)."""
    names: Tuple[str, ...]
    pad_rows_to: int = 0


def _rounded(n: int, to: int) -> int:
    return (n + to - 1) // to * to


def plan_arena(expected: Dict[str, TensorSpec], stored: Dict[str, torch.dtype], compute: torch.dtype,
               groups: Sequence[FusedGroup] = ()) -> Tuple[Dict[str, Tuple[int, torch.dtype]], int]:
    """Where every tensor that the files hold goes in one allocation: ``{name: (byte offset, type)}``
    and the size.  A group's members stand one after the other without a gap (and with their rows of
    zeros), if they are all there, 2-d, of one width and of one final type; else each stands alone."""
    place: Dict[str, Tuple[int, torch.dtype]] = {}
    at = 0

    def size(n, rows=None):
        shape = expected[n].shape
        count = 1
        for k, dim in enumerate(shape):
            count *= (rows if (rows and k == 0) else dim)
        return count * torch.empty(0, dtype=final[n]).element_size()

    final = {n: final_dtype(stored[n], expected[n], compute) for n in expected if n in stored}
    for g in groups:
        names = [n for n in g.names]
        ok = all(n in final and len(expected[n].shape) == 2 for n in names) and \
            len({(final[n], expected[n].shape[1]) for n in names}) == 1 and \
            all(not g.pad_rows_to or expected[n].shape[0] <= g.pad_rows_to for n in names)
        if not ok or any(n in place for n in names):
            continue
        at = _rounded(at, ALIGN)
        for n in names:
            place[n] = (at, final[n])
            at += size(n, g.pad_rows_to or None)
    for n in expected:
        if n in final and n not in place:
            at = _rounded(at, ALIGN)
            place[n] = (at, final[n])
            at += size(n)
    return place, _rounded(at, ALIGN)


class _Stager:
    """Bytes from host memory (a memory-mapped file) to the device through two pinned buffers in
    turn: while one buffer's copy to the device is on its way, the next piece is copied into the
    other (the reference stages through pinned slabs the same way, llama.cu/src/load/loader.rs:28-60)."""

    def __init__(self, device: torch.device):
        self.device = device
        self.cuda = device.type == "cuda"
        self.buffers = [torch.empty(STAGE_BYTES, dtype=torch.uint8, pin_memory=True) for _ in range(2)] if self.cuda else []
        self.free = [None, None]          # the event after which a buffer may be written again
        self.turn = 0

    def copy(self, dst: torch.Tensor, src: torch.Tensor) -> None:
        """``dst`` (uint8, on the device, contiguous) takes the bytes of ``src`` (uint8, on the host)."""
        n = src.numel()
        if not self.cuda:
            dst.copy_(src)
            return
        for a in range(0, n, STAGE_BYTES):
            b = min(a + STAGE_BYTES, n)
            k = self.turn
            self.turn ^= 1
            if self.free[k] is not None:
                self.free[k].synchronize()
            self.buffers[k][:b - a].copy_(src[a:b])
            dst[a:b].copy_(self.buffers[k][:b - a], non_blocking=True)
            self.free[k] = torch.cuda.Event()
            self.free[k].record()

    def finish(self) -> None:
        for e in self.free:
            if e is not None:
                e.synchronize()


def load_weights(files: List[SafetensorsFile], expected: Dict[str, TensorSpec], compute: torch.dtype,
                 device: torch.device, groups: Sequence[FusedGroup] = (), log=None,
                 ignored: Sequence[str] = ()) -> Dict[str, torch.Tensor]:
    """All expected tensors, checked, converted and on ``device``, as views of one allocation
    (the reference lays all weights out in one region too, llama.cu/src/load/mod.rs:28-44).  The
    members of a fused group stand one after the other in it.  The bytes go through pinned host
    buffers, two in turn; a tensor whose file stores another type than the engine keeps is staged
    on the device and converted there, so the most that is ever allocated beside the weights
    themselves is one tensor.  ``log``: a function that takes the line with the size and the rate
    (llama.cu/src/load/mod.rs:110-117 logs the same).  ``ignored``: as in ``check_tensors``."""
    import time
    device = torch.device(device)
    where: Dict[str, SafetensorsFile] = {}
    dup = []
    for f in files:
        for n in f.names():
            if n in where:
                dup.append(n)
            where[n] = f
    if dup:
        raise WeightError("tensors that more than one file holds: " + ", ".join(sorted(dup)))
    check_tensors(expected, {n: f.shape(n) for n, f in where.items()}, ignored)
    stored = {n: where[n].dtype(n) for n in expected if n in where}
    for n, dt in stored.items():
        try:
            final_dtype(dt, expected[n], compute)
        except WeightError as e:
            raise WeightError(f"tensor {n!r}: {e}") from None
    place, total = plan_arena(expected, stored, compute, groups)
    t0 = time.time()
    arena = torch.zeros(total, dtype=torch.uint8, device=device)          # rows of zeros between fused members stay zero
    stager = _Stager(device)
    out: Dict[str, torch.Tensor] = {}
    for n, (at, dt) in place.items():
        spec = expected[n]
        src = where[n].tensor(n)
        nbytes = src.numel() * torch.empty(0, dtype=dt).element_size()
        view = arena[at:at + nbytes].view(dt).view(tuple(spec.shape))
        raw = src.reshape(-1).view(torch.uint8)
        if src.dtype == dt:
            stager.copy(arena[at:at + nbytes], raw)
        else:
            stage = torch.empty(raw.numel(), dtype=torch.uint8, device=device)     # one tensor as its file holds it
            stager.copy(stage, raw)
            view.copy_(stage.view(src.dtype).view(tuple(spec.shape)))             # converted on the device
            del stage
        out[n] = view
    stager.finish()
    if device.type == "cuda":
        torch.cuda.synchronize(device)
    seconds = max(time.time() - t0, 1e-9)
    if log is not None:
        log(f"weights: {len(out)} tensors, {total / 1e9:.2f} GB in one allocation, {seconds:.2f} s ({total / 1e9 / seconds:.2f} GB/s)")
    return out


def fused_rows(parts: Sequence[torch.Tensor], pad_rows_to: int = 0) -> torch.Tensor:
    """The matrix whose rows are those of ``parts`` one after the other (each followed by rows of
    zeros up to ``pad_rows_to`` rows): a view, if the loader laid them out so; else a new tensor."""
    first = parts[0]
    rows = [pad_rows_to or p.shape[0] for p in parts]
    elem = first.element_size()
    adjacent = all(p.dim() == 2 and p.is_contiguous() and p.dtype == first.dtype and p.shape[1] == first.shape[1]
                   and p.device == first.device for p in parts)
    if adjacent:
        at = first.data_ptr()
        for p, r in zip(parts, rows):
            adjacent = adjacent and p.data_ptr() == at and p.untyped_storage().data_ptr() == first.untyped_storage().data_ptr()
            at += r * first.shape[1] * elem
    if adjacent:
        end = first.storage_offset() + sum(rows) * first.shape[1]
        if end * elem <= first.untyped_storage().nbytes():
            return torch.as_strided(first, (sum(rows), first.shape[1]), (first.shape[1], 1), first.storage_offset())
    if len({p.dtype for p in parts}) != 1:
        parts = [p.float() for p in parts]
    pieces = []
    for p, r in zip(parts, rows):
        pieces.append(p)
        if r > p.shape[0]:
            pieces.append(torch.zeros((r - p.shape[0], p.shape[1]), dtype=p.dtype, device=p.device))
    return torch.cat(pieces, dim=0)
