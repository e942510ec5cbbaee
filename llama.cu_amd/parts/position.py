"""Position encodings of the attention mixer.

A position encoding tells the attention mixer how queries and keys depend on a
token's place.  The interface:

  ``load(build)``                       make tables on the device
  ``rotary_tables() -> (cos, sin, rot_dim, pairing) or None``
        if not None, the mixer applies the rotation in the same kernel that writes
        keys and values to the cache;
  ``apply(qkv, positions, heads, kv_heads, head_dim)``
        any other change of queries and keys, in place, before the cache write
        (the default does nothing);
  ``score_slopes() -> float32 [heads] or None``
        a bias inside the scores that grows with the distance between key and query
        (the default: none).
"""
from __future__ import annotations

import weakref

import numpy as np
import torch

from .base import BuildContext, Part, register_part


class NoPosition(Part):
    graph_safe = True

    """Queries and keys are used as they are."""

    def load(self, tensors, build: BuildContext) -> None:
        pass

    def score_slopes(self):
        """None, or float32 [heads] on the device: the encoding is (also) a bias inside the scores,
        ``slope[h] * (key position - query position)`` added to the scaled score.  The mixer hands it to
        the attention kernel (the generic one: the matrix-core kernels take no bias)."""
        return None


class _Tables:
    """The cosine and sine tables of one (theta, rotated dims, positions) on one device."""

    def __init__(self, cos: torch.Tensor, sin: torch.Tensor):
        self.cos, self.sin = cos, sin


# The tables depend on (theta, rotated dims, positions, device) alone, so the layers of a model that agree in
# these share one pair: 32 layers at 131,072 positions would else build and hold 32 x 67 MB.  The table lives as
# long as a part holds it.
_tables: "weakref.WeakValueDictionary" = weakref.WeakValueDictionary()


class Rotary(NoPosition):
    """Rotation of pairs of dims by ``pos * theta^(-2i/rot_dim)``.

    The tables follow llama.cu/src/model/mod.rs:200-209: the frequency
    ``theta^(-2i/dh)`` and the angle ``pos * freq`` are 32-bit values; the table holds
    the sine and cosine of that 32-bit angle (taken in 64-bit, rounded once).  The
    pairing is a parameter: ``interleaved`` pairs neighbours ``(2i, 2i+1)`` as
    llama.cu/src/op/rope.cuh:21-34 does; otherwise ``(i, i + rot_dim/2)``, the order in
    which files with config.json's tensor names hold the rows of q and k.
    """

    def __init__(self, head_dim: int, theta: float, max_positions: int, interleaved: bool = False,
                 rot_dim: int = 0):
        self.head_dim = int(head_dim)
        self.rot_dim = int(rot_dim) if rot_dim else int(head_dim)
        if self.rot_dim % 2 or self.rot_dim > self.head_dim:
            raise ValueError(f"rotary: rot_dim {self.rot_dim} must be even and at most head_dim {self.head_dim}")
        self.theta = float(theta)
        self.max_positions = int(max_positions)
        self.interleaved = bool(interleaved)
        self.cos = self.sin = None

    def host_tables(self):
        half = self.rot_dim // 2
        # 32-bit throughout, as the reference: theta.powf(-((2 * i) as f32 / dh as f32))
        expo = -(np.float32(2.0) * np.arange(half, dtype=np.float32) / np.float32(self.rot_dim))
        freq = np.power(np.float32(self.theta), expo.astype(np.float32)).astype(np.float32)
        pos = np.arange(self.max_positions, dtype=np.float32)
        ang = (pos[:, None] * freq[None, :]).astype(np.float32).astype(np.float64)   # the 32-bit product
        return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)

    def load(self, tensors, build: BuildContext) -> None:
        key = (self.theta, self.rot_dim, self.max_positions, str(torch.device(build.device)))
        tables = _tables.get(key)
        if tables is None:
            cos, sin = self.host_tables()
            tables = _tables[key] = _Tables(torch.from_numpy(cos).to(build.device).contiguous(),
                                            torch.from_numpy(sin).to(build.device).contiguous())
        self._tables = tables                  # keeps the shared pair alive
        self.cos, self.sin = tables.cos, tables.sin

    def rotary_tables(self):
        return self.cos, self.sin, self.rot_dim, 1 if self.interleaved else 0


register_part("position", "none", NoPosition)
register_part("position", "rotary", Rotary)
