"""Sampling options, with the reference's names, defaults and checks
(llama.cu/src/op/random_sample/mod.rs:38-83): ``temperature``, ``top_p``, ``top_k``; the
default is arg-max; a negative temperature, ``top_k == 0`` or ``top_p <= 0`` is an
error; ``top_p`` above 1 is taken as 1; a draw is arg-max when ``temperature == 0`` or
``top_k == 1``.  ``seed`` is this engine's own: the reference draws from an unseeded
generator (llama.cu/src/exec/output_head.rs:111)."""
from __future__ import annotations

import sys
from dataclasses import dataclass

TOP_K_ALL = sys.maxsize


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0
    top_p: float = 1.0
    top_k: int = TOP_K_ALL
    seed: int = 0

    def __post_init__(self):
        if not self.temperature >= 0:
            raise ValueError(f"temperature must be >= 0, got {self.temperature}")
        if self.top_k is None or self.top_k < 1:
            raise ValueError(f"top_k must be >= 1, got {self.top_k}")
        if not self.top_p > 0:
            raise ValueError(f"top_p must be > 0, got {self.top_p}")
        if self.top_p > 1:
            object.__setattr__(self, "top_p", 1.0)

    @property
    def is_argmax(self) -> bool:
        return self.temperature == 0 or self.top_k == 1


GREEDY = SamplingParams()
