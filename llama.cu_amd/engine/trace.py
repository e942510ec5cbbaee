"""Trace replay: given token ids go through the model step by step and logits come
out.  Nothing is sampled.  It drives the same runner, step function, cache manager and
kernels that generation uses.

A step is a JSON object ``{"step": k, "entries": [{"id": "a", "tokens": [...], "want":
[...]}, ...], "end": ["a", ...]}``: every entry is a request's next tokens and the
places among them whose logits are wanted; all entries of a step are one batch;
``end`` names requests that are finished after this step (their pages are given back).
"""
from __future__ import annotations

import os
from typing import Any, Dict, List, Optional

import numpy as np
import torch

from .runner import DTYPES, ModelRunner

PAGE_SIZE = 16            # divides 64: a request's pages never exceed its count rounded up to 64
MAX_LIVE = 8              # state slots (a trace holds up to four live requests)


class TraceReplayer:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int, device: str = "cuda:0",
                 page_size: int = PAGE_SIZE):
        if dtype not in ("bfloat16", "float32"):
            raise ValueError(f"--dtype must be bfloat16 or float32, got {dtype!r}")
        max_tokens = max(int(max_tokens), page_size)
        self.runner = ModelRunner.from_folder(
            model_dir, dtype=dtype, device=device, page_size=page_size, max_tokens=max_tokens,
            max_seqs=MAX_LIVE, max_batch_tokens=max_tokens, max_model_len=None)
        self.ids: Dict[Any, int] = {}
        self.next_id = 0

    def _rid(self, name) -> int:
        if name not in self.ids:
            self.ids[name] = self.next_id
            self.next_id += 1
        return self.ids[name]

    def step(self, obj: Dict[str, Any]) -> Optional[np.ndarray]:
        """Run one step; returns the wanted logits ``[wanted, vocab]`` (float32) or None if
        nothing was wanted."""
        entries = [e for e in obj.get("entries", []) if len(e.get("tokens", [])) > 0]
        out = None
        if entries:
            names = [e["id"] for e in entries]
            if len(set(names)) != len(names):
                raise ValueError(f"step {obj.get('step')}: a request appears twice in one step")
            ids = [self._rid(n) for n in names]
            tokens = [list(e["tokens"]) for e in entries]
            want = [list(e.get("want", [])) for e in entries]
            logits = self.runner.step(ids, tokens, want)
            if logits.shape[0]:
                out = logits.detach().to("cpu", torch.float32).numpy()
        for name in obj.get("end", []):
            if name in self.ids:
                self.runner.end(self.ids.pop(name))
        torch.cuda.synchronize()
        return out


def write_logits(out_dir: str, step, logits: np.ndarray) -> str:
    path = os.path.join(out_dir, f"{step}.f32")
    logits.astype("<f4", copy=False).tofile(path)
    return path
