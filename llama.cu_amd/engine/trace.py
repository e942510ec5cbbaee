"""Trace replay: given token ids go through the model step by step and logits come
out.  Nothing is sampled.  It drives the same runner, step function, cache manager and
kernels that generation uses.

A step is a JSON object ``{"step": k, "entries": [{"id": "a", "tokens": [...], "want":
[...]}, ...], "end": ["a", ...], "preempt": ["b", ...]}``: every entry is a request's next
tokens and the places among them whose logits are wanted; all entries of a step are one
batch; ``end`` names requests that are finished after this step (their pages are given
back); ``preempt`` names requests that lose their pages after this step but go on later:
the next step that names such a request computes all its earlier tokens again, in the same
batch as its new ones (what the scheduler does with a request it had to preempt).
"""
from __future__ import annotations

import os
from typing import Any, Dict, List, Optional

import numpy as np
import torch

from .runner import ModelRunner

PAGE_SIZE = 16            # the default: divides 64, so a request's pages never exceed its count rounded up to 64
MAX_LIVE = 8              # the default number of state slots (a trace holds up to four live requests)


class TraceReplayer:
    def __init__(self, runner: ModelRunner):
        """Replays on ``runner`` (``open`` makes one for a model folder)."""
        self.runner = runner
        self.ids: Dict[Any, int] = {}
        self.next_id = 0
        self.preempted: set = set()
        # what a test may ask afterwards: which requests held each page of each group in turn, and how many
        # steps held a portion of several tokens beside a single token
        self.page_users: List[Dict[int, set]] = [dict() for _ in self.runner.groups]
        self.mixed_steps = 0
        self.fed: Dict[Any, List[int]] = {}       # every live request's tokens so far (a preempted one is computed again)

    @classmethod
    def open(cls, model_dir: str, dtype: str, max_tokens: int, device: str = "cuda:0", page_size: int = PAGE_SIZE,
             num_pages: Optional[int] = None, max_live: int = MAX_LIVE, random_weights: Optional[int] = None,
             poison_freed: bool = False) -> "TraceReplayer":
        """``max_tokens``: the most tokens that live requests hold at a time, each request's count
        rounded up to a multiple of 64; the pool is made for that many (``num_pages`` overrides it).
        ``random_weights``: a seed; the folder then needs config.json only.  ``poison_freed``: pages
        that are given back are filled with NaN (a read of memory that no live request owns shows)."""
        if dtype not in ("bfloat16", "float32"):
            raise ValueError(f"--dtype must be bfloat16 or float32, got {dtype!r}")
        max_tokens = max(int(max_tokens), page_size)
        kw = dict(dtype=dtype, device=device, page_size=page_size, max_seqs=int(max_live),
                  max_batch_tokens=max_tokens, max_model_len=None, poison_freed=poison_freed)
        if num_pages is not None:
            kw["num_pages"] = int(num_pages)
        else:
            kw["max_tokens"] = max_tokens
        if random_weights is None:
            return cls(ModelRunner.from_folder(model_dir, **kw))
        from .. import models  # noqa: F401  (registers the architectures)
        from ..config import load_config
        _, cfg = load_config(model_dir)
        return cls(ModelRunner.from_config(cfg, int(random_weights), **kw))

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
            tokens, want = [], []
            for e in entries:
                new = [int(t) for t in e["tokens"]]
                places = [int(k) for k in e.get("want", [])]
                before = self.fed.setdefault(e["id"], [])
                if e["id"] in self.preempted:           # its cache is gone: everything again, the new tokens at the end
                    self.preempted.discard(e["id"])
                    tokens.append(before + new)
                    want.append([len(before) + k for k in places])
                else:
                    tokens.append(new)
                    want.append(places)
                before.extend(new)
            logits = self.runner.step(ids, tokens, want)
            sizes = [len(t) for t in tokens]
            self.mixed_steps += int(min(sizes) == 1 and max(sizes) > 1)
            for g, users in enumerate(self.page_users):
                for page, owner in enumerate(self.runner.cache.page_owners(g)):
                    if owner >= 0:
                        users.setdefault(page, set()).add(owner)
            if logits.shape[0]:
                out = logits.detach().to("cpu", torch.float32).numpy()
        for name in obj.get("preempt", []):
            if name in self.ids and name not in self.preempted:
                self.runner.end(self.ids[name])
                self.preempted.add(name)
        for name in obj.get("end", []):
            if name in self.ids:
                self.runner.end(self.ids.pop(name))
            self.fed.pop(name, None)
            self.preempted.discard(name)
        torch.cuda.synchronize()
        return out


    def pages_used_again(self, group: int = 0) -> int:
        """How many pages of ``group`` more than one request has held so far."""
        return sum(1 for users in self.page_users[group].values() if len(users) > 1)


def write_logits(out_dir: str, step, logits: np.ndarray) -> str:
    path = os.path.join(out_dir, f"{step}.f32")
    logits.astype("<f4", copy=False).tofile(path)
    return path
