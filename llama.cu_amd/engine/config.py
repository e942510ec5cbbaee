"""The engine's own constants as one typed record (the model's come from config.json).

The reference holds its counterparts in code: the token-count buckets, the depth of its input buffers and
``max_steps``'s default (llama.cu/src/exec/engine.rs:68,209; llama.cu/xtask/src/main.rs:70-72).
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from typing import Any, Dict, Optional


@dataclass(frozen=True)
class EngineConfig:
    dtype: str = "bfloat16"                 # the compute type: "bfloat16" or "float32" (true 32-bit everywhere)
    device: str = "cuda:0"
    page_size: int = 16                     # tokens per page of the cache (a multiple of 8; of 16 for the matrix-core attention)
    num_pages: Optional[int] = None         # pages in the pool; or
    max_tokens: Optional[int] = None        # tokens the pool holds; neither: what kv_fraction of the free memory holds
    kv_fraction: float = 0.85
    max_seqs: int = 8                       # requests that run at a time (and state slots)
    max_batch_tokens: int = 2048            # tokens per step
    prefill_chunk: Optional[int] = None     # most tokens of one prompt per step (default: max_batch_tokens)
    max_model_len: Optional[int] = None     # most tokens a request may hold (default, and at most: the model's positions)
    use_graphs: bool = True                 # replay decode steps from captured graphs
    pack_weights: Optional[bool] = None     # a second copy of the matrices in the decode kernels' order (default: if memory allows)
    run_ahead: bool = True                  # launch a round before the round before has been read
    logprobs: bool = False                  # every sampled token comes with the log of the probability the model gave it
    poison_freed: bool = False              # debugging: fill pages that change hands with NaN

    def __post_init__(self):
        def fail(field, why):
            raise ValueError(f"engine configuration: {field} = {getattr(self, field)!r} {why}")
        if self.dtype not in ("bfloat16", "bf16", "float32", "f32", "fp32"):
            fail("dtype", "is neither bfloat16 nor float32")
        for f in ("page_size", "max_seqs", "max_batch_tokens"):
            if not isinstance(getattr(self, f), int) or getattr(self, f) <= 0:
                fail(f, "must be a positive integer")
        if self.page_size % 8:
            fail("page_size", "must be a multiple of 8")
        for f in ("num_pages", "max_tokens", "prefill_chunk", "max_model_len"):
            v = getattr(self, f)
            if v is not None and (not isinstance(v, int) or v <= 0):
                fail(f, "must be a positive integer or None")
        if self.num_pages is not None and self.max_tokens is not None:
            fail("num_pages", "and max_tokens both give the pool's size: name one")
        if not 0.0 < float(self.kv_fraction) <= 1.0:
            fail("kv_fraction", "must lie in (0, 1]")

    @classmethod
    def of(cls, config: Optional["EngineConfig"] = None, **overrides: Any) -> "EngineConfig":
        """``config`` (or the defaults) with ``overrides``; a name that is no field is an error that lists the fields."""
        names = [f.name for f in dataclasses.fields(cls)]
        unknown = sorted(set(overrides) - set(names))
        if unknown:
            raise TypeError(f"engine configuration: no field {unknown}; fields: {names}")
        return dataclasses.replace(config or cls(), **overrides)

    def runner_kwargs(self) -> Dict[str, Any]:
        """What ``ModelRunner`` takes (the scheduler's and the engine's own fields apart)."""
        kw = {k: getattr(self, k) for k in ("dtype", "device", "page_size", "max_seqs", "max_batch_tokens", "max_model_len",
                                             "kv_fraction", "use_graphs", "pack_weights", "poison_freed")}
        if self.num_pages is not None:
            kw["num_pages"] = self.num_pages
        if self.max_tokens is not None:
            kw["max_tokens"] = self.max_tokens
        return kw
