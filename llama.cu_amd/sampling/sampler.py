"""Sampling on the device from rows of float32 logits (kernels: csrc/kernels/sampling.hip).

The uniform number of a draw comes from a counter-based generator keyed by the
request's seed, its id and the index of the token it draws: a request's tokens do not
depend on what else is in the batch or on how its prompt was cut.
"""
from __future__ import annotations

import ctypes
from typing import List, Sequence, Tuple

import torch

from ..kernels import build, ops
from ..kernels.ops import KernelError, _check, _gpu, _ptr, _stream, to_device as _to_device
from .params import SamplingParams

_MASK = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform(seed: int, request: int, index: int) -> float:
    """A number in [0, 1) with 24 random bits, a pure function of its three keys."""
    h = _splitmix64(seed & _MASK)
    h = _splitmix64(h ^ (request & _MASK))
    h = _splitmix64(h ^ (index & _MASK))
    return (h >> 40) / float(1 << 24)


def argmax(logits: torch.Tensor) -> torch.Tensor:
    """The index of the largest logit of each row (the lowest among equals), int32."""
    _gpu(logits)
    if logits.dim() != 2 or logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise KernelError("argmax: logits must be float32 [rows, vocab] with contiguous rows")
    rows, vocab = logits.shape
    out = torch.empty(rows, dtype=torch.int32, device=logits.device)
    # a long row is read by several workgroups, whose winners a second kernel compares
    parts = max(1, min(16, vocab // 8192))
    part_val = torch.empty(rows * parts, dtype=torch.float32, device=logits.device) if parts > 1 else None
    part_idx = torch.empty(rows * parts, dtype=torch.int32, device=logits.device) if parts > 1 else None
    lib = build.load("sampling")
    _check(lib.lcu_argmax(_ptr(logits), logits.stride(0), rows, vocab, _ptr(out), parts, _ptr(part_val), _ptr(part_idx),
                          _stream()), "argmax")
    return out


def sample_rows(logits: torch.Tensor, temperature: Sequence[float], top_p: Sequence[float], top_k: Sequence[int],
                u: Sequence[float]) -> torch.Tensor:
    """One draw per row with the row's temperature (> 0), top_p, top_k and uniform number."""
    _gpu(logits)
    if logits.dim() != 2 or logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise KernelError("sample: logits must be float32 [rows, vocab] with contiguous rows")
    rows, vocab = logits.shape
    if not (len(temperature) == len(top_p) == len(top_k) == len(u) == rows):
        raise KernelError("sample: one temperature, top_p, top_k and uniform number per row")
    if any(not t > 0 for t in temperature) or any(not 0 <= x < 1 for x in u):
        raise KernelError("sample: temperatures must be > 0 and uniform numbers in [0, 1)")
    dev = logits.device
    fl = _to_device([list(temperature), list(top_p), list(u)], torch.float32, dev)
    kk = _to_device([min(int(k), vocab) for k in top_k], torch.int32, dev)
    out = torch.empty(rows, dtype=torch.int32, device=dev)
    lib = build.load("sampling")
    # a long row is cut into parts, one workgroup each: about one workgroup per compute unit in all
    parts = max(1, min(16, 256 // rows, vocab // 4096))
    lib.lcu_sample_scratch_bytes.restype = ctypes.c_size_t
    scratch = torch.zeros(int(lib.lcu_sample_scratch_bytes(rows, parts)), dtype=torch.uint8, device=dev)
    any_top_k = any(int(k) < vocab for k in top_k)
    _check(lib.lcu_sample(_ptr(logits), logits.stride(0), rows, vocab, _ptr(fl[0]), _ptr(fl[1]), _ptr(kk), _ptr(fl[2]),
                          _ptr(out), int(any_top_k), parts, _ptr(scratch), _stream()), "sample")
    return out


def token_logprobs(logits: torch.Tensor, tokens: torch.Tensor) -> torch.Tensor:
    """``log softmax(logits[r])[tokens[r]]`` for every row: the natural logarithm of the probability that the model
    gives each row's token (float32, on the device).  The reference hands back the chosen token's value beside its
    index (``KVPair``, llama.cu/src/op/random_sample/mod.rs:29-36); this is that value made comparable across rows."""
    _gpu(logits, tokens)
    if logits.dim() != 2 or logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise KernelError("token_logprobs: logits must be float32 [rows, vocab] with contiguous rows")
    rows, vocab = logits.shape
    if tokens.dtype != torch.int32 or tokens.numel() != rows or not tokens.is_contiguous():
        raise KernelError(f"token_logprobs: tokens must be a contiguous int32 tensor of {rows} entries")
    out = torch.empty(rows, dtype=torch.float32, device=logits.device)
    lib = build.load("sampling")
    _check(lib.lcu_token_logprob(_ptr(logits), logits.stride(0), rows, vocab, _ptr(tokens), _ptr(out), _stream()), "token_logprobs")
    return out


class Sampler:
    def sample_device(self, logits: torch.Tensor, params: Sequence[SamplingParams],
                      keys: Sequence[Tuple[int, int]]) -> torch.Tensor:
        """A token for every row, left on the device (int32)."""
        random_rows = [i for i, p in enumerate(params) if not p.is_argmax]
        if random_rows and len(random_rows) == logits.shape[0]:
            return sample_rows(logits, [p.temperature for p in params], [p.top_p for p in params], [p.top_k for p in params],
                               [uniform(p.seed, k[0], k[1]) for p, k in zip(params, keys)])
        out = argmax(logits)
        if random_rows:
            # the rows that draw are gathered, drawn from and put back by the engine's own small kernels
            both = _to_device([random_rows, list(range(len(random_rows)))], torch.int32, logits.device)
            sub = ops.gather_rows(logits, both[0])
            drawn = sample_rows(sub, [params[i].temperature for i in random_rows], [params[i].top_p for i in random_rows],
                                [params[i].top_k for i in random_rows],
                                [uniform(params[i].seed, keys[i][0], keys[i][1]) for i in random_rows])
            ops.feed_tokens(out, drawn, both[1], both[0])               # out[random_rows[i]] = drawn[i]
        return out

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams],
               keys: Sequence[Tuple[int, int]]) -> List[int]:
        """A token for every row.  ``keys[i] = (request id, index of the drawn token)``."""
        rows = logits.shape[0]
        if rows == 0:
            return []
        greedy = argmax(logits)
        random_rows = [i for i, p in enumerate(params) if not p.is_argmax]
        if not random_rows:
            return greedy.tolist()
        sub = logits if len(random_rows) == rows else ops.gather_rows(logits, _to_device(random_rows, torch.int32, logits.device))
        drawn = sample_rows(sub, [params[i].temperature for i in random_rows], [params[i].top_p for i in random_rows],
                            [params[i].top_k for i in random_rows],
                            [uniform(params[i].seed, keys[i][0], keys[i][1]) for i in random_rows]).tolist()
        out = greedy.tolist()
        for i, t in zip(random_rows, drawn):
            out[i] = t
        return out
