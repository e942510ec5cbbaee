"""The plain C++ references of the kernels (csrc/ref/ref.cpp, part of the host library) as
Python functions on float32 CPU tensors.  They run no GPU code and are what the kernels'
tests compare with, beside the plain Python implementation of the tests."""
from __future__ import annotations

import ctypes
from typing import Optional, Sequence

import torch

from . import build


def _lib() -> ctypes.CDLL:
    return build.load(build.HOST_LIBRARY)


def _f32(t: torch.Tensor, what: str) -> torch.Tensor:
    if t.is_cuda or t.dtype != torch.float32 or not t.is_contiguous():
        raise ValueError(f"{what}: the references take contiguous float32 tensors on the host")
    return t


def _i32(values) -> torch.Tensor:
    return values.to(torch.int32).contiguous() if isinstance(values, torch.Tensor) else torch.tensor(list(values), dtype=torch.int32)


def _p(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def embedding(table: torch.Tensor, ids: Sequence[int]) -> torch.Tensor:
    ids = _i32(ids)
    out = torch.empty(ids.numel(), table.shape[1])
    _lib().lcu_ref_embedding(_p(_f32(table, "table")), _p(ids), ids.numel(), table.shape[1], _p(out))
    return out


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    out = torch.empty_like(_f32(x, "x"))
    _lib().lcu_ref_rms_norm(_p(x), _p(_f32(w, "w")), ctypes.c_float(eps), x.shape[0], x.shape[1], _p(out))
    return out


def gemm_nt(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    out = torch.empty(a.shape[0], w.shape[0])
    _lib().lcu_ref_gemm_nt(_p(_f32(a, "a")), _p(_f32(w, "w")), a.shape[0], w.shape[0], a.shape[1], _p(out))
    return out


def swiglu(gate_up: torch.Tensor) -> torch.Tensor:
    n, two_di = _f32(gate_up, "gate_up").shape
    out = torch.empty(n, two_di // 2)
    _lib().lcu_ref_swiglu(_p(gate_up), n, two_di // 2, _p(out))
    return out


def rope_kv_write(qkv: torch.Tensor, positions, slots, theta: float, heads: int, kv_heads: int, head_dim: int,
                  rot_dim: int, pairing: int, page_size: int, cache: Optional[torch.Tensor]) -> torch.Tensor:
    """Rotates q and k of ``qkv [n, (heads + 2 kv_heads) * head_dim]`` in place and writes k and v into
    ``cache [pages, 2, kv_heads * head_dim * page_size]`` at ``slots``; returns ``qkv``."""
    positions, slots = _i32(positions), _i32(slots)
    _lib().lcu_ref_rope_kv_write(_p(_f32(qkv, "qkv")), qkv.shape[0], _p(positions), _p(slots), ctypes.c_float(theta), heads,
                                 kv_heads, head_dim, rot_dim, pairing, page_size,
                                 _p(None if cache is None else _f32(cache, "cache")))
    return qkv


def paged_attention(q: torch.Tensor, cache: torch.Tensor, block_table: torch.Tensor, q_start, ctx_len, heads: int,
                    kv_heads: int, head_dim: int, page_size: int, scale: float, window: int = 0) -> torch.Tensor:
    """``q [n, >= heads * head_dim]``: rows may be wider than the queries (the q, k, v rows of a step)."""
    block_table, q_start, ctx_len = _i32(block_table), _i32(q_start), _i32(ctx_len)
    out = torch.empty(q.shape[0], heads * head_dim)
    if q.is_cuda or q.dtype != torch.float32 or q.stride(1) != 1:
        raise ValueError("q: the references take float32 rows on the host")
    _lib().lcu_ref_paged_attention(_p(q), q.stride(0), _p(_f32(cache, "cache")), _p(block_table),
                                   block_table.shape[1], _p(q_start), _p(ctx_len), ctx_len.numel(), heads, kv_heads, head_dim,
                                   page_size, ctypes.c_float(scale), int(window), _p(out))
    return out


def sample(logits: torch.Tensor, temperature: float, top_p: float, top_k: int, u: float) -> int:
    return int(_lib().lcu_ref_sample(_p(_f32(logits, "logits")), logits.numel(), ctypes.c_float(temperature),
                                     ctypes.c_float(top_p), ctypes.c_longlong(min(int(top_k), 2 ** 62)), ctypes.c_float(u)))
