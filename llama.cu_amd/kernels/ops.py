"""The hand-written gfx950 kernels as Python functions on torch tensors.

Every function checks on the host that the operands' shapes, types, layout and
device are what its kernel and its grid assume, and raises before anything is
launched if they are not; then it launches on torch's current stream.  There is no
CPU path: a tensor that is not on the GPU is an error.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import build
from .tuning import TUNING, Tuning, for_device  # noqa: F401  (ops.TUNING may be replaced to try other numbers)

F32, BF16 = 0, 1
_TYPE = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    pass


def tune_for(device) -> None:
    """Put the facts of the card at ``device`` (its number of compute units) into ``TUNING``."""
    global TUNING
    TUNING = for_device(TUNING, device)


_said: set = set()


def say_once(line: str) -> None:
    """A line for the log (standard error), once per process however often the same thing happens."""
    if line not in _said:
        _said.add(line)
        import sys
        print(f"[llama.cu_amd] {line}", file=sys.stderr, flush=True)


def _type(t: torch.Tensor, what: str) -> int:
    code = _TYPE.get(t.dtype)
    if code is None:
        raise KernelError(f"{what}: type {t.dtype} is not supported (float32 or bfloat16)")
    return code


def _gpu(*tensors: Optional[torch.Tensor]) -> None:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelError("kernel operands must be on the GPU (there is no CPU path)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise KernelError("kernel operands are on different devices")


def _rows(t: torch.Tensor, what: str) -> None:
    if t.dim() != 2 or t.stride(1) != 1:
        raise KernelError(f"{what}: need a 2-d tensor with contiguous rows, got shape {tuple(t.shape)} "
                          f"strides {tuple(t.stride())}")


def _contig(t: torch.Tensor, what: str) -> None:
    if not t.is_contiguous():
        raise KernelError(f"{what}: must be contiguous")


def _i32(t: torch.Tensor, what: str, n: Optional[int] = None) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{what}: must be a contiguous int32 tensor")
    if n is not None and t.numel() != n:
        raise KernelError(f"{what}: expected {n} entries, got {t.numel()}")


_scoped_stream: Optional[ctypes.c_void_p] = None


class stream_scope:
    """Within the scope the kernels are launched on the stream that is torch's current one at
    its entry.  Asking torch for its current stream at every launch costs more host time than
    the launch itself; a model's forward pass asks once."""

    def __enter__(self):
        global _scoped_stream
        self._before = _scoped_stream
        _scoped_stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        return self

    def __exit__(self, *exc):
        global _scoped_stream
        _scoped_stream = self._before
        return False


def _stream() -> ctypes.c_void_p:
    if _scoped_stream is not None:
        return _scoped_stream
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def to_device(values, dtype: torch.dtype, device) -> torch.Tensor:
    """Host values to the device without waiting for the GPU: through pinned memory, as a copy on the
    current stream.  (A copy from pageable memory makes the host wait until the stream has reached it:
    an engine that runs ahead of the GPU would stand still for a whole step.)"""
    return torch.tensor(values, dtype=dtype, pin_memory=True).to(device, non_blocking=True)


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _check(rc: int, name: str) -> None:
    if rc == 0:
        return
    if rc == -1:
        raise KernelError(f"{name}: the kernel refused its arguments (unsupported size or shape)")
    if rc == -2:
        raise KernelError(f"{name}: unsupported configuration")
    if rc == -3:
        raise KernelError(f"{name}: the call needs more scratch memory than the library's fixed buffer holds")
    if rc == -4:
        raise KernelError(f"{name}: the HIP runtime refused a call that is no launch (device or symbol look-up)")
    raise KernelError(f"{name}: launch failed with HIP error {rc}")


# ------------------------------------------------------------------ elementwise


def embedding_gather(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``out[i, :] = table[ids[i], :]`` (converted to ``out``'s type)."""
    _gpu(table, ids, out)
    _rows(table, "embedding table"); _contig(table, "embedding table"); _contig(out, "embedding out")
    n = ids.numel()
    _i32(ids, "token ids")
    if out.shape != (n, table.shape[1]):
        raise KernelError(f"embedding out: shape {tuple(out.shape)}, expected {(n, table.shape[1])}")
    lib = build.load("elementwise")
    _check(lib.lcu_embedding_gather(_ptr(out), _type(out, "embedding out"), _ptr(table), _type(table, "embedding table"),
                                    _ptr(ids), n, table.shape[1], table.shape[0], _stream()), "embedding_gather")
    return out


def gather_rows(x: torch.Tensor, rows: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[i, :] = x[rows[i], :]``."""
    _gpu(x, rows, out)
    _rows(x, "gather source"); _contig(x, "gather source")
    _i32(rows, "row indices")
    n = rows.numel()
    if out is None:
        out = torch.empty((n, x.shape[1]), dtype=x.dtype, device=x.device)
    if out.shape != (n, x.shape[1]) or out.dtype != x.dtype or not out.is_contiguous():
        raise KernelError("gather out: wrong shape, type or layout")
    lib = build.load("elementwise")
    _check(lib.lcu_gather_rows(_ptr(out), _ptr(x), _type(x, "gather source"), _ptr(rows), n, x.shape[1], x.shape[0],
                               _stream()), "gather_rows")
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
            delta: Optional[torch.Tensor] = None, write_back: bool = True) -> torch.Tensor:
    """``y = x' * rsqrt(mean(x'^2) + eps) * weight`` with ``x' = x + delta`` (``x`` if there is
    no ``delta``), all in 32-bit.  With ``write_back`` the sum ``x'`` replaces ``x`` (the
    residual stream takes in the branch's output).  ``delta`` may also be float32 planes
    ``[planes, n, d]`` (a product's partial sums, ``gemm_mid(..., slices=)``) beside a float32
    ``x``: they are added one after the other, in the order of the planes."""
    _gpu(x, weight, out, delta)
    _rows(x, "norm input"); _contig(x, "norm input"); _contig(out, "norm out"); _contig(weight, "norm weight")
    n, d = x.shape
    if out.shape != (n, d):
        raise KernelError(f"norm out: shape {tuple(out.shape)}, expected {(n, d)}")
    if weight.shape != (d,):
        raise KernelError(f"norm weight: shape {tuple(weight.shape)}, expected {(d,)}")
    xt, at = _type(x, "norm input"), _type(out, "norm out")
    if delta is not None and delta.dim() == 3:
        _contig(delta, "norm delta")
        if delta.shape[1:] != (n, d) or delta.dtype != torch.float32 or x.dtype != torch.float32 or d % 4:
            raise KernelError("norm delta: planes must be float32 [planes, n, d] beside a float32 input, d a multiple of 4")
        lib = build.load("elementwise")
        _check(lib.lcu_rmsnorm_planes(_ptr(x), _ptr(delta), delta.shape[0], _ptr(weight), _type(weight, "norm weight"),
                                      _ptr(out), at, n, d, ctypes.c_float(eps), int(bool(write_back)), _stream()),
               "rmsnorm (planes)")
        return out
    if delta is not None:
        _contig(delta, "norm delta")
        if delta.shape != (n, d) or delta.dtype != out.dtype:
            raise KernelError("norm delta: must have the output's shape and type")
    if (xt, at) not in ((F32, F32), (F32, BF16), (BF16, BF16)):
        raise KernelError(f"norm: input {x.dtype} with output {out.dtype} is not supported")
    lib = build.load("elementwise")
    _check(lib.lcu_rmsnorm(_ptr(x), xt, _ptr(delta), _ptr(weight), _type(weight, "norm weight"), _ptr(out), at,
                           n, d, ctypes.c_float(eps), int(bool(write_back)), _stream()), "rmsnorm")
    return out


def residual_add(x: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    """``x += delta`` in 32-bit (``x`` is float32)."""
    _gpu(x, delta)
    _contig(x, "residual"); _contig(delta, "delta")
    if x.dtype != torch.float32 or x.shape != delta.shape:
        raise KernelError("residual_add: x must be float32 and delta of the same shape")
    lib = build.load("elementwise")
    _check(lib.lcu_residual_add(_ptr(x), _ptr(delta), _type(delta, "delta"), ctypes.c_longlong(x.numel()), _stream()),
           "residual_add")
    return x


def swiglu(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out = gate * sigmoid(gate) * up`` for ``gate_up = [gate | up]`` of shape ``[n, 2*di]``."""
    _gpu(gate_up, out)
    _rows(gate_up, "gate_up"); _contig(gate_up, "gate_up")
    n, two_di = gate_up.shape
    if two_di % 2:
        raise KernelError("swiglu: the input's width must be even (gate and up side by side)")
    di = two_di // 2
    if out is None:
        out = torch.empty((n, di), dtype=gate_up.dtype, device=gate_up.device)
    if out.shape != (n, di) or out.dtype != gate_up.dtype or not out.is_contiguous():
        raise KernelError("swiglu out: wrong shape, type or layout")
    lib = build.load("elementwise")
    _check(lib.lcu_swiglu(_ptr(out), _ptr(gate_up), _type(gate_up, "gate_up"), n, di, _stream()), "swiglu")
    return out


def feed_tokens(tokens: torch.Tensor, sampled: torch.Tensor, src: torch.Tensor, dst: torch.Tensor) -> None:
    """``tokens[dst[i]] = sampled[src[i]]`` on the device."""
    _gpu(tokens, sampled, src, dst)
    _i32(tokens, "tokens"); _i32(sampled, "sampled"); _i32(src, "src"); _i32(dst, "dst", src.numel())
    lib = build.load("elementwise")
    _check(lib.lcu_feed_tokens(_ptr(tokens), tokens.numel(), _ptr(sampled), sampled.numel(), _ptr(src), _ptr(dst),
                               src.numel(), _stream()), "feed_tokens")


def random_fill(out: torch.Tensor, key: int, std: float, shift: float = 0.0, first: int = 0) -> torch.Tensor:
    """``out[i] = normal(key, first + i) * std + shift`` over the flattened ``out`` (float32 or bfloat16):
    the counter-based generator that the host library has too (weights.random)."""
    _gpu(out)
    _contig(out, "random_fill out")
    lib = build.load("random_fill")
    _check(lib.lcu_random_fill(_ptr(out), _type(out, "random_fill out"), ctypes.c_longlong(out.numel()),
                               ctypes.c_ulonglong(key & ((1 << 64) - 1)), ctypes.c_longlong(first), ctypes.c_float(std),
                               ctypes.c_float(shift), _stream()), "random_fill")
    return out


# ------------------------------------------------------------------ rotation and cache write


def rope_kv_store(qkv: torch.Tensor, positions: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int,
                  cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], rot_dim: int, pairing: int,
                  cache: Optional[torch.Tensor], slots: Optional[torch.Tensor], page_size: int) -> None:
    """Rotate the queries (in place) and the keys of ``qkv [n, (heads + 2 kv_heads) * head_dim]``
    and write keys and values into ``cache`` at ``slots``.  With ``cache=None`` the row holds
    queries only and nothing is stored."""
    _gpu(qkv, positions, cos, sin, cache, slots)
    _rows(qkv, "qkv")
    n = qkv.shape[0]
    store = cache is not None
    need = (n_heads + (2 * n_kv_heads if store else 0)) * head_dim
    if qkv.shape[1] != need:
        raise KernelError(f"qkv: width {qkv.shape[1]}, expected {need}")
    _i32(positions, "positions", n)
    if head_dim % 8:
        raise KernelError(f"head_dim {head_dim} must be a multiple of 8")
    max_pos = 0
    if cos is not None:
        if sin is None or cos.shape != sin.shape or cos.dtype != torch.float32 or sin.dtype != torch.float32 \
                or cos.dim() != 2 or cos.shape[1] * 2 != rot_dim or not cos.is_contiguous() or not sin.is_contiguous():
            raise KernelError("rotation tables must be two contiguous float32 tensors [max_pos, rot_dim/2]")
        max_pos = cos.shape[0]
    if store:
        _i32(slots, "cache slots", n)
        _contig(cache, "cache")
        if cache.dtype != qkv.dtype:
            raise KernelError("cache and qkv must have one type")
        if cache.dim() != 3 or cache.shape[1] != 2 or cache.shape[2] != n_kv_heads * head_dim * page_size:
            raise KernelError(f"cache: shape {tuple(cache.shape)}, expected [pages, 2, {n_kv_heads * head_dim * page_size}]")
    lib = build.load("rope_kv")
    _check(lib.lcu_rope_kv_store(_ptr(qkv), _type(qkv, "qkv"), n, qkv.stride(0), _ptr(positions), _ptr(slots),
                                 _ptr(cos), _ptr(sin), max_pos, _ptr(cache), n_heads, n_kv_heads, head_dim, rot_dim,
                                 pairing, page_size, int(store), _stream()), "rope_kv_store")


# ------------------------------------------------------------------ attention


def _attention_args(q, out, cache, block_table, q_start, ctx_len, req_of_token, n_heads, n_kv_heads, head_dim,
                    page_size):
    _gpu(q, out, cache, block_table, q_start, ctx_len, req_of_token)
    _rows(q, "attention q"); _rows(out, "attention out")
    n = q.shape[0]
    if q.shape[1] < n_heads * head_dim or out.shape != (n, n_heads * head_dim) or out.dtype != q.dtype:
        raise KernelError("attention: q or out has a wrong shape or type")
    if cache.dtype != q.dtype or not cache.is_contiguous() or cache.dim() != 3 or cache.shape[1] != 2 \
            or cache.shape[2] != n_kv_heads * head_dim * page_size:
        raise KernelError("attention: cache has a wrong shape, type or layout")
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or not block_table.is_contiguous():
        raise KernelError("attention: block_table must be a contiguous int32 [requests, pages]")
    n_req = block_table.shape[0]
    _i32(q_start, "q_start", n_req + 1); _i32(ctx_len, "ctx_len", n_req); _i32(req_of_token, "req_of_token", n)
    if n_heads % n_kv_heads:
        raise KernelError("attention: heads must be a multiple of kv heads")
    return n


def paged_attention_generic(q: torch.Tensor, out: torch.Tensor, cache: torch.Tensor, block_table: torch.Tensor,
                            q_start: torch.Tensor, ctx_len: torch.Tensor, req_of_token: torch.Tensor,
                            n_heads: int, n_kv_heads: int, head_dim: int, page_size: int, scale: float,
                            window: int = 0, head_slopes: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention of the step's queries over the paged cache (every shape).  ``head_slopes``
    (float32 [n_heads]) adds ``slope[h] * (key position - query position)`` to the scaled scores."""
    n = _attention_args(q, out, cache, block_table, q_start, ctx_len, req_of_token, n_heads, n_kv_heads, head_dim,
                        page_size)
    if head_dim % 8 or head_dim > 256:
        raise KernelError(f"attention: head_dim {head_dim} must be a multiple of 8, at most 256")
    if head_slopes is not None:
        _gpu(head_slopes)
        if head_slopes.dtype != torch.float32 or head_slopes.shape != (n_heads,) or not head_slopes.is_contiguous():
            raise KernelError(f"attention: head_slopes must be contiguous float32 [{n_heads}], got {head_slopes.dtype} {tuple(head_slopes.shape)}")
    lib = build.load("attention_generic")
    _check(lib.lcu_paged_attention_generic(_ptr(q), q.stride(0), _ptr(out), out.stride(0), _type(q, "q"), _ptr(cache),
                                           _ptr(block_table), block_table.shape[1], _ptr(q_start), _ptr(ctx_len),
                                           _ptr(req_of_token), n, n_heads, n_kv_heads, head_dim, page_size,
                                           ctypes.c_float(scale), int(window), _ptr(head_slopes), _stream()), "paged_attention_generic")
    return out


# ------------------------------------------------------------------ matrix products


def gemm_nt(a: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None,
            out_dtype: Optional[torch.dtype] = None, accumulate: bool = False) -> torch.Tensor:
    """``out (+)= a @ w.T`` with ``w [N, K]``, 32-bit accumulation, any mix of float32 and
    bfloat16 operands.  With float32 operands this is a true 32-bit product."""
    _gpu(a, w, out)
    _rows(a, "gemm a"); _rows(w, "gemm w")
    m, k = a.shape
    nn, k2 = w.shape
    if k != k2:
        raise KernelError(f"gemm: a is [{m}, {k}] but w is [{nn}, {k2}]")
    if out is None:
        if accumulate:
            raise KernelError("gemm: accumulate needs an output to add to")
        out = torch.empty((m, nn), dtype=out_dtype or a.dtype, device=a.device)
    _rows(out, "gemm out")
    if out.shape != (m, nn):
        raise KernelError(f"gemm out: shape {tuple(out.shape)}, expected {(m, nn)}")
    lib = build.load("gemm_generic")
    _check(lib.lcu_gemm_nt(_ptr(a), _type(a, "gemm a"), a.stride(0), _ptr(w), _type(w, "gemm w"), w.stride(0),
                           _ptr(out), _type(out, "gemm out"), out.stride(0), m, nn, k, int(bool(accumulate)),
                           _stream()), "gemm_nt")
    return out


def mfma_attention_refusal(dtype: torch.dtype, n_heads: int, n_kv_heads: int, head_dim: int, page_size: int) -> Optional[str]:
    """None if the matrix-core attention kernels take this shape, else why not (the generic kernel, one wave per
    token and head with plain multiply-adds, takes the rest): bfloat16, head_dim 32, 64, 96 or 128, pages of a
    multiple of 16 tokens, groups of at most 16 heads or of a multiple of 16."""
    g = n_heads // n_kv_heads
    if dtype != torch.bfloat16:
        return f"the type is {dtype}, not bfloat16"
    if head_dim not in (32, 64, 96, 128):
        return f"the head size is {head_dim}, not 32, 64, 96 or 128"
    if page_size % 16:
        return f"a page holds {page_size} tokens, no multiple of 16"
    if not (g <= 16 or g % 16 == 0):
        return f"{g} heads share a key/value head: more than 16 and no multiple of 16"
    return None


def mfma_attention_supported(q: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int, page_size: int) -> bool:
    """Whether the matrix-core attention kernels take these queries (``mfma_attention_refusal`` says why not)."""
    return mfma_attention_refusal(q.dtype, n_heads, n_kv_heads, head_dim, page_size) is None and q.stride(0) % 8 == 0


def attention_decode(q, out, cache, block_table, q_start, ctx_len, n_req, n_heads, n_kv_heads, head_dim, page_size,
                     scale, window, n_splits, req_list: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Matrix-core attention for requests that feed one token each: all ``n_req`` requests of
    the batch, or the ``n_req`` whose indices ``req_list`` holds."""
    if req_list is not None:
        _i32(req_list, "req_list", n_req)
    part_o = part_ml = None
    if n_splits > 1:
        part_o = torch.empty(n_req * n_heads * n_splits * head_dim, dtype=torch.float32, device=q.device)
        part_ml = torch.empty(n_req * n_heads * n_splits * 2, dtype=torch.float32, device=q.device)
    lib = build.load("attention_mfma")
    _check(lib.lcu_attention_decode_bf16(_ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(cache), _ptr(block_table),
                                         block_table.shape[1], _ptr(q_start), _ptr(ctx_len), _ptr(req_list), n_req, n_heads,
                                         n_kv_heads,
                                         head_dim, page_size, ctypes.c_float(scale), int(window), int(n_splits),
                                         _ptr(part_o), _ptr(part_ml), _stream()), "attention_decode")
    return out


def cut_into_tasks(q_lens, ctx_lens, tokens_per_task: int, skip_single: bool = False, window: int = 0):
    """Cut the batch into the prefill kernel's tasks: (request index, first token) pairs, in the order in which the
    workgroups should start.  Workgroups start in the order of the list, two to a compute unit, and the card fills
    the compute units' first places in turn before their second ones: so the longer half of the tasks (those that
    walk the most keys) comes first, longest first, and the shorter half follows shortest first; a compute unit then
    holds a long task beside a short one, and the long ones do not start last and leave the other compute units
    waiting for them.  (Against all tasks longest first: 60.4 -> 57.8 us for 2,048 tokens over 2k keys, 251.6 ->
    242.7 us over 8k; a long and a short one in turns, or as one workgroup's two tasks, was slower.)  ``skip_single``:
    requests that feed one token get no task (they go to the decode kernel).  ``window``: a task of a layer with a
    window walks no more keys than its tokens and the window."""
    tasks = []
    start = 0
    for r, n in enumerate(q_lens):
        for t in range(0, n if not (skip_single and n == 1) else 0, tokens_per_task):
            keys = ctx_lens[r] - n + min(t + tokens_per_task, n)        # keys the task's last token sees
            if window > 0:
                keys = min(keys, window + tokens_per_task)
            tasks.append((-keys, r, start + t))
        start += n
    tasks.sort()
    half = len(tasks) // 2
    tasks = tasks[:half] + tasks[half:][::-1]
    return [(t[1], t[2]) for t in tasks]


def prefill_tasks(q_lens, ctx_lens, tokens_per_task: int, device, skip_single: bool = False, per_wg: int = 1,
                  window: int = 0):
    """``cut_into_tasks`` as two arrays on the device, with their length; ``per_wg`` tasks go to one workgroup, one
    after the other."""
    tasks = cut_into_tasks(q_lens, ctx_lens, tokens_per_task, skip_single, window)
    if not tasks:
        return None, None, 0, 1
    both = to_device([[t[0] for t in tasks], [t[1] for t in tasks]], torch.int32, device)
    return both[0], both[1], len(tasks), per_wg


def attention_prefill(q, out, cache, block_table, q_start, ctx_len, task_req, task_tok0, n_tasks, tasks_per_wg, n_heads,
                      n_kv_heads, head_dim, page_size, scale, window, n_tasks_dev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Matrix-core attention for any mix of portions and single tokens.  ``n_tasks_dev`` (int32 on the device, one
    entry): the lists hold that many tasks, at most ``n_tasks``, for which the grid is made."""
    if task_req.numel() < n_tasks or task_tok0.numel() < n_tasks:
        raise KernelError(f"attention_prefill: the task lists hold fewer than {n_tasks} entries")
    _i32(task_req, "task_req"); _i32(task_tok0, "task_tok0")
    if n_tasks_dev is not None:
        _gpu(n_tasks_dev)
        _i32(n_tasks_dev, "n_tasks_dev")
    lib = build.load("attention_mfma")
    _check(lib.lcu_attention_prefill_bf16(_ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(cache),
                                          ctypes.c_longlong(cache.shape[0]), _ptr(block_table),
                                          block_table.shape[1], _ptr(q_start), _ptr(ctx_len), _ptr(task_req),
                                          _ptr(task_tok0), n_tasks, _ptr(n_tasks_dev), tasks_per_wg, n_heads, n_kv_heads, head_dim,
                                          page_size, ctypes.c_float(scale), int(window), _stream()), "attention_prefill")
    return out


class AttentionPlan:
    """How the matrix-core kernels share out a step that is not all single tokens: the requests that feed one token go
    to the decode kernel (``singles``: their indices, most keys first), every other request's tokens are cut into the
    prefill kernel's tasks (``task_req``, ``task_tok0``; ``n_tasks`` on the device says how many).  The launches' sizes
    (``max_tasks``, ``n_single``, ``single_splits``) follow from the step's sizes and the longest context rounded up to
    a power of two; what the lists hold is data."""
    __slots__ = ("task_req", "task_tok0", "n_tasks_dev", "max_tasks", "per_wg", "singles", "n_single", "single_splits")

    @property
    def signature(self):
        """What fixes the launches that ``paged_attention`` makes with this plan: two steps with equal signatures are
        served by the same recorded launches."""
        return (self.max_tasks, self.per_wg, self.n_single, self.single_splits)


def plan_attention(step, n_heads: int, n_kv_heads: int, window: int = 0) -> Optional[AttentionPlan]:
    """The AttentionPlan of ``step`` for layers with these heads and this window (one per step and kind of layer,
    kept in ``step.scratch``); None for a step of single tokens only, which needs none.  Called before the step's
    arrays go to the device (``Part.prepare``) it lays its lists into the step's own memory (``step.extra``): their
    addresses are then the same in every step, and launches recorded into a graph read the new step's lists.
    Called later (a step made by hand) it brings its lists to the device itself."""
    if step.decode_only:
        return None
    lib = build.load("attention_mfma")
    tpt = lib.lcu_attention_prefill_tokens_per_task(n_heads, n_kv_heads)
    if tpt <= 0:
        return None
    key = ("attention_plan", tpt, int(window))
    plan = step.scratch.get(key)
    if plan is not None:
        return plan
    singles = sorted((r for r, n in enumerate(step.q_lens) if n == 1), key=lambda r: -step.ctx_lens[r])    # most keys first
    tasks = cut_into_tasks(step.q_lens, step.ctx_lens, tpt, skip_single=bool(singles), window=window)
    plan = AttentionPlan()
    plan.per_wg = 1
    plan.n_single = len(singles)
    # the most tasks that a step of these sizes can have: a request of q tokens has at most q / tpt + 1
    plan.max_tasks = (step.n - len(singles)) // tpt + (step.n_req - len(singles))
    plan.single_splits = decode_splits(len(singles), n_heads, n_kv_heads, max([step.ctx_lens[r] for r in singles], default=0)) if singles else 1
    builder = getattr(step, "builder", None)
    if builder is not None:
        cap_tasks = builder.max_tokens // tpt + builder.max_reqs
        host, dev = step.extra(f"attention/{tpt}/{int(window)}", 4 + 2 * cap_tasks + builder.max_reqs)
        host[0] = len(tasks)
        if tasks:
            host[4:4 + len(tasks)] = torch.tensor([t[0] for t in tasks], dtype=torch.int32)
            host[4 + cap_tasks:4 + cap_tasks + len(tasks)] = torch.tensor([t[1] for t in tasks], dtype=torch.int32)
        if singles:
            host[4 + 2 * cap_tasks:4 + 2 * cap_tasks + len(singles)] = torch.tensor(singles, dtype=torch.int32)
        plan.n_tasks_dev = dev[0:1]
        plan.task_req = dev[4:4 + cap_tasks]
        plan.task_tok0 = dev[4 + cap_tasks:4 + 2 * cap_tasks]
        plan.singles = dev[4 + 2 * cap_tasks:4 + 2 * cap_tasks + len(singles)] if singles else None
    else:
        room = max(plan.max_tasks, 1)
        flat = to_device([len(tasks)] + [t[0] for t in tasks] + [0] * (room - len(tasks)) + [t[1] for t in tasks]
                         + [0] * (room - len(tasks)) + singles, torch.int32, step.tokens.device)
        plan.n_tasks_dev = flat[0:1]
        plan.task_req = flat[1:1 + room]
        plan.task_tok0 = flat[1 + room:1 + 2 * room]
        plan.singles = flat[1 + 2 * room:] if singles else None
    step.scratch[key] = plan
    return plan


def decode_splits(n_req: int, n_heads: int, n_kv_heads: int, max_ctx_len: int) -> int:
    """Into how many parts the decode kernel cuts each request's keys (the numbers are ``TUNING``'s).
    Few requests: about one workgroup for each compute unit, no part shorter than 512 keys, at most
    32 parts (measured from 2k to 128k keys: more parts cost more in the merge than they gain; a
    single request with 128k keys wants 32).  Between half the chip's worth of workgroups and all of
    it (17 to 31 requests of 8 key/value heads), where one part leaves compute units idle and two
    parts are a wave and a bit: one part up to 1k keys, beyond that up to 4 parts of at least 1024
    keys, the fewest with which the workgroups fill whole waves of 256 about as well as any (20
    requests are 160 workgroups: over 8k keys 161 us in one part, 118 in three, the whole step 8.7
    against 7.9 ms; over 2k keys the step of 17 requests 4.64 against 4.39 ms, of 20 requests 4.72
    against 4.55).  From 256 workgroups on
    one part: the chip is full, and more parts gained nothing (48 requests over 8k keys: 13.1 ms a
    step in one part, 13.2 in two).  The length counts rounded up to a power of two, so that a
    growing context changes the choice, and with it the rounding of the result and the captured
    graph that fits, only rarely."""
    t = TUNING
    base = max(1, n_req * n_kv_heads * ((n_heads // n_kv_heads + 15) // 16))
    rounded = 1 << max(int(max_ctx_len) - 1, 0).bit_length()     # up to a power of two: the choice changes rarely
    if base <= t.decode_few_workgroups:
        return max(1, min(t.decode_max_parts, t.compute_units // base, rounded // t.decode_min_part_keys))
    most = min(t.decode_long_max_parts, rounded // t.decode_long_part_keys) \
        if (rounded >= t.decode_long_context and base < t.compute_units) else 1
    fill = [(base * s / t.compute_units) / -(-base * s // t.compute_units) for s in range(1, most + 1)]
    return 1 + next(i for i, f in enumerate(fill) if f >= max(fill) - t.decode_fill_slack)


def paged_attention(q: torch.Tensor, out: torch.Tensor, cache: torch.Tensor, step, group: int, n_heads: int,
                    n_kv_heads: int, head_dim: int, page_size: int, scale: float, window: int = 0,
                    force_generic: bool = False, head_slopes: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention for the batch ``step`` (an engine.batch.StepContext) over cache group
    ``group``: picks the kernel for the batch's shape and type.  A bias inside the scores
    (``head_slopes``) is the generic kernel's: the matrix-core kernels take none."""
    bt = step.block_table(group)
    if force_generic or head_slopes is not None or not mfma_attention_supported(q, n_heads, n_kv_heads, head_dim, page_size):
        return paged_attention_generic(q, out, cache, bt, step.q_start, step.ctx_len, step.req_of_token, n_heads,
                                       n_kv_heads, head_dim, page_size, scale, window, head_slopes)
    n = _attention_args(q, out, cache, bt, step.q_start, step.ctx_len, step.req_of_token, n_heads, n_kv_heads, head_dim,
                        page_size)
    if step.decode_only:
        splits = step.attn_splits or decode_splits(step.n_req, n_heads, n_kv_heads, step.max_ctx_len)
        # the workgroups start in the order of the requests' list: the requests with the most keys first, where the
        # batch says which they are (64 requests of 150 to 2,200 keys: the step 11.2 -> 11.0 ms)
        return attention_decode(q, out, cache, bt, step.q_start, step.ctx_len, step.n_req, n_heads, n_kv_heads, head_dim,
                                page_size, scale, window, splits, req_list=step.decode_order)
    # a mixed batch: the requests that decode one token go to the decode kernel, the portions
    # to the prefill kernel (each would be slow at the other's work)
    plan = plan_attention(step, n_heads, n_kv_heads, window)
    if plan.n_single:
        attention_decode(q, out, cache, bt, step.q_start, step.ctx_len, plan.n_single, n_heads, n_kv_heads, head_dim, page_size,
                         scale, window, plan.single_splits, req_list=plan.singles)
    if plan.max_tasks:
        attention_prefill(q, out, cache, bt, step.q_start, step.ctx_len, plan.task_req, plan.task_tok0, plan.max_tasks,
                          plan.per_wg, n_heads, n_kv_heads, head_dim, page_size, scale, window, n_tasks_dev=plan.n_tasks_dev)
    return out


SKINNY_MAX_ROWS = 32      # what the kernel takes


def skinny_max_rows(packed: bool) -> int:
    """The most rows for which the weight-streaming kernel is ever chosen over the library."""
    return TUNING.skinny_rows_short_k if packed else TUNING.skinny_rows


_EPILOGUES = {"bf16": 0, "f32": 1, "add_f32": 2, "swiglu": 3}


def skinny_supported(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype) -> bool:
    """Whether the weight-streaming kernel for few rows takes this product: bfloat16
    operands, at most 32 rows, K a multiple of 8 (16-byte loads)."""
    return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2 and w.dim() == 2
            and 0 < x.shape[0] <= SKINNY_MAX_ROWS and x.shape[1] % 8 == 0 and x.stride(1) == 1 and w.stride(1) == 1
            and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and out_dtype in (torch.bfloat16, torch.float32)
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def packable(w: torch.Tensor) -> bool:
    """Whether ``pack_weight`` takes ``w``: bfloat16 ``[n, k]`` of whole blocks of 16 rows x 128 k."""
    return w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[0] % 16 == 0 and w.shape[1] % 128 == 0


def pack_weight(w: torch.Tensor) -> torch.Tensor:
    """``w [n, k]`` in the order in which the weight-streaming kernel loads it: the block of
    16 rows and 128 k of a tile and a macro-step in 4 KB of its own, inside it
    ``[load j][lane = 16 * group + row][8 k]`` (k = 32 * group + 8 * j + 0..7), the blocks of a
    tile one after the other.  The result has the shape of ``w`` and is given to
    ``gemm_skinny(..., packed=True)``."""
    if not packable(w):
        raise KernelError(f"pack_weight: need a bfloat16 [n, k] weight with n % 16 == 0 and k % 128 == 0, got {tuple(w.shape)} {w.dtype}")
    n, k = w.shape
    return w.view(n // 16, 16, k // 128, 4, 4, 8).permute(0, 2, 4, 3, 1, 5).contiguous().view(n, k)


def skinny_weight_ok(w: torch.Tensor) -> bool:
    """Whether the weight-streaming kernel takes ``w`` as its weight (for any rows it takes)."""
    return (w.dtype == torch.bfloat16 and w.dim() == 2 and w.is_cuda and w.shape[1] % 8 == 0 and w.stride(1) == 1
            and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0)


def skinny_preferred(m: int, n: int, k: int, out_dtype: torch.dtype, packed: bool = False) -> bool:
    """Whether the weight-streaming kernel is the faster choice for a plain bfloat16 product
    of ``m`` rows with an ``[n, k]`` weight (``TUNING``'s numbers): always for very few rows and for
    float32 output; with a packed weight up to 24 rows, and up to 32 where K is at most 8192 (there
    it is within a tenth of the library on the large weights, and its epilogues save the kernels
    around the product); without one, beyond 4 and up to 16 rows, only for small weights (the
    library's split over K wins on the large ones)."""
    t = TUNING
    if m > skinny_max_rows(packed):
        return False
    if packed and m > t.skinny_rows_packed:
        return k <= t.skinny_short_k       # up to 32 rows, but not the products with a long K (the down projection)
    return m <= (t.skinny_rows_packed if packed else t.skinny_rows_any_weight) or out_dtype == torch.float32 \
        or n * k <= t.skinny_small_weight


def _skinny_tiles(n_features: int, m: int, packed: bool = False) -> int:
    """Output tiles of 16 features per workgroup.  Plain weights: as many as still leave about four
    workgroups for each compute unit.  Packed weights: two from 6144 features on, four for the
    widest with more than 8 rows."""
    t = TUNING
    if packed:
        if n_features >= t.skinny_four_tiles_from and m > 8:
            return 4
        return 2 if n_features >= t.skinny_two_tiles_from else 1
    for tiles in (4, 2):
        if n_features // (16 * tiles) >= t.skinny_workgroups_per_cu * t.compute_units and (tiles < 4 or m <= 32):
            return tiles
    return 1


def gemm_skinny(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None,
                out_dtype: Optional[torch.dtype] = None, accumulate: bool = False, swiglu: bool = False,
                tiles: Optional[int] = None, waves: Optional[int] = None,
                row_sumsq: Optional[torch.Tensor] = None, norm_width: int = 0, eps: float = 0.0,
                packed: bool = False) -> torch.Tensor:
    """``out (+)= x @ w.T`` for at most 32 rows of bfloat16 ``x`` by streaming ``w`` once.
    ``swiglu``: ``w`` holds gate rows, then up rows; ``out = silu(x @ gate.T) * (x @ up.T)``.
    ``row_sumsq [m, parts]``: the rows of ``x`` wait for their normalisation (see
    ``gemm_skinny_add_norm``); row ``i`` of the product is multiplied by
    ``rsqrt(sum(row_sumsq[i]) / norm_width + eps)`` before the epilogue.
    ``packed``: ``w`` is the result of ``pack_weight``."""
    _gpu(x, w, out, row_sumsq)
    if packed and not (packable(w) and w.is_contiguous()):
        raise KernelError("gemm_skinny: a packed weight is a contiguous result of pack_weight")
    _rows(x, "skinny x"); _rows(w, "skinny w")
    m, k = x.shape
    n = w.shape[0]
    out_dtype = out.dtype if out is not None else (out_dtype or torch.bfloat16)
    if w.shape[1] != k or not skinny_supported(x, w, out_dtype):
        raise KernelError(f"gemm_skinny: x {tuple(x.shape)} {x.dtype} with w {tuple(w.shape)} {w.dtype} is not supported")
    if swiglu:
        if n % 2 or out_dtype != torch.bfloat16 or accumulate:
            raise KernelError("gemm_skinny: the SwiGLU epilogue needs an even number of rows of w and a bfloat16 output")
        epi, width = "swiglu", n // 2
    elif accumulate:
        if out is None or out.dtype != torch.float32:
            raise KernelError("gemm_skinny: accumulate needs a float32 output to add to")
        epi, width = "add_f32", n
    else:
        epi, width = ("f32" if out_dtype == torch.float32 else "bf16"), n
    if out is None:
        out = torch.empty((m, width), dtype=out_dtype, device=x.device)
    _rows(out, "skinny out")
    if out.shape != (m, width):
        raise KernelError(f"gemm_skinny out: shape {tuple(out.shape)}, expected {(m, width)}")
    tiles = tiles or ((4 if (m > 8 or packed) else 2) if swiglu else _skinny_tiles(width, m, packed))
    waves = waves or (8 if width <= TUNING.skinny_eight_waves_to else 4)
    lib = build.load("gemm_skinny")
    if row_sumsq is not None:
        if row_sumsq.dtype != torch.float32 or row_sumsq.dim() != 2 or row_sumsq.shape[0] != m or not row_sumsq.is_contiguous() \
                or norm_width <= 0:
            raise KernelError("gemm_skinny: row_sumsq must be a contiguous float32 [rows, parts] tensor, with the norm's width")
        _check(lib.lcu_gemm_skinny_bf16_scaled(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(out), out.stride(0), m, n, k,
                                               _EPILOGUES[epi], tiles, waves, int(packed), _ptr(row_sumsq), row_sumsq.shape[1],
                                               int(norm_width), ctypes.c_float(eps), _stream()), "gemm_skinny (scaled rows)")
        return out
    _check(lib.lcu_gemm_skinny_bf16(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(out), out.stride(0), m, n, k,
                                    _EPILOGUES[epi], tiles, waves, int(packed), _stream()),
           "gemm_skinny")
    return out


MID_MAX_ROWS = 256
MID_MAX_SCALED_ROWS = 64


def mid_supported(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether ``gemm_mid`` takes these operands: up to 256 bfloat16 rows with K a multiple of 128
    and a bfloat16 weight of a multiple of 16 rows."""
    return (x.is_cuda and w.is_cuda and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2
            and w.dim() == 2 and 0 < x.shape[0] <= MID_MAX_ROWS and x.shape[1] == w.shape[1] and w.shape[1] % 128 == 0
            and w.shape[0] % 16 == 0 and x.stride(1) == 1 and w.stride(1) == 1 and x.stride(0) % 8 == 0
            and w.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def mid_planes(k: int, slices: int) -> int:
    """The number of planes ``gemm_mid(..., slices=)`` writes for a weight with ``k`` columns."""
    steps = k // 128
    per = -(-steps // slices)
    return -(-steps // per)


def gemm_mid(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None, swiglu: bool = False,
             slices: Optional[int] = None, packed: bool = False, row_sumsq: Optional[torch.Tensor] = None,
             norm_width: int = 0, eps: float = 0.0) -> torch.Tensor:
    """``x @ w.T`` for up to 256 rows of bfloat16 ``x`` (chosen from 12 to 33 rows on, by the product), streaming ``w`` once while
    the waves of a workgroup share ``x`` through LDS.  ``slices=None``: ``out [m, n]`` bfloat16
    (``swiglu``: ``w`` holds gate rows, then up rows, ``out [m, n/2] = silu(gate) * up``).
    ``slices=s``: K is cut into (at most) ``s`` slices and ``out [planes, m, n]`` float32 holds
    each slice's sum; whoever reads it adds the planes (``rmsnorm(..., delta=planes)`` does).
    ``packed``: ``w`` is the result of ``pack_weight``.  ``row_sumsq [m, parts]``: the rows of ``x``
    wait for their normalisation, as in ``gemm_skinny``."""
    _gpu(x, w, out, row_sumsq)
    _rows(x, "mid x"); _rows(w, "mid w")
    if packed and not (packable(w) and w.is_contiguous()):
        raise KernelError("gemm_mid: a packed weight is a contiguous result of pack_weight")
    if not mid_supported(x, w):
        raise KernelError(f"gemm_mid: x {tuple(x.shape)} {x.dtype} with w {tuple(w.shape)} {w.dtype} is not supported "
                          f"(at most {MID_MAX_ROWS} bfloat16 rows, K a multiple of 128, a multiple of 16 features)")
    m, k = x.shape
    n = w.shape[0]
    if swiglu:
        if n % 32 or slices is not None:
            raise KernelError("gemm_mid: the SwiGLU epilogue needs a multiple of 32 rows of w and no slices")
        epi, shape, dtype = 2, (m, n // 2), torch.bfloat16
    elif slices is None:
        epi, shape, dtype = 0, (m, n), torch.bfloat16
    else:
        if not 1 <= slices <= 64:
            raise KernelError("gemm_mid: 1 to 64 slices")
        epi, shape, dtype = 1, (mid_planes(k, slices), m, n), torch.float32
    if out is None:
        out = torch.empty(shape, dtype=dtype, device=x.device)
    if out.shape != shape or out.dtype != dtype or out.stride(-1) != 1 or out.data_ptr() % 16 or out.stride(-2) % 4 \
            or (out.dim() == 3 and out.stride(0) != m * out.stride(1)):
        raise KernelError(f"gemm_mid out: need {dtype} {shape} with rows a multiple of 4 elements apart and planes one after the other")
    lib = build.load("gemm_mid")
    if row_sumsq is not None:
        if row_sumsq.dtype != torch.float32 or row_sumsq.dim() != 2 or row_sumsq.shape[0] != m or not row_sumsq.is_contiguous() \
                or norm_width <= 0 or row_sumsq.data_ptr() % 16 or m > MID_MAX_SCALED_ROWS:
            raise KernelError(f"gemm_mid: row_sumsq must be a contiguous float32 [rows, parts] tensor, with the norm's width, "
                              f"for at most {MID_MAX_SCALED_ROWS} rows")
        _check(lib.lcu_gemm_mid_bf16_scaled(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(out), out.stride(-2), m, n, k, epi,
                                            slices or 1, int(packed), _ptr(row_sumsq), row_sumsq.shape[1], int(norm_width),
                                            ctypes.c_float(eps), _stream()), "gemm_mid (scaled rows)")
        return out
    _check(lib.lcu_gemm_mid_bf16(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(out), out.stride(-2), m, n, k, epi,
                                 slices or 1, int(packed), _stream()), "gemm_mid")
    return out


ADD_NORM_MAX_ROWS = 32


def gemm_skinny_add_norm(x: torch.Tensor, w: torch.Tensor, residual: torch.Tensor, norm_weight: torch.Tensor,
                         tiles: Optional[int] = None, waves: Optional[int] = None, packed: bool = False):
    """The product that ends a branch, the residual sum and the next norm's weight in one
    kernel: ``residual += x @ w.T`` (float32, in place); returns ``(h, sumsq)`` with
    ``h = bfloat16(residual * norm_weight)``, not yet normalised, and ``sumsq [rows, parts]``,
    the workgroups' shares of each row's sum of squares, for ``gemm_skinny(..., row_sumsq=)``.
    At most 32 rows."""
    _gpu(x, w, residual, norm_weight)
    _rows(x, "skinny x"); _rows(w, "skinny w"); _rows(residual, "residual")
    if packed and not (packable(w) and w.is_contiguous()):
        raise KernelError("gemm_skinny_add_norm: a packed weight is a contiguous result of pack_weight")
    m, k = x.shape
    n = w.shape[0]
    if w.shape[1] != k or m > ADD_NORM_MAX_ROWS or not skinny_supported(x, w, torch.float32):
        raise KernelError(f"gemm_skinny_add_norm: x {tuple(x.shape)} {x.dtype} with w {tuple(w.shape)} {w.dtype} is not supported")
    if residual.dtype != torch.float32 or residual.shape != (m, n):
        raise KernelError(f"gemm_skinny_add_norm: the residual must be float32 {(m, n)}")
    if norm_weight.shape != (n,) or not norm_weight.is_contiguous():
        raise KernelError(f"gemm_skinny_add_norm: the norm's weight must be a contiguous [{n}] tensor")
    tiles = tiles or (1 if n <= TUNING.skinny_eight_waves_to else 2)
    waves = waves or (8 if n <= TUNING.skinny_eight_waves_to else 4)
    parts = (n + 16 * tiles - 1) // (16 * tiles)
    h = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    sumsq = torch.empty((m, parts), dtype=torch.float32, device=x.device)
    lib = build.load("gemm_skinny")
    _check(lib.lcu_gemm_skinny_bf16_add_norm(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(residual), residual.stride(0),
                                             m, n, k, _ptr(norm_weight), _type(norm_weight, "norm weight"), _ptr(h),
                                             h.stride(0), _ptr(sumsq), parts, tiles, waves, int(packed), _stream()),
           "gemm_skinny_add_norm")
    return h, sumsq


MID_ADD_NORM_MAX_ROWS = 64


def gemm_mid_add_norm(x: torch.Tensor, w: torch.Tensor, residual: torch.Tensor, norm_weight: torch.Tensor, packed: bool = False):
    """``gemm_skinny_add_norm`` for up to 64 rows, by the kernel that shares the rows through LDS: ``residual += x @ w.T``
    (float32, in place); returns ``(h, sumsq)`` with ``h = bfloat16(residual * norm_weight)``, not yet normalised, and
    ``sumsq [rows, out / 16]``, the workgroups' shares of each row's sum of squares.  A workgroup takes 16 output
    features over all of K and reads every row: for products with a short K (the output projection)."""
    _gpu(x, w, residual, norm_weight)
    _rows(x, "mid x"); _rows(w, "mid w"); _rows(residual, "residual")
    if packed and not (packable(w) and w.is_contiguous()):
        raise KernelError("gemm_mid_add_norm: a packed weight is a contiguous result of pack_weight")
    m, k = x.shape
    n = w.shape[0]
    if w.shape[1] != k or m > MID_ADD_NORM_MAX_ROWS or not mid_supported(x, w):
        raise KernelError(f"gemm_mid_add_norm: x {tuple(x.shape)} {x.dtype} with w {tuple(w.shape)} {w.dtype} is not supported "
                          f"(at most {MID_ADD_NORM_MAX_ROWS} bfloat16 rows, K a multiple of 128, a multiple of 16 features)")
    if residual.dtype != torch.float32 or residual.shape != (m, n) or residual.stride(0) % 4 or residual.data_ptr() % 16:
        raise KernelError(f"gemm_mid_add_norm: the residual must be float32 {(m, n)} with rows a multiple of 4 elements apart")
    if norm_weight.shape != (n,) or not norm_weight.is_contiguous():
        raise KernelError(f"gemm_mid_add_norm: the norm's weight must be a contiguous [{n}] tensor")
    h = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    sumsq = torch.empty((m, n // 16), dtype=torch.float32, device=x.device)
    lib = build.load("gemm_mid")
    _check(lib.lcu_gemm_mid_bf16_add_norm(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(residual), residual.stride(0), m, n, k,
                                          _ptr(norm_weight), _type(norm_weight, "norm weight"), _ptr(h), h.stride(0), _ptr(sumsq),
                                          int(packed), _stream()), "gemm_mid_add_norm")
    return h, sumsq


QKV_ROPE_MAX_ROWS = 32


def qkv_rope_supported(x: torch.Tensor, w: torch.Tensor, heads: int, kv_heads: int, head_dim: int) -> bool:
    """Whether ``gemm_skinny_qkv_rope`` takes these operands: at most 32 rows, bfloat16, whole
    heads whose halves are multiples of 16."""
    return (x.dim() == 2 and x.shape[0] <= QKV_ROPE_MAX_ROWS and head_dim % 32 == 0
            and w.shape[0] == (heads + 2 * kv_heads) * head_dim and skinny_supported(x, w, torch.bfloat16))


def gemm_skinny_qkv_rope(x: torch.Tensor, w: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor,
                         cos: torch.Tensor, sin: torch.Tensor, cache: torch.Tensor, heads: int, kv_heads: int,
                         head_dim: int, page_size: int, row_sumsq: Optional[torch.Tensor] = None, norm_width: int = 0,
                         eps: float = 0.0, packed: bool = False, waves: Optional[int] = None) -> torch.Tensor:
    """The q, k, v product of an attention layer with the rotation and the cache write in its
    epilogue: ``w`` holds the rows of q, k and v (whole heads, in this order); returns the rotated
    queries ``[rows, heads * head_dim]``; the rotated keys and the values of row ``i`` are written
    into ``cache`` at ``slots[i]`` (negative: not stored).  Pairs are ``(i, i + head_dim / 2)`` and
    the rotation covers the whole head.  ``row_sumsq``: as in ``gemm_skinny``."""
    _gpu(x, w, positions, slots, cos, sin, cache, row_sumsq)
    if packed and not (packable(w) and w.is_contiguous()):
        raise KernelError("gemm_skinny_qkv_rope: a packed weight is a contiguous result of pack_weight")
    _rows(x, "skinny x"); _rows(w, "skinny w")
    m, k = x.shape
    if w.shape[1] != k or not qkv_rope_supported(x, w, heads, kv_heads, head_dim):
        raise KernelError(f"gemm_skinny_qkv_rope: x {tuple(x.shape)} {x.dtype} with w {tuple(w.shape)} {w.dtype}, {heads} + 2 * "
                          f"{kv_heads} heads of {head_dim} is not supported")
    _i32(positions, "positions", m); _i32(slots, "cache slots", m)
    if cos.shape != sin.shape or cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.dim() != 2 \
            or cos.shape[1] * 2 != head_dim or not cos.is_contiguous() or not sin.is_contiguous():
        raise KernelError("rotation tables must be two contiguous float32 tensors [max_pos, head_dim/2]")
    _contig(cache, "cache")
    if cache.dtype != torch.bfloat16 or cache.dim() != 3 or cache.shape[1] != 2 \
            or cache.shape[2] != kv_heads * head_dim * page_size:
        raise KernelError(f"cache: {cache.dtype} {tuple(cache.shape)}, expected bfloat16 [pages, 2, {kv_heads * head_dim * page_size}]")
    n_in = 0
    if row_sumsq is not None:
        if row_sumsq.dtype != torch.float32 or row_sumsq.dim() != 2 or row_sumsq.shape[0] != m or not row_sumsq.is_contiguous() \
                or norm_width <= 0:
            raise KernelError("gemm_skinny_qkv_rope: row_sumsq must be a contiguous float32 [rows, parts] tensor, with the norm's width")
        n_in = row_sumsq.shape[1]
    q = torch.empty((m, heads * head_dim), dtype=torch.bfloat16, device=x.device)
    waves = waves or 8
    lib = build.load("gemm_skinny")
    _check(lib.lcu_gemm_skinny_bf16_qkv_rope(_ptr(x), x.stride(0), _ptr(w), w.stride(0), m, k, _ptr(q), q.stride(0),
                                             _ptr(positions), _ptr(slots), _ptr(cos), _ptr(sin), cos.shape[0], _ptr(cache),
                                             heads, kv_heads, head_dim, page_size, waves, int(packed), _ptr(row_sumsq), n_in,
                                             int(norm_width), ctypes.c_float(eps), _stream()), "gemm_skinny_qkv_rope")
    return q


def mid_qkv_rope_supported(x: torch.Tensor, w: torch.Tensor, heads: int, kv_heads: int, head_dim: int) -> bool:
    """Whether ``gemm_mid_qkv_rope`` takes these operands: what ``gemm_mid`` takes, and whole heads whose halves
    are multiples of 16."""
    return (head_dim % 32 == 0 and w.dim() == 2 and w.shape[0] == (heads + 2 * kv_heads) * head_dim and mid_supported(x, w))


def gemm_mid_qkv_rope(x: torch.Tensor, w: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor,
                      cos: torch.Tensor, sin: torch.Tensor, cache: torch.Tensor, heads: int, kv_heads: int,
                      head_dim: int, page_size: int, packed: bool = False) -> torch.Tensor:
    """``gemm_skinny_qkv_rope`` for 17 to 256 rows: the q, k, v product with the rotation and the cache write in its
    epilogue, by the kernel that shares the rows through LDS (its four consumer waves share each 128 k and add
    their sums at the end; nothing is cut over workgroups).  Returns the rotated queries ``[rows, heads * head_dim]``."""
    _gpu(x, w, positions, slots, cos, sin, cache)
    if packed and not (packable(w) and w.is_contiguous()):
        raise KernelError("gemm_mid_qkv_rope: a packed weight is a contiguous result of pack_weight")
    _rows(x, "mid x"); _rows(w, "mid w")
    m, k = x.shape
    if w.shape[1] != k or not mid_qkv_rope_supported(x, w, heads, kv_heads, head_dim):
        raise KernelError(f"gemm_mid_qkv_rope: x {tuple(x.shape)} {x.dtype} with w {tuple(w.shape)} {w.dtype}, {heads} + 2 * "
                          f"{kv_heads} heads of {head_dim} is not supported")
    _i32(positions, "positions", m); _i32(slots, "cache slots", m)
    if cos.shape != sin.shape or cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.dim() != 2 \
            or cos.shape[1] * 2 != head_dim or not cos.is_contiguous() or not sin.is_contiguous():
        raise KernelError("rotation tables must be two contiguous float32 tensors [max_pos, head_dim/2]")
    _contig(cache, "cache")
    if cache.dtype != torch.bfloat16 or cache.dim() != 3 or cache.shape[1] != 2 \
            or cache.shape[2] != kv_heads * head_dim * page_size or page_size % 8:
        raise KernelError(f"cache: {cache.dtype} {tuple(cache.shape)}, expected bfloat16 [pages, 2, {kv_heads * head_dim * page_size}]")
    q = torch.empty((m, heads * head_dim), dtype=torch.bfloat16, device=x.device)
    lib = build.load("gemm_mid")
    _check(lib.lcu_gemm_mid_bf16_qkv_rope(_ptr(x), x.stride(0), _ptr(w), w.stride(0), m, k, _ptr(q), q.stride(0),
                                          _ptr(positions), _ptr(slots), _ptr(cos), _ptr(sin), cos.shape[0], _ptr(cache),
                                          heads, kv_heads, head_dim, page_size, int(packed), _stream()), "gemm_mid_qkv_rope")
    return q


def skinny_f32_supported(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype) -> bool:
    """Whether the float32 weight-streaming kernel takes this product: all float32, K a
    multiple of 4 (16-byte loads)."""
    return (x.dtype == torch.float32 and w.dtype == torch.float32 and out_dtype == torch.float32 and x.dim() == 2
            and w.dim() == 2 and x.shape[0] > 0 and x.shape[1] % 4 == 0 and x.stride(1) == 1 and w.stride(1) == 1
            and x.stride(0) % 4 == 0 and w.stride(0) % 4 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def gemm_skinny_f32(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None,
                    accumulate: bool = False) -> torch.Tensor:
    """``out (+)= x @ w.T`` in true 32-bit on the matrix cores (v_mfma_f32_16x16x4_f32), any
    number of rows; a row's result does not depend on the other rows."""
    _gpu(x, w, out)
    _rows(x, "skinny x"); _rows(w, "skinny w")
    m, k = x.shape
    n = w.shape[0]
    if w.shape[1] != k or not skinny_f32_supported(x, w, torch.float32):
        raise KernelError(f"gemm_skinny_f32: x {tuple(x.shape)} {x.dtype} with w {tuple(w.shape)} {w.dtype} is not supported")
    if out is None:
        if accumulate:
            raise KernelError("gemm_skinny_f32: accumulate needs an output to add to")
        out = torch.empty((m, n), dtype=torch.float32, device=x.device)
    _rows(out, "skinny out")
    if out.shape != (m, n) or out.dtype != torch.float32:
        raise KernelError("gemm_skinny_f32 out: wrong shape or type")
    lib = build.load("gemm_skinny")
    _check(lib.lcu_gemm_skinny_f32(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(out), out.stride(0), m, n, k,
                                   int(bool(accumulate)), _stream()), "gemm_skinny_f32")
    return out
