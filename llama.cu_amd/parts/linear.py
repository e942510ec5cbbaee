"""``y = x @ W.T`` for a weight stored ``[out, in]`` (llama.cu/src/op/linear.rs:85-89).

Which routine multiplies is decided here and nowhere else:

* bfloat16 activations and weights: few rows (decoding) go to the hand-written
  weight-streaming kernel, many rows to the library's matrix product (hipBLASLt through
  torch, with bfloat16 or, for logits, float32 output), as the reference's engine calls
  its vendor library (llama.cu/src/op/linear.rs:91-118);
* all float32 (the true 32-bit path): the hand-written weight-streaming kernel on the
  32-bit matrix instruction, for any number of rows;
* everything else (mixed types: a weight that its file stores in 32-bit beside
  bfloat16 activations; widths the others refuse): the generic hand-written kernel with
  32-bit multiply-adds.
"""
from __future__ import annotations

import sys
from typing import Optional, Union

import torch

from ..kernels import ops
from .base import ScaledRows


class Weight:
    """A matrix ``[out, in]`` as its file holds it (``plain``: what the library's product and
    the generic kernels take) and, if the engine keeps one, a second copy in the order in
    which the weight-streaming kernel loads it (``packed``, see ``ops.pack_weight``): decoding
    then reads one contiguous run of memory per workgroup, which HBM serves 10 to 25 % faster
    (measured on the Llama-3-8B shapes).  The copy doubles the memory of the matrices;
    ``BuildContext.pack_weights`` switches it off."""

    def __init__(self, tensor: torch.Tensor, build=None, packed_from: Optional[torch.Tensor] = None, halves: bool = False):
        """``packed_from``: the matrix to pack if it is not ``tensor`` (a gate/up matrix whose plain copy
        has rows of zeros for the library's sake, see ``library_friendly_rows``, is packed without them).
        ``halves``: the matrix is two matrices one above the other (gate and up) whose rows a kernel pairs:
        it is packed only if each half is whole blocks of 16 rows."""
        self.plain = tensor.contiguous()
        want = build is None or getattr(build, "pack_weights", True)
        src = self.plain if packed_from is None else packed_from.contiguous()
        fits = ops.packable(src) and (not halves or src.shape[0] % 32 == 0)
        self.packed = ops.pack_weight(src) if (want and src.is_cuda and fits) else None

    @property
    def shape(self):
        return self.plain.shape

    @property
    def dtype(self):
        return self.plain.dtype


def _split(weight):
    if isinstance(weight, Weight):
        return weight.plain, weight.packed
    return weight, None


def linear(x: torch.Tensor, weight: Union[torch.Tensor, Weight], out_dtype: Optional[torch.dtype] = None,
           out: Optional[torch.Tensor] = None, accumulate: bool = False) -> torch.Tensor:
    """``out (+)= x @ weight.T``.  ``accumulate`` adds into a float32 ``out`` in 32-bit."""
    if not x.is_cuda:
        raise ops.KernelError("linear: operands must be on the GPU (there is no CPU path)")
    weight, packed = _split(weight)
    out_dtype = out.dtype if out is not None else (out_dtype or x.dtype)
    all_bf16 = x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
    if all_bf16 and ops.skinny_supported(x, weight, out_dtype) and (
            accumulate or ops.skinny_preferred(x.shape[0], weight.shape[0], weight.shape[1], out_dtype, packed is not None)):
        if packed is not None:
            return ops.gemm_skinny(x, packed, out=out, out_dtype=out_dtype, accumulate=accumulate, packed=True)
        return ops.gemm_skinny(x, weight, out=out, out_dtype=out_dtype, accumulate=accumulate)
    if all_bf16 and out_dtype == torch.bfloat16 and not accumulate:
        if out is None:
            return torch.matmul(x, weight.t())
        return torch.matmul(x, weight.t(), out=out)
    if all_bf16 and out_dtype == torch.float32 and not accumulate and out is None and x.shape[0] > ops.skinny_max_rows(packed is not None):
        if packed is not None and ops.TUNING.mid_f32_rows < x.shape[0] <= ops.TUNING.mid_f32_max_rows and ops.mid_supported(x, weight):
            return ops.gemm_mid(x, packed, slices=1, packed=True)[0]  # one plane of 32-bit sums: K is not cut
        return torch.mm(x, weight.t(), out_dtype=torch.float32)      # 32-bit accumulation, stored unrounded (logits)
    if ops.skinny_f32_supported(x, weight, out_dtype):
        return ops.gemm_skinny_f32(x, weight, out=out, accumulate=accumulate)
    return ops.gemm_nt(x, weight, out=out, out_dtype=out_dtype, accumulate=accumulate)


def linear_swiglu(h, weight: Union[torch.Tensor, Weight], row_sumsq=None, norm_width: int = 0, eps: float = 0.0):
    """``silu(h @ gate.T) * (h @ up.T)`` with the weight-streaming kernel (``weight`` holds the gate
    rows, then the up rows); ``row_sumsq``: the rows wait for their normalisation."""
    weight, packed = _split(weight)
    kw = dict(row_sumsq=row_sumsq, norm_width=norm_width, eps=eps) if row_sumsq is not None else {}
    if packed is not None:
        return ops.gemm_skinny(h, packed, swiglu=True, packed=True, **kw)
    return ops.gemm_skinny(h, weight, swiglu=True, **kw)


def linear_scaled(rows, weight: Union[torch.Tensor, Weight], out_dtype: Optional[torch.dtype] = None):
    """``rows.rows @ weight.T`` with the rows' normalisation applied in the epilogue (``rows``: ScaledRows)."""
    weight, packed = _split(weight)
    kw = dict(row_sumsq=rows.sumsq, norm_width=rows.width, eps=rows.eps, out_dtype=out_dtype)
    if packed is not None:
        return ops.gemm_skinny(rows.rows, packed, packed=True, **kw)
    return ops.gemm_skinny(rows.rows, weight, **kw)


_friendly_rows: dict = {}


def library_friendly_rows(di: int, d: int, device) -> int:
    """The number of rows to which each half of a bfloat16 gate/up matrix ``[2 * di, d]`` is filled up
    with rows of zeros for the library's product of many rows.  The library's choice of kernel
    depends on the number of output features in ways that no rule predicts: with 2,048 rows and
    K = 4096 it takes 417 us for 22,016 features (the Llama-2-7B shape) and 320 us for 24,576.
    So a large matrix is timed once, at 2,048 rows, as it is and with each half filled up to the
    next multiples of 1024, 2048 and 4096; rows are added only if that is at least 15 % faster
    (``TUNING.library_rows`` fixes the answer instead, for runs that must not depend on a timing).
    The rows of zeros give zeros (silu(0) * 0), which whoever multiplies next leaves out."""
    if 2 * di * d < (1 << 25):
        return di                                   # small matrices: nothing to gain, and timings of a few us say nothing
    fixed = ops.TUNING.library_rows                 # a run that must not depend on a timing says so there
    if fixed >= 0:
        return di if fixed == 0 else -(-di // fixed) * fixed
    key = (di, d, str(device))
    if key not in _friendly_rows:
        free, _ = torch.cuda.mem_get_info(device)
        if free < 4 * (2 * (di + 4096) * d * 2):
            _friendly_rows[key] = di                # no room to try (and none to spare for rows of zeros): decided once, so
            return di                               # that the loader's layout and the part's agree
        x = torch.randn(2048, d, device=device, dtype=torch.bfloat16)
        times = {}
        for rows in sorted({di} | {-(-di // m) * m for m in (1024, 2048, 4096)}):
            # numbers as a model's, zeros only where the rows of zeros would be: with a matrix of zeros the card's clock is
            # higher (its power limit is further away) and the comparison another
            w = torch.zeros(2 * rows, d, device=device, dtype=torch.bfloat16)
            for half in (0, 1):
                w[half * rows:half * rows + di].normal_(0.0, 0.02)
            for _ in range(2):
                torch.matmul(x, w.t())
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            for _ in range(4):
                torch.matmul(x, w.t())
            end.record()
            end.synchronize()
            times[rows] = start.elapsed_time(end)
            del w
        best = min(times, key=times.get)
        _friendly_rows[key] = best if times[best] <= 0.85 * times[di] else di
        # the choice enters the log: it rests on a timing, and a run should say what it chose
        took = ", ".join(f"{rows}: {t / 4 * 1e3:.0f} us" for rows, t in sorted(times.items()))
        print(f"[llama.cu_amd] gate/up product of 2,048 rows with halves of {di} x {d}: the library takes {took} per "
              f"half size; each half of the plain copy is {'filled up to ' + str(_friendly_rows[key]) + ' rows' if _friendly_rows[key] != di else 'left as it is'}",
              file=sys.stderr, flush=True)
    return _friendly_rows[key]


def _mid_slices(n_features: int, k: int) -> int:
    """Into how many slices of K the kernel that shares the rows through LDS (up to 256 rows) cuts a product, so that about one
    workgroup (64 features and a slice) stands on each compute unit; a slice keeps at least four
    macro-steps of 128."""
    t = ops.TUNING
    groups = -(-n_features // 64)
    return max(1, min(round(t.compute_units / groups), t.mid_max_slices, k // (128 * t.mid_min_slice_steps)))


def mid_takes(n_rows: int, weight: Union[torch.Tensor, Weight]) -> bool:
    """Whether the kernel that shares the rows through LDS (up to 256 rows) is the faster choice for this many bfloat16 rows and
    this weight (measured against the library on the Llama-3-8B shapes: the products with few
    output features, which are cut over K, 10 to 30 % faster with a packed weight at 64 rows and
    more beyond, the down projection with a plain one too).  A packed weight with a long K (the
    down projection) it takes from 12 rows on: 24 us and 5 for the norm kernel against 33 to 40 of
    the weight-streaming kernel at 16 and more rows (every workgroup of that kernel reads all rows,
    which at 16 rows and K = 14336 is as many bytes as its share of the weight)."""
    t = ops.TUNING
    w, packed = _split(weight)
    long_k = w.dim() == 2 and w.shape[1] > t.mid_long_k
    fewest = t.mid_long_k_rows if (packed is not None and long_k) else t.skinny_rows_short_k
    most = min(ops.MID_MAX_ROWS, t.mid_long_k_max_rows if long_k else t.mid_short_k_max_rows)
    if not (fewest < n_rows <= most and w.dtype == torch.bfloat16 and w.is_cuda and w.dim() == 2
            and w.shape[1] % 128 == 0 and w.shape[0] % 16 == 0):
        return False
    # products that are not cut over K stay with the library; a plain weight only with a long K (measured: the
    # output projections of the 8B and 70B shapes with plain weights are no faster than the library's)
    return _mid_slices(w.shape[0], w.shape[1]) >= 2 and (packed is not None or long_k)


def linear_planes(a: torch.Tensor, weight: Union[torch.Tensor, Weight]) -> torch.Tensor:
    """``a @ weight.T`` as float32 planes ``[planes, rows, out]`` of partial sums over slices of K
    (``mid_takes`` says when); the norm that follows adds them to the residual stream."""
    w, packed = _split(weight)
    slices = _mid_slices(w.shape[0], w.shape[1])
    if packed is not None:
        return ops.gemm_mid(a, packed, slices=slices, packed=True)
    return ops.gemm_mid(a, w, slices=slices)


def mid_swiglu_takes(n_rows: int, weight: Union[torch.Tensor, Weight]) -> bool:
    """Whether the gate/up product of this many rows goes to the kernel that shares the rows through LDS, with
    SwiGLU in its epilogue (with a packed weight it is faster than the library's product and the
    activation kernel after it, and from 15 rows on than the weight-streaming kernel: 46 against
    48 us at 16 rows, 52 to 55 from 17 on, on the Llama-3-8B shape)."""
    w, packed = _split(weight)
    return (ops.TUNING.mid_swiglu_rows < n_rows <= min(ops.MID_MAX_ROWS, ops.TUNING.mid_swiglu_max_rows) and packed is not None and w.shape[0] % 32 == 0
            and w.shape[1] % 128 == 0 and w.shape[0] >= ops.TUNING.mid_swiglu_features)


def linear_swiglu_mid(h, weight: Union[torch.Tensor, Weight]) -> torch.Tensor:
    """``h``: bfloat16 rows or ScaledRows (the factor then goes into the epilogue)."""
    if isinstance(h, ScaledRows):
        return ops.gemm_mid(h.rows, _split(weight)[1], swiglu=True, packed=True, row_sumsq=h.sumsq, norm_width=h.width, eps=h.eps)
    return ops.gemm_mid(h, _split(weight)[1], swiglu=True, packed=True)


def skinny_row_limit(weight: Union[torch.Tensor, Weight]) -> int:
    """Up to how many rows the weight-streaming kernel may be chosen for this weight."""
    return ops.skinny_max_rows(_split(weight)[1] is not None)


def skinny_takes(n_rows: int, weight: Union[torch.Tensor, Weight], preferred: bool = False) -> bool:
    """Whether the weight-streaming kernel takes ``n_rows`` bfloat16 rows with this weight (and,
    with ``preferred``, is the faster choice for a plain product)."""
    w, packed = _split(weight)
    if not ops.skinny_weight_ok(w):
        return False
    return not preferred or ops.skinny_preferred(n_rows, w.shape[0], w.shape[1], torch.bfloat16, packed is not None)


def mid_add_norm_takes(n_rows: int, weight: Union[torch.Tensor, Weight]) -> bool:
    """Whether the product that ends a branch goes, with the residual sum and the next norm's weight in its epilogue, to
    the kernel that shares the rows through LDS: a packed weight with a short K (the output projection), 17 to 32 rows,
    and no more workgroups (one for 16 output features, each reads every row) than compute units."""
    w, packed = _split(weight)
    t = ops.TUNING
    return (packed is not None and t.mid_add_norm_rows < n_rows <= min(ops.MID_ADD_NORM_MAX_ROWS, t.mid_add_norm_max_rows)
            and w.dim() == 2 and w.shape[1] % 128 == 0 and w.shape[1] <= t.mid_long_k and w.shape[0] % 16 == 0
            and w.shape[0] // 16 <= t.compute_units)


def linear_into_norm(a: torch.Tensor, weight: Union[torch.Tensor, Weight], residual: torch.Tensor, norm_weight: torch.Tensor):
    """``residual += a @ weight.T`` and the rows for the product after the next norm, in one
    kernel: returns ``(rows, sumsq)`` for a ``ScaledRows``, or None if the kernel for it does
    not take these operands (then nothing has been done)."""
    whole = weight
    weight, packed = _split(weight)
    if not (a.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and residual.dtype == torch.float32
            and norm_weight.dtype in (torch.bfloat16, torch.float32)):
        return None
    if mid_add_norm_takes(a.shape[0], whole) and ops.mid_supported(a, weight) and residual.stride(0) % 4 == 0 \
            and residual.data_ptr() % 16 == 0:
        return ops.gemm_mid_add_norm(a, packed, residual, norm_weight, packed=True)
    if not (a.shape[0] <= ops.ADD_NORM_MAX_ROWS and ops.skinny_supported(a, weight, torch.float32)):
        return None
    if packed is not None:
        return ops.gemm_skinny_add_norm(a, packed, residual, norm_weight, packed=True)
    return ops.gemm_skinny_add_norm(a, weight, residual, norm_weight)


def mid_qkv_takes(n_rows: int, weight: Union[torch.Tensor, Weight]) -> bool:
    """Whether the q, k, v product of this many rows goes to the kernel that shares the rows through LDS, with the
    rotation and the cache write in its epilogue (with a packed weight, beyond the rows of the weight-streaming
    kernel: it replaces the library's product and the rotation kernel after it)."""
    w, packed = _split(weight)
    t = ops.TUNING
    if not (packed is not None and t.mid_qkv_rows < n_rows <= min(ops.MID_MAX_ROWS, t.mid_qkv_max_rows)
            and w.dim() == 2 and w.shape[1] % 128 == 0):
        return False
    # a workgroup takes 32 of the weight's rows over all of K and reads every row of the batch: beyond 32 rows of the
    # batch that pays only while the workgroups run in one round (the Llama-3-8B shape has 192 of them; with the 384 of
    # the Llama-2-7B shape and the 320 of the 70B shape, whole steps of 64 and 128 requests were 4 to 8 % slower than
    # with the library's product, those of 24 requests 3 to 4 % faster)
    return n_rows <= t.mid_qkv_one_round_rows or w.shape[0] // 32 <= t.compute_units


def linear_qkv_rope(h, weight: Union[torch.Tensor, Weight], positions, slots, cos, sin, cache_pages, heads: int,
                    kv_heads: int, head_dim: int, page_size: int):
    """The q, k, v product with the rotation of q and k and the write of k and v into the cache in
    its epilogue (``h``: bfloat16 rows or ScaledRows): returns the rotated queries, or None if no
    kernel for it takes these operands (then nothing has been done)."""
    whole = weight
    weight, packed = _split(weight)
    rows = h.rows if isinstance(h, ScaledRows) else h
    if not (rows.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and cache_pages.dtype == torch.bfloat16):
        return None
    if not isinstance(h, ScaledRows) and mid_qkv_takes(rows.shape[0], whole) \
            and ops.mid_qkv_rope_supported(rows, weight, heads, kv_heads, head_dim):
        return ops.gemm_mid_qkv_rope(rows, packed, positions, slots, cos, sin, cache_pages, heads, kv_heads, head_dim,
                                     page_size, packed=True)
    if not ops.qkv_rope_supported(rows, weight, heads, kv_heads, head_dim):
        return None
    kw = dict(row_sumsq=h.sumsq, norm_width=h.width, eps=h.eps) if isinstance(h, ScaledRows) else {}
    if packed is not None:
        return ops.gemm_skinny_qkv_rope(rows, packed, positions, slots, cos, sin, cache_pages, heads, kv_heads, head_dim,
                                        page_size, packed=True, **kw)
    return ops.gemm_skinny_qkv_rope(rows, weight, positions, slots, cos, sin, cache_pages, heads, kv_heads, head_dim,
                                    page_size, **kw)
