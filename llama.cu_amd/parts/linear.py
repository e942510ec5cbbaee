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

from typing import Optional

import torch

from ..kernels import ops


def linear(x: torch.Tensor, weight: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
           out: Optional[torch.Tensor] = None, accumulate: bool = False) -> torch.Tensor:
    """``out (+)= x @ weight.T``.  ``accumulate`` adds into a float32 ``out`` in 32-bit."""
    if not x.is_cuda:
        raise ops.KernelError("linear: operands must be on the GPU (there is no CPU path)")
    out_dtype = out.dtype if out is not None else (out_dtype or x.dtype)
    all_bf16 = x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
    if all_bf16 and ops.skinny_supported(x, weight, out_dtype) and (
            accumulate or ops.skinny_preferred(x.shape[0], weight.shape[0], weight.shape[1], out_dtype)):
        return ops.gemm_skinny(x, weight, out=out, out_dtype=out_dtype, accumulate=accumulate)
    if all_bf16 and out_dtype == torch.bfloat16 and not accumulate:
        if out is None:
            return torch.matmul(x, weight.t())
        return torch.matmul(x, weight.t(), out=out)
    if all_bf16 and out_dtype == torch.float32 and not accumulate and out is None and x.shape[0] > ops.SKINNY_ROWS:
        return torch.mm(x, weight.t(), out_dtype=torch.float32)      # 32-bit accumulation, stored unrounded (logits)
    if ops.skinny_f32_supported(x, weight, out_dtype):
        return ops.gemm_skinny_f32(x, weight, out=out, accumulate=accumulate)
    return ops.gemm_nt(x, weight, out=out, out_dtype=out_dtype, accumulate=accumulate)


def linear_into_norm(a: torch.Tensor, weight: torch.Tensor, residual: torch.Tensor, norm_weight: torch.Tensor):
    """``residual += a @ weight.T`` and the rows for the product after the next norm, in one
    kernel: returns ``(rows, sumsq)`` for a ``ScaledRows``, or None if the kernel for it does
    not take these operands (then nothing has been done)."""
    if not (a.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and a.shape[0] <= ops.ADD_NORM_MAX_ROWS
            and residual.dtype == torch.float32 and ops.skinny_supported(a, weight, torch.float32)
            and norm_weight.dtype in (torch.bfloat16, torch.float32)):
        return None
    return ops.gemm_skinny_add_norm(a, weight, residual, norm_weight)
