"""The dense feed-forward: ``down(gate * sigmoid(gate) * up)``.

gate and up projections as one matrix product (gate rows first, the layout of the
reference's fused tensor, llama.cu/src/model/mod.rs:140-147), the activation of
llama.cu/src/op/swiglu.cuh:1-20 in 32-bit, then the down projection
(llama.cu/src/model/mod.rs:148-153).
"""
from __future__ import annotations

from typing import Dict

import torch

from ..kernels import ops
from .base import BuildContext, Part, ScaledRows, TensorSpec, register_part
from ..weights.loader import fused_rows
from .linear import (Weight, library_friendly_rows, linear, linear_into_norm, linear_planes, linear_swiglu,
                     linear_swiglu_mid, mid_swiglu_takes, mid_takes, skinny_row_limit, skinny_takes)


class SwiGLU(Part):
    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.w_gate_up = self.w_down = None

    def tensors(self) -> Dict[str, TensorSpec]:
        d, di = self.hidden_size, self.intermediate_size
        return {"gate_proj.weight": TensorSpec((di, d)), "up_proj.weight": TensorSpec((di, d)),
                "down_proj.weight": TensorSpec((d, di))}

    def _padded_rows(self, dtype, device) -> int:
        """Rows of each half of the plain gate/up matrix: more than ``intermediate_size`` where the library's
        product of many rows is faster with rows of zeros behind each half (``library_friendly_rows``)."""
        if dtype == torch.bfloat16 and torch.device(device).type == "cuda":
            return library_friendly_rows(self.intermediate_size, self.hidden_size, device)
        return self.intermediate_size

    def fused_groups(self, dtype, device):
        rows = self._padded_rows(dtype, device)
        return [(("gate_proj.weight", "up_proj.weight"), rows if rows != self.intermediate_size else 0)]

    def load(self, tensors, build: BuildContext) -> None:
        g, u = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        rows = self.intermediate_size
        if build.dtype == torch.bfloat16 and g.dtype == u.dtype == torch.bfloat16 and g.is_cuda:
            rows = self._padded_rows(build.dtype, g.device)
        if rows != self.intermediate_size:
            # the plain copy, which the library multiplies, has rows of zeros behind each half; the
            # copy that the decode kernels stream does not
            plain = fused_rows([g, u], pad_rows_to=rows)
            self.w_gate_up = Weight(plain, build, packed_from=torch.cat([g, u], dim=0) if build.pack_weights else None, halves=True)
        else:
            self.w_gate_up = Weight(fused_rows([g, u]), build, halves=True)
        self.w_down = Weight(tensors["down_proj.weight"], build)
        self.dtype = build.dtype

    def takes_scaled_rows(self, n_rows: int) -> bool:
        """Whether ``forward`` could be given ScaledRows of ``n_rows`` rows in the place of
        plain rows: the factor then goes into the first product's epilogue."""
        if self.dtype != torch.bfloat16:
            return False
        if n_rows <= min(ops.ADD_NORM_MAX_ROWS, skinny_row_limit(self.w_gate_up)) and skinny_takes(n_rows, self.w_gate_up):
            return True
        # more rows: the kernel that shares the rows through LDS applies the factor too
        return n_rows <= ops.MID_MAX_SCALED_ROWS and mid_swiglu_takes(n_rows, self.w_gate_up)

    # forward(..., into=(residual, norm)) may end with the residual sum and that norm's weight
    # in the down projection and return ScaledRows instead of the branch's output
    ends_in_norm = True
    # forward(..., planes_ok=True) may return the branch's output as float32 planes of partial sums
    ends_in_planes = True

    def forward(self, h, into=None, planes_ok=False):
        if isinstance(h, ScaledRows) and mid_swiglu_takes(h.rows.shape[0], self.w_gate_up) and ops.mid_supported(h.rows, self.w_gate_up.plain):
            act = linear_swiglu_mid(h, self.w_gate_up)
        elif isinstance(h, ScaledRows):
            if not ops.skinny_supported(h.rows, self.w_gate_up.plain, self.dtype):
                raise ops.KernelError("feed-forward: rows that wait for their normalisation need the kernel for few rows")
            act = linear_swiglu(h.rows, self.w_gate_up, row_sumsq=h.sumsq, norm_width=h.width, eps=h.eps)
        elif self.dtype == torch.bfloat16 and mid_swiglu_takes(h.shape[0], self.w_gate_up) and ops.mid_supported(h, self.w_gate_up.plain):
            # 15 to 192 rows (mid_swiglu_max_rows): the rows shared through LDS, the activation in the product's epilogue
            act = linear_swiglu_mid(h, self.w_gate_up)
        elif (self.dtype == torch.bfloat16 and h.shape[0] <= skinny_row_limit(self.w_gate_up)
              and ops.skinny_supported(h, self.w_gate_up.plain, self.dtype)):
            # few rows: one pass over the weights, the activation in the product's epilogue
            act = linear_swiglu(h, self.w_gate_up)
        else:
            gu = linear(h, self.w_gate_up, out_dtype=self.dtype)
            act = ops.swiglu(gu)
        if act.shape[1] != self.intermediate_size:
            act = act[:, :self.intermediate_size]      # without what the rows of zeros gave
        if planes_ok and act.dtype == torch.bfloat16 and mid_takes(act.shape[0], self.w_down):
            # from 12 rows on the product cut over K and the norm kernel that adds its planes are faster
            # than the weight-streaming product with that norm in its epilogue (30 against 35 us)
            return linear_planes(act, self.w_down)
        if into is not None and act.dtype == torch.bfloat16 and skinny_takes(act.shape[0], self.w_down, preferred=True):
            # only where the kernel for few rows is the faster one for this product anyway
            residual, norm = into
            fused = linear_into_norm(act, self.w_down, residual, norm.weight)
            if fused is not None:
                return ScaledRows(fused[0], fused[1], norm.size, norm.eps)
        return linear(act, self.w_down, out_dtype=self.dtype)


register_part("ffn", "swiglu", SwiGLU)
