"""RMS normalisation, fused with the residual sum that precedes it.

``y = x * rsqrt(sum(x^2)/d + eps) * w`` (llama.cu/src/op/rms_norm.cuh:21-29), in
32-bit with one rounding at the store; the weight may be stored in another type than
the activations (llama.cu/src/op/rms_norm.rs:19-31).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import BuildContext, Part, TensorSpec, register_part


class RMSNorm(Part):
    graph_safe = True

    def __init__(self, size: int, eps: float):
        self.size = int(size)
        self.eps = float(eps)
        self.weight: Optional[torch.Tensor] = None
        self.dtype = None

    def tensors(self) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((self.size,), init="one_plus_normal")}

    def load(self, tensors, build: BuildContext) -> None:
        self.weight = tensors["weight"].contiguous()
        self.dtype = build.dtype

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``x`` (float32 residual stream) takes in ``delta`` if there is one (rows in the compute
        type, or float32 planes ``[planes, n, d]`` of partial sums); returns the normalised rows
        in the compute type."""
        out = torch.empty(x.shape, dtype=self.dtype, device=x.device)
        return ops.rmsnorm(x, self.weight, self.eps, out, delta=delta, write_back=True)


    # This norm is a factor per row times a weight per column, so its factor may be applied
    # after a matrix product instead of before (see ScaledRows); whoever does that reads
    # ``weight``, ``size`` and ``eps``.
    deferrable = True

    # ``delta`` may be planes of partial sums: a product cut over K leaves its slices' sums for
    # this kernel to add.  A branch hands them only to a norm that says so.
    takes_planes = True


register_part("norm", "rmsnorm", RMSNorm)
