"""The attention mixer: grouped-query causal attention over the paged cache.

q, k, v projections as one matrix product (rows q, then k, then v, the layout of the
reference's fused tensor, llama.cu/src/model/mod.rs:114-119), position encoding of q
and k and the write of k and v into the request's pages in one kernel, attention of
the step's queries over the cache, output projection (llama.cu/src/model/mod.rs:125-130).
The call contract of the attention itself is llama.cu/src/exec/step.rs:162-178: causal,
offset by the request's position.  Scores, softmax and the output sum are 32-bit.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import BuildContext, PagedKV, Part, PartSpec, ScaledRows, TensorSpec, make_part, register_part
from .linear import (Weight, linear, linear_into_norm, linear_planes, linear_qkv_rope, linear_scaled, mid_qkv_takes, mid_takes,
                     skinny_takes)
from ..weights.loader import fused_rows


class Attention(Part):

    def __init__(self, hidden_size: int, heads: int, kv_heads: int, head_dim: int, scale: Optional[float] = None,
                 window: int = 0, position: Optional[PartSpec] = None, shares_kv: bool = False, page_size: int = 0):
        if heads % kv_heads:
            raise ValueError(f"attention: {heads} heads are no multiple of {kv_heads} key/value heads")
        if head_dim % 16 or head_dim > 256:
            raise ValueError(f"attention: head_dim {head_dim} is not supported by the kernels "
                             f"(multiples of 16 up to 256)")
        self.hidden_size, self.heads, self.kv_heads, self.head_dim = int(hidden_size), int(heads), int(kv_heads), int(head_dim)
        self.scale = float(scale) if scale is not None else float(head_dim) ** -0.5
        self.window = int(window or 0)
        self.own_page_size = int(page_size or 0)  # tokens per page of this layer's cache; 0: the engine's default
        self.shares_kv = bool(shares_kv)          # reads another layer's keys and values: has q and o only
        self.position = make_part("position", position or PartSpec("none"))
        self.graph_safe = self.position.graph_safe
        self.w_qkv = self.w_o = None
        self.page_size = 0

    def tensors(self) -> Dict[str, TensorSpec]:
        d, nh, nkv, dh = self.hidden_size, self.heads, self.kv_heads, self.head_dim
        t = {"q_proj.weight": TensorSpec((nh * dh, d)), "o_proj.weight": TensorSpec((d, nh * dh))}
        if not self.shares_kv:
            t["k_proj.weight"] = TensorSpec((nkv * dh, d))
            t["v_proj.weight"] = TensorSpec((nkv * dh, d))
        return t

    def fused_groups(self, dtype, device):
        return [] if self.shares_kv else [(("q_proj.weight", "k_proj.weight", "v_proj.weight"), 0)]

    def cache_need(self):
        return PagedKV(self.kv_heads, self.head_dim, self.window, self.own_page_size)

    def decode_splits(self, batch: int, max_ctx_len: int) -> int:
        """Into how many parts the decode kernel should cut each request's keys when ``batch``
        requests decode over at most ``max_ctx_len`` keys (a captured graph fixes the number)."""
        return ops.decode_splits(batch, self.heads, self.kv_heads, max_ctx_len)

    def load(self, tensors, build: BuildContext) -> None:
        if self.shares_kv:
            self.w_qkv = Weight(tensors["q_proj.weight"], build)
        else:
            # one matrix with the rows of q, then k, then v: in place where the loader laid them out so
            self.w_qkv = Weight(fused_rows([tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]]), build)
        self.w_o = Weight(tensors["o_proj.weight"], build)
        self.position.load({}, build)
        # a position encoding that is its rotation tables alone (apply() does nothing of its own)
        self._rotation_only = type(self.position).apply is Part.apply
        self.page_size = build.page_size
        self.dtype = build.dtype
        if self.dtype == torch.bfloat16:
            # a bfloat16 model whose attention the matrix-core kernels do not take still runs, on the generic
            # kernel: correct, and several times slower over long contexts, so the log says so and why
            why = ops.mfma_attention_refusal(self.dtype, self.heads, self.kv_heads, self.head_dim, self.own_page_size or self.page_size)
            if why is None and self.position.score_slopes() is not None:
                why = "the position encoding is a bias inside the scores, which the matrix-core kernels do not take"
            if why is not None:
                ops.say_once(f"attention with {self.heads} heads of {self.head_dim} in {self.kv_heads} groups runs on the generic "
                             f"kernel, not on the matrix cores: {why}")

    def prepare(self, step) -> None:
        """The lists by which the matrix-core kernels share out a step that is not all single tokens are made here, on
        the host, and go to the device with the step's arrays; ``forward`` then launches work whose sizes follow from
        the step's sizes alone."""
        page_size = self.own_page_size or self.page_size
        if self.dtype == torch.bfloat16 and self.position.score_slopes() is None \
                and ops.mfma_attention_refusal(self.dtype, self.heads, self.kv_heads, self.head_dim, page_size) is None:
            ops.plan_attention(step, self.heads, self.kv_heads, self.window)

    # forward(..., into=(residual, norm)) may end with the residual sum and that norm's weight
    # in the output projection and return ScaledRows instead of the branch's output
    ends_in_norm = True
    # forward(..., planes_ok=True) may return the branch's output as float32 planes of partial sums
    ends_in_planes = True

    def takes_scaled_rows(self, n_rows: int) -> bool:
        """Whether ``forward`` could be given ScaledRows of ``n_rows`` rows in the place of
        plain rows: only where the kernel for few rows is the faster one for the q, k, v
        product anyway."""
        return self.dtype == torch.bfloat16 and n_rows <= ops.ADD_NORM_MAX_ROWS and skinny_takes(n_rows, self.w_qkv, preferred=True)

    def forward(self, h, step, cache, into=None, planes_ok=False):
        nh, nkv, dh = self.heads, self.kv_heads, self.head_dim
        if self.shares_kv == cache.writes:
            raise ops.KernelError("attention: a layer that shares another's keys and values must be given that "
                                  "layer's cache in the run order (and only such a layer)")
        page_size = cache.page_size or self.page_size          # the cache's own page size (the engine's default)
        rot = self.position.rotary_tables()
        cos, sin, rot_dim, pairing = rot if rot is not None else (None, None, 0, 0)
        store = cache.writes and not self.shares_kv
        n_rows = (h.rows if isinstance(h, ScaledRows) else h).shape[0]
        qkv = None
        if store and self._rotation_only and rot is not None and pairing == 0 and rot_dim == dh \
                and self.dtype == torch.bfloat16 and (skinny_takes(n_rows, self.w_qkv, preferred=True)
                                                      or (not isinstance(h, ScaledRows) and mid_qkv_takes(n_rows, self.w_qkv))):
            # up to 256 rows: the product rotates q and k and writes k and v into the pages itself
            qkv = linear_qkv_rope(h, self.w_qkv, step.positions, step.slots(cache.group), cos, sin, cache.pages,
                                  nh, nkv, dh, page_size)
        if qkv is None:
            if isinstance(h, ScaledRows):
                qkv = linear_scaled(h, self.w_qkv)
            else:
                qkv = linear(h, self.w_qkv, out_dtype=self.dtype)
            self.position.apply(qkv, step.positions, nh, 0 if self.shares_kv else nkv, dh)
            ops.rope_kv_store(qkv, step.positions, nh, nkv, dh, cos, sin, rot_dim, pairing,
                              cache.pages if store else None, step.slots(cache.group) if store else None,
                              page_size)
        out = torch.empty((n_rows, nh * dh), dtype=self.dtype, device=qkv.device)
        ops.paged_attention(qkv, out, cache.pages, step, cache.group, nh, nkv, dh, page_size, self.scale,
                            self.window, head_slopes=self.position.score_slopes())
        if into is not None:
            residual, norm = into
            fused = linear_into_norm(out, self.w_o, residual, norm.weight)
            if fused is not None:
                return ScaledRows(fused[0], fused[1], norm.size, norm.eps)
        if planes_ok and self.dtype == torch.bfloat16 and mid_takes(n_rows, self.w_o):
            return linear_planes(out, self.w_o)
        return linear(out, self.w_o, out_dtype=self.dtype)


register_part("mixer", "attention", Attention)
