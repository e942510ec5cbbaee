"""The arrangement of norm, mixer, norm and feed-forward in one layer.

``prenorm``: ``x += mixer(norm1(x)); x += ffn(norm2(x))``
(llama.cu/src/model/mod.rs:100-157, ``TransformerBlk::new(norm, attention, norm, mlp)``;
the residual is added where the output and down projections end,
llama.cu/src/op/linear.rs:35-62).  Here the residual stream ``x`` is float32 and each
sum is made in 32-bit inside the norm kernel that follows it: a block returns its last
branch's output as ``pending``, and whoever norms next adds it.
"""
from __future__ import annotations

from typing import Dict

import torch

from .base import BuildContext, Part, PartSpec, ScaledRows, TensorSpec, make_part, prefixed, register_part


class PreNormBlock(Part):
    def __init__(self, norm1: PartSpec, mixer: PartSpec, norm2: PartSpec, ffn: PartSpec):
        self.specs = {"norm1": norm1, "mixer": mixer, "norm2": norm2, "ffn": ffn}
        self.norm1 = make_part("norm", norm1)
        self.mixer = make_part("mixer", mixer)
        self.norm2 = make_part("norm", norm2)
        self.ffn = make_part("ffn", ffn)
        self.graph_safe = all(p.graph_safe for p in (self.norm1, self.mixer, self.norm2, self.ffn))
        # parts that say so may pass rows between them whose normalisation is still to be applied
        self._fuse = self.mixer.ends_in_norm and self.norm2.deferrable

    def _children(self):
        return [(self.specs[k].name, getattr(self, k)) for k in ("norm1", "mixer", "norm2", "ffn")]

    def tensors(self) -> Dict[str, TensorSpec]:
        out = {}
        for name, part in self._children():
            for k, v in part.tensors().items():
                out[prefixed(name, k)] = v
        return out

    def load(self, tensors, build: BuildContext) -> None:
        for name, part in self._children():
            pre = name + "." if name else ""
            part.load({k[len(pre):]: v for k, v in tensors.items() if k.startswith(pre)}, build)

    def fused_groups(self, dtype, device):
        out = []
        for name, part in self._children():
            out += [(tuple(prefixed(name, n) for n in names), pad) for names, pad in part.fused_groups(dtype, device)]
        return out

    def cache_need(self):
        return self.mixer.cache_need()

    def prepare(self, step) -> None:
        for _, part in self._children():
            part.prepare(step)

    def decode_splits(self, batch: int, max_ctx_len: int) -> int:
        return int(self.mixer.decode_splits(batch, max_ctx_len))

    @property
    def first_norm(self):
        return self.norm1

    ends_in_next_norm = True     # forward takes ``next_norm``
    ends_in_planes = True        # forward takes ``planes_ok``

    @property
    def takes_planes(self) -> bool:
        """Whether ``pending`` may be float32 planes of partial sums: the first norm adds them."""
        return bool(self.norm1.takes_planes)

    def takes_scaled_rows(self, n_rows: int) -> bool:
        """Whether ``forward`` could be given, as ``pending``, ScaledRows of ``n_rows`` rows made
        with this block's first norm in the place of the last branch's output."""
        return bool(self.norm1.deferrable and self.mixer.takes_scaled_rows(n_rows))

    def forward(self, x: torch.Tensor, pending, step, cache, next_norm=None, planes_ok=False):
        """``pending``: the last branch's output, not yet added to ``x`` (or None, or ScaledRows
        made with ``norm1`` by the block before, the sum then being in ``x`` already).
        ``next_norm``: the norm that will follow this block, if whoever runs it takes
        ScaledRows; then the feed-forward may end in it.  ``planes_ok``: whoever takes the new
        ``pending`` adds float32 planes of partial sums as well as plain rows.  Returns the new
        ``pending``."""
        h = pending if isinstance(pending, ScaledRows) else self.norm1.forward(x, pending)
        n_rows = x.shape[0]
        ffn_into = (x, next_norm) if next_norm is not None and self.ffn.ends_in_norm else None
        ffn_kw = {"into": ffn_into} if ffn_into else {}
        if planes_ok and self.ffn.ends_in_planes:
            ffn_kw["planes_ok"] = True
        mixer_kw = {}
        if self.norm2.takes_planes and self.mixer.ends_in_planes:
            mixer_kw["planes_ok"] = True
        if self._fuse and self.ffn.takes_scaled_rows(n_rows):
            # the mixer may end with the residual sum and the second norm's weight in its last
            # product; then the feed-forward applies the norm's factor in its first one
            a = self.mixer.forward(h, step, cache, into=(x, self.norm2), **mixer_kw)
            if isinstance(a, ScaledRows):
                return self.ffn.forward(a, **ffn_kw)
        else:
            a = self.mixer.forward(h, step, cache, **mixer_kw)
        h2 = self.norm2.forward(x, a)
        return self.ffn.forward(h2, **ffn_kw)


register_part("block", "prenorm", PreNormBlock)
