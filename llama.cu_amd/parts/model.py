"""A decoder built from a ModelSpec: embedding, the layers in their run order, final
norm and output matrix.

Embedding is a row copy with no scale and no position term
(llama.cu/src/op/embedding.cuh:6-8, llama.cu/src/model/mod.rs:91-99).  The output
selects the wanted rows first, then norms them, then multiplies by the output matrix,
which is the embedding table when the model ties them
(llama.cu/src/exec/output_head.rs:69-100, llama.cu/src/model/mod.rs:83-88).  Logits are
float32 on both paths.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .base import BuildContext, ModelSpec, Part, ScaledRows, TensorSpec, make_part, prefixed, register_part
from .linear import Weight, linear, linear_scaled, skinny_takes


class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.weight = None

    def tensors(self):
        return {"weight": TensorSpec((self.vocab_size, self.hidden_size))}

    def load(self, tensors, build: BuildContext) -> None:
        self.weight = tensors["weight"].contiguous()

    def forward(self, tokens: torch.Tensor) -> torch.Tensor:
        """The residual stream of the step's tokens, float32 ``[n, d]``."""
        out = torch.empty((tokens.numel(), self.hidden_size), dtype=torch.float32, device=tokens.device)
        return ops.embedding_gather(self.weight, tokens, out)


class OutputHead(Part):
    graph_safe = True

    """``logits = y @ W.T``; ``tied``: W is the embedding table."""

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool = False):
        self.vocab_size, self.hidden_size, self.tied = int(vocab_size), int(hidden_size), bool(tied)
        self.weight = None

    def tensors(self):
        # a file may hold the matrix although the model ties it (then it is not used), or
        # hold none although it does not (then the table is used: the reference's rule)
        return {"weight": TensorSpec((self.vocab_size, self.hidden_size), optional=True, random=not self.tied)}

    def load(self, tensors, build: BuildContext, table: Optional[torch.Tensor] = None) -> None:
        own = tensors.get("weight")
        self.weight = Weight(table if (self.tied or own is None) else own, build)
        self.dtype = build.dtype

    def takes_scaled_rows(self, n_rows: int) -> bool:
        """Whether ``forward`` could be given ScaledRows of ``n_rows`` rows made with the final norm."""
        return (self.dtype == torch.bfloat16 and n_rows <= ops.ADD_NORM_MAX_ROWS
                and skinny_takes(n_rows, self.weight, preferred=True))

    def forward(self, y) -> torch.Tensor:
        if isinstance(y, ScaledRows):
            return linear_scaled(y, self.weight, out_dtype=torch.float32)
        return linear(y, self.weight, out_dtype=torch.float32)


register_part("embedding", "tokens", TokenEmbedding)
register_part("head", "linear", OutputHead)


class DecoderModel:
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.embedding = make_part("embedding", spec.embedding)
        self.layers: List[Part] = [make_part("block", s) for s in spec.layers]
        self.final_norm = make_part("norm", spec.final_norm)
        self.head = make_part("head", spec.head)
        self.graph_safe = all(p.graph_safe for p in [self.embedding, self.final_norm, self.head] + self.layers)
        n = len(self.layers)
        for i, e in enumerate(spec.run_order):
            if not 0 <= e.layer < n:
                raise ValueError(f"run order entry {i} names layer {e.layer}, but there are {n} layers")
            if e.cache_of is not None:
                if not 0 <= e.cache_of < i:
                    raise ValueError(f"run order entry {i} reads the cache of entry {e.cache_of}, which does not run before it")
                if spec.run_order[e.cache_of].cache_of is not None:
                    raise ValueError(f"run order entry {i} reads the cache of entry {e.cache_of}, which has none of its own")

    # ---- weights
    def _named_parts(self):
        yield self.spec.embedding.name, self.embedding
        for s, p in zip(self.spec.layers, self.layers):
            yield s.name, p
        yield self.spec.final_norm.name, self.final_norm
        yield self.spec.head.name, self.head

    def tensors(self) -> Dict[str, TensorSpec]:
        out: Dict[str, TensorSpec] = {}
        for prefix, part in self._named_parts():
            for k, v in part.tensors().items():
                out[prefixed(prefix, k)] = v
        return out

    def fused_groups(self, dtype, device):
        """The parts' fused groups under their full tensor names, as the weight loader takes them."""
        from ..weights.loader import FusedGroup
        out = []
        for prefix, part in self._named_parts():
            out += [FusedGroup(tuple(prefixed(prefix, n) for n in names), pad) for names, pad in part.fused_groups(dtype, device)]
        return out

    def load(self, tensors: Dict[str, torch.Tensor], build: BuildContext) -> None:
        for prefix, part in self._named_parts():
            pre = prefix + "." if prefix else ""
            mine = {k[len(pre):]: v for k, v in tensors.items() if k.startswith(pre)}
            if part is self.head:
                part.load(mine, build, table=self.embedding.weight)
            else:
                part.load(mine, build)

    # ---- caches
    def cache_needs(self):
        """For every entry of the run order: the need of its layer's mixer, or None if it
        reads another entry's cache (or needs none)."""
        needs = []
        for e in self.spec.run_order:
            needs.append(None if e.cache_of is not None else self.layers[e.layer].cache_need())
        return needs

    # ---- one step
    def prepare(self, step) -> None:
        """What the parts derive from the batch on the host (``Part.prepare``), before the step runs."""
        for layer in self.layers:
            layer.prepare(step)

    def forward(self, step, caches) -> torch.Tensor:
        """Logits ``[len(step.logit_rows), vocab]`` (float32) for the batch ``step``;
        ``caches[i]`` is the cache of run-order entry ``i``."""
        with ops.stream_scope():                  # the whole pass goes to one stream, asked for once
            x = self.embedding.forward(step.tokens)
            pending = None
            order = self.spec.run_order
            for i, e in enumerate(order):
                # a block may end in the norm that follows it, if what comes then takes such rows: the
                # next block with its first norm, or, when every token's logits are wanted, the output
                # matrix with the final norm
                if i + 1 < len(order):
                    follower = self.layers[order[i + 1].layer]
                    norm = follower.first_norm
                else:
                    follower = self.head if step.logits_all and self.final_norm.deferrable else None
                    norm = self.final_norm
                layer = self.layers[e.layer]
                kw = {}
                if follower is not None and norm is not None and layer.ends_in_next_norm and follower.takes_scaled_rows(x.shape[0]):
                    kw["next_norm"] = norm
                # a block may leave its last product's partial sums to the norm that adds its output,
                # if that norm takes them: the next block's first, or the final norm when no rows are
                # gathered before it
                if layer.ends_in_planes:
                    takes = self.layers[order[i + 1].layer].takes_planes if i + 1 < len(order) \
                        else (step.logits_all and self.final_norm.takes_planes)
                    if takes:
                        kw["planes_ok"] = True
                pending = layer.forward(x, pending, step, caches[i], **kw)
            if step.n_logits == 0:
                return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=x.device)
            if isinstance(pending, ScaledRows):          # the last block ended in the final norm
                return self.head.forward(pending)
            if step.logits_all:
                xs, ps = x, pending
            else:
                xs = ops.gather_rows(x, step.logit_rows)
                ps = ops.gather_rows(pending, step.logit_rows) if pending is not None else None
            y = self.final_norm.forward(xs, ps)
            return self.head.forward(y)
