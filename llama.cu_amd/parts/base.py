"""What a model is made of: specifications (data), parts (objects that hold weights
and run kernels) and the registries that turn the first into the second.

A *specification* is plain data: a kind, parameters, and the name under which the
part's tensors lie in the weight file.  A *part* is built from a specification by
the registry of its category:

  ``norm``      ``forward(x, delta) -> y``             x: float32 [n, d] residual stream, updated in
                                                    place by ``x += delta`` (``delta`` may be None);
                                                    y: [n, d] in the compute type
  ``mixer``     ``forward(h, step, cache) -> delta``   h, delta: [n, d] compute type; ``step`` is the
                ``cache_need() -> need or None``       batch (engine.batch.StepContext); ``cache`` is
                                                    what the engine made for ``cache_need()``
  ``ffn``       ``forward(h) -> delta``
  ``position``  ``tables(...)``/``apply(...)``         see parts.position
  ``block``     ``forward(x, pending, step, cache) -> pending``   the arrangement of the four above

Every part also has ``tensors() -> {relative name: TensorSpec}``,
``load(tensors, build)`` and the flag ``graph_safe`` (see Part).  No part knows which model it is in: sizes and constants
arrive as parameters.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Tuple

import torch


@dataclass(frozen=True)
class TensorSpec:
    """One tensor a part binds: its shape, and how a random model fills it: the name of an
    initialiser (``normal``: N(0, std); ``one_plus_normal``: 1 + N(0, std), for norm weights;
    ``zeros``; ``ones``; or one that ``weights.register_initialiser`` has made known).
    ``integer`` tensors are kept as int32, all others follow the weight policy."""
    shape: Tuple[int, ...]
    init: str = "normal"
    integer: bool = False
    optional: bool = False        # a file may lack it
    random: bool = True           # the random-weights mode makes it


@dataclass
class PartSpec:
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    name: str = ""           # the part's component in tensor names ("self_attn", "mlp", ...)


@dataclass(frozen=True)
class RunEntry:
    """One step of the run order: which layer runs, and whose cache it uses.  ``cache_of``
    None: a cache of its own.  ``cache_of = j``: it reads the cache that entry ``j`` of the
    run order wrote (and writes none)."""
    layer: int
    cache_of: Optional[int] = None


@dataclass
class ModelSpec:
    """A whole decoder as data."""
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec
    layers: List[PartSpec]              # block specifications, each with its tensor-name prefix
    run_order: List[RunEntry]
    final_norm: PartSpec
    head: PartSpec
    eos_token_ids: Tuple[int, ...] = ()


# ------------------------------------------------------------------ cache needs


@dataclass
class LayerCache:
    """What one entry of the run order gets: the pages of its layer (``pages``,
    ``[num_pages, 2, kv_heads * head_dim * page_size]``) with the group whose block tables
    index them, whether the entry writes them, and/or its per-request state
    (``state``, ``[slots, *shape]``)."""
    group: int = -1
    pages: Optional[torch.Tensor] = None
    writes: bool = True
    state: Optional[torch.Tensor] = None
    page_size: int = 0          # tokens per page of ``pages`` (0: no pages)


class CacheNeed:
    """What a mixer asks of the cache manager.  The engine knows no kind of need by name: it asks
    every need these questions.

    ``pool()``        None, or ``(window, page_size)``: the need is pages of keys and values, and needs
                      with an equal answer share one pool of page ids and one block table per request
                      (``window`` 0: every token is kept; w: pages that a window of w tokens has
                      passed are given back; ``page_size`` 0: the engine's default);
    ``page_bytes(page_size, elem_size)``   bytes of one page of this need (0 if it has no pages);
    ``allocate(group, num_pages, page_size, slots, dtype, device)``   the memory, as a LayerCache;
    ``can_truncate``  whether what the need holds for a request can be cut back to a shorter
                      length (pages can; a state that has folded tokens in cannot).  A request
                      whose cache cannot be cut back and has to be (an end-of-sequence token
                      learned after more was computed) loses its cache and is computed again from
                      its tokens when it goes on.
    """
    can_truncate = True

    def pool(self):
        return None

    def page_bytes(self, page_size: int, elem_size: int) -> int:
        return 0

    def allocate(self, group: int, num_pages: int, page_size: int, slots: int, dtype, device) -> LayerCache:
        return LayerCache()


@dataclass(frozen=True)
class PagedKV(CacheNeed):
    """Keys and values of every token (or of the last ``window`` tokens), in pages."""
    kv_heads: int
    head_dim: int
    window: int = 0          # 0: all tokens
    page_size: int = 0       # tokens per page; 0: the engine's default

    def pool(self):
        return (self.window, self.page_size)

    def page_bytes(self, page_size: int, elem_size: int) -> int:
        return 2 * self.kv_heads * self.head_dim * page_size * elem_size

    def allocate(self, group, num_pages, page_size, slots, dtype, device) -> LayerCache:
        pages = torch.zeros((num_pages, 2, self.kv_heads * self.head_dim * page_size), dtype=dtype, device=device)
        return LayerCache(group=group, pages=pages, page_size=page_size)


@dataclass(frozen=True)
class SlotState(CacheNeed):
    """A state of fixed size per request (``shape`` without the slot axis).  The mixer that owns
    it starts it anew when a request's first token (position 0) comes."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32
    can_truncate = False

    def allocate(self, group, num_pages, page_size, slots, dtype, device) -> LayerCache:
        return LayerCache(state=torch.zeros((slots,) + tuple(self.shape), dtype=self.dtype, device=device))


# ------------------------------------------------------------------ building


@dataclass
class BuildContext:
    """What a part may need to know about the engine while it binds its weights."""
    dtype: torch.dtype               # the compute type: torch.bfloat16 or torch.float32
    device: torch.device
    max_positions: int
    page_size: int
    pack_weights: bool = True        # keep a second copy of bfloat16 matrices in the order the decode kernel streams them


@dataclass
class ScaledRows:
    """Rows on their way from a norm to a matrix product whose normalisation is still to be
    applied: the norm's weight is in already, and row ``i`` of whatever is multiplied with
    them is to be multiplied by ``rsqrt(sum(sumsq[i]) / width + eps)``.  A mixer that can end
    with the residual sum and the next norm's weight in its last product hands these to a
    feed-forward that can apply the factor in its first product's epilogue, and no norm
    kernel runs between them.  A part that does not know of this never sees one: the block
    offers it only to parts that say they take it."""
    rows: torch.Tensor          # [n, width], the compute type
    sumsq: torch.Tensor         # [n, parts] float32 shares of the rows' sums of squares
    width: int
    eps: float


class Part:
    # Whether a step through this part may be captured into a graph and replayed: true only
    # if all it does is launch work on the current stream whose shape depends on the batch's
    # sizes alone, never on values it reads on the host (lengths, positions, slots).
    graph_safe = False

    # ---- what a part may offer so that kernels between it and its neighbours are saved.  All of it is
    # optional: a part that leaves these as they are is never given anything but plain rows, and
    # everything it returns is plain rows; blocks and the model ask through these names only.
    #
    # norm:  ``deferrable``: the norm is a factor per row times a weight per column (``weight``, ``size``,
    #        ``eps``), so the factor may be applied after the next matrix product (ScaledRows);
    #        ``takes_planes``: ``forward(x, delta)`` also takes float32 planes ``[planes, rows, width]``
    #        of partial sums as ``delta``.
    # mixer, feed-forward:  ``ends_in_norm``: ``forward(..., into=(residual, norm))`` may add its output to
    #        the residual stream itself and return ScaledRows made with ``norm``;
    #        ``ends_in_planes``: ``forward(..., planes_ok=True)`` may return float32 planes;
    #        ``takes_scaled_rows(n_rows)``: whether ``forward`` takes ScaledRows of that many rows.
    # block: ``ends_in_next_norm``: ``forward(..., next_norm=)`` may end in the norm that follows the block;
    #        ``ends_in_planes`` / ``takes_planes`` / ``takes_scaled_rows`` as above, for its last branch
    #        and its first norm.
    deferrable = False
    takes_planes = False
    ends_in_norm = False
    ends_in_planes = False
    ends_in_next_norm = False

    def takes_scaled_rows(self, n_rows: int) -> bool:
        return False

    # block: the norm that a block starts with, if whoever runs before it may end in it (else None)
    first_norm = None

    def decode_splits(self, batch: int, max_ctx_len: int) -> int:
        """Into how many parts a mixer (or a block, for its mixer) wants a decoding request's keys cut when
        ``batch`` requests decode over at most ``max_ctx_len`` keys; a captured graph fixes the number."""
        return 1

    # position: what a position encoding may be, each optional (``parts/position.py`` describes them): tables of
    # a rotation, any other change of queries and keys in place, a bias inside the scores.
    def rotary_tables(self):
        return None

    def apply(self, qkv, positions, heads, kv_heads, head_dim) -> None:
        pass

    def score_slopes(self):
        return None

    def tensors(self) -> Dict[str, TensorSpec]:
        return {}

    def load(self, tensors: Dict[str, torch.Tensor], build: BuildContext) -> None:
        pass

    def prepare(self, step) -> None:
        """Called once per step for every layer, on the host, before the step's arrays go to the device and
        before anything of the step runs or is replayed from a graph: a part that derives arrays from the batch
        (lists of tasks, orders) writes them into ``step.extra(name, size)`` here, so that its ``forward`` launches
        work whose shape depends on the step's sizes alone and a graph-safe part stays one."""
        pass

    def fused_groups(self, dtype: torch.dtype, device: torch.device) -> List[Tuple[Tuple[str, ...], int]]:
        """Tensors that this part multiplies as one matrix: ``[(names in row order, rows to which each
        is filled up with zeros, or 0)]``.  The weight loader lays such tensors out one after the other,
        so that the part finds the fused matrix in place (``weights.loader.fused_rows``)."""
        return []


_REGISTRIES: Dict[str, Dict[str, Callable[..., Part]]] = {
    "norm": {}, "mixer": {}, "ffn": {}, "position": {}, "block": {}, "embedding": {}, "head": {}}


def register_part(category: str, kind: str, factory: Callable[..., Part], replace: bool = False) -> None:
    """Make ``kind`` known in ``category``; ``factory(**params)`` builds the part."""
    reg = _REGISTRIES.get(category)
    if reg is None:
        raise ValueError(f"no part category {category!r}; categories: {sorted(_REGISTRIES)}")
    if kind in reg and not replace:
        raise ValueError(f"{category} part {kind!r} is already registered")
    reg[kind] = factory


def make_part(category: str, spec: PartSpec) -> Part:
    reg = _REGISTRIES[category]
    factory = reg.get(spec.kind)
    if factory is None:
        raise ValueError(f"no {category} part of kind {spec.kind!r}; registered: {sorted(reg)}")
    return factory(**spec.params)


def registered_parts(category: str) -> List[str]:
    return sorted(_REGISTRIES[category])


def prefixed(prefix: str, name: str) -> str:
    return f"{prefix}.{name}" if prefix else name
