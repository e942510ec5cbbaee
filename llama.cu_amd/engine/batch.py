"""The batch of one step, as the model's parts see it, and the builder that lays it
out in pinned host memory and brings it to the device in one copy.

The reference builds the same facts per round: the tokens, their positions
(``pos()``), the rows whose output is wanted (``out_idx()``) and one ``Req{cache, pos,
seq}`` per request (llama.cu/src/exec/engine.rs:352-371, llama.cu/src/exec/group.rs:19-24),
staged through pinned buffers (llama.cu/src/exec/engine.rs:373-429).  Here a request's
tokens may be any portion of its prompt or one decoded token, and the requests' pages
come as block tables.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence

import torch

from ..cache import CacheManager


@dataclass
class StepContext:
    """Everything about one step that kernels need.  All tensors are int32 on the device.

    ``tokens, positions, req_of_token``: per token.  ``q_start``: [requests + 1] offsets
    of each request's tokens; ``ctx_len``: tokens each request holds after this step;
    ``state_slot``: each request's slot for per-request state; ``logit_rows``: the tokens
    whose logits are wanted.  A request's tokens stand at positions
    ``ctx_len - q_len .. ctx_len - 1``.  The lists hold the same facts on the host, for
    the choice of kernels."""
    n: int
    n_req: int
    tokens: torch.Tensor
    positions: torch.Tensor
    req_of_token: torch.Tensor
    q_start: torch.Tensor
    ctx_len: torch.Tensor
    state_slot: torch.Tensor
    logit_rows: torch.Tensor
    n_logits: int
    block_tables: List[torch.Tensor]
    slot_maps: List[torch.Tensor]
    q_lens: List[int] = field(default_factory=list)
    ctx_lens: List[int] = field(default_factory=list)
    req_ids: List[int] = field(default_factory=list)
    state_slots: List[int] = field(default_factory=list)    # ``state_slot`` on the host
    logits_all: bool = False                    # the logits of every token are wanted, in order (logit_rows is 0, 1, ...)
    attn_splits: Optional[int] = None           # fixed number of key parts for the decode kernel (captured graphs)
    scratch: dict = field(default_factory=dict)  # what kernels' wrappers derive from the batch once per step
    # tokens that the step before sampled and the host does not know yet: tokens[feed_dst[i]] is
    # to be taken from row feed_src[i] of that step's sampled ids, on the device
    feed_src: Optional[torch.Tensor] = None
    feed_dst: Optional[torch.Tensor] = None
    # the requests' indices, the one that holds most tokens first: the order in which the decode attention starts its
    # workgroups (those that walk the most keys must not start last)
    decode_order: Optional[torch.Tensor] = None
    # who built the step, if its memory can take more arrays (``extra``)
    builder: Optional["BatchBuilder"] = None

    def extra(self, name: str, size: int):
        """``(host, device)``: two int32 arrays of ``size`` entries under ``name`` in the step's own memory, for what
        a part derives from the batch on the host before the step runs (``Part.prepare``): the host array goes to
        the device with the batch's one copy, and the device array's address is the same in every step, so a
        captured graph reads the new step's values.  None if the step was not made by a builder."""
        return self.builder.extra(name, size) if self.builder is not None else None

    def block_table(self, group: int) -> torch.Tensor:
        return self.block_tables[group]

    def slots(self, group: int) -> torch.Tensor:
        return self.slot_maps[group]

    @property
    def max_q_len(self) -> int:
        return max(self.q_lens) if self.q_lens else 0

    @property
    def max_ctx_len(self) -> int:
        return max(self.ctx_lens) if self.ctx_lens else 0

    @property
    def decode_only(self) -> bool:
        return self.max_q_len == 1


class BatchBuilder:
    """Lays the arrays of a step out in one pinned host buffer and one device buffer of
    fixed capacity, so a step costs one host-to-device copy and the device addresses
    never change (a captured graph can read them)."""

    def __init__(self, cache: CacheManager, max_tokens: int, max_reqs: int, max_pages: Sequence[int],
                 device: torch.device, extra_ints: Optional[int] = None):
        """``extra_ints``: room for the arrays that parts add to a step (``StepContext.extra``); by default two
        entries per token and eight per request."""
        self.cache = cache
        self.max_tokens, self.max_reqs = int(max_tokens), int(max_reqs)
        self.max_pages = [int(m) for m in max_pages]
        self.device = device
        n, r = self.max_tokens, self.max_reqs
        sizes = [("tokens", n), ("positions", n), ("req_of_token", n), ("logit_rows", n),
                 ("q_start", r + 1), ("ctx_len", r), ("state_slot", r), ("feed_src", r), ("feed_dst", r), ("decode_order", r)]
        for g, mp in enumerate(self.max_pages):
            sizes += [(f"slots{g}", n), (f"block_table{g}", r * mp)]
        self.extra_ints = int(extra_ints) if extra_ints is not None else 2 * n + 8 * r + 256
        sizes.append(("extra", self.extra_ints))
        self._extra_used = 0
        self._extras = {}                       # name -> (offset in the extra area, size): the same in every step
        self.offsets = {}
        total = 0
        for name, size in sizes:
            self.offsets[name] = (total, size)
            total += (size + 3) // 4 * 4
        pin = device.type == "cuda"
        self.host = torch.zeros(total, dtype=torch.int32, pin_memory=pin)
        self.dev = torch.zeros(total, dtype=torch.int32, device=device)
        self._copied: Optional[torch.cuda.Event] = None

    def _h(self, name: str) -> torch.Tensor:
        o, s = self.offsets[name]
        return self.host[o:o + s]

    def _d(self, name: str, count: int) -> torch.Tensor:
        o, s = self.offsets[name]
        return self.dev[o:o + count]

    def extra(self, name: str, size: int):
        """``(host, device)`` views of ``size`` entries that ``name`` owns from its first call on (the same
        addresses in every step)."""
        at = self._extras.get(name)
        if at is None:
            if self._extra_used + size > self.extra_ints:
                raise ValueError(f"the step's memory has no room for {size} more entries under {name!r} "
                                 f"({self._extra_used} of {self.extra_ints} are taken): build with a larger extra_ints")
            at = self._extras[name] = (self._extra_used, int(size))
            self._extra_used += (int(size) + 3) // 4 * 4
        if at[1] < size:
            raise ValueError(f"{name!r} holds {at[1]} entries, {size} were asked for")
        o = self.offsets["extra"][0] + at[0]
        return self.host[o:o + size], self.dev[o:o + size]

    def upload(self) -> None:
        """The step's arrays go to the device (one copy on the current stream)."""
        self.dev.copy_(self.host, non_blocking=True)
        if self.device.type == "cuda":
            self._copied = torch.cuda.Event()
            self._copied.record()

    def build(self, req_ids: Sequence[int], tokens: Sequence[Sequence[int]], want: Sequence[Sequence[int]],
              vocab_size: int, feed: Sequence[tuple] = (), upload: bool = True) -> StepContext:
        """The batch in which request ``req_ids[i]`` feeds ``tokens[i]`` and wants the logits
        at the places ``want[i]`` among them.  The requests' pages must be reserved.
        ``feed``: pairs (row of the last step's sampled ids, request index here) for requests
        whose last token here is a placeholder that the device fills in.  ``upload=False``: the
        caller lets parts add their arrays (``StepContext.extra``) and calls ``upload`` then."""
        n_req = len(req_ids)
        n_new = [len(t) for t in tokens]
        n = sum(n_new)
        if n_req == 0 or n == 0:
            raise ValueError("a step needs at least one request with at least one token")
        if n > self.max_tokens or n_req > self.max_reqs:
            raise ValueError(f"step of {n} tokens / {n_req} requests exceeds the builder's capacity "
                             f"({self.max_tokens} / {self.max_reqs})")
        if self._copied is not None:
            self._copied.synchronize()          # the last copy out of the host buffer has ended
        flat = [t for ts in tokens for t in ts]
        lo, hi = min(flat), max(flat)
        if lo < 0 or hi >= vocab_size:
            raise ValueError(f"token id {lo if lo < 0 else hi} is outside the vocabulary of {vocab_size}")
        self._h("tokens")[:n] = torch.tensor(flat, dtype=torch.int32)
        rows = []
        start = 0
        for i, w in enumerate(want):
            for k in w:
                if not 0 <= k < n_new[i]:
                    raise ValueError(f"request {req_ids[i]}: wanted place {k} is outside its {n_new[i]} tokens")
                rows.append(start + k)
            start += n_new[i]
        if rows:
            self._h("logit_rows")[:len(rows)] = torch.tensor(rows, dtype=torch.int32)
        if feed:
            if len(feed) > self.max_reqs:
                raise ValueError(f"{len(feed)} fed tokens exceed the builder's capacity of {self.max_reqs}")
            ends, at = [], 0
            for c in n_new:
                at += c
                ends.append(at - 1)
            self._h("feed_src")[:len(feed)] = torch.tensor([f[0] for f in feed], dtype=torch.int32)
            self._h("feed_dst")[:len(feed)] = torch.tensor([ends[f[1]] for f in feed], dtype=torch.int32)
        ptr = lambda name: self._h(name).data_ptr()
        self.cache.fill_batch(req_ids, n_new, ptr("positions"), ptr("req_of_token"), ptr("q_start"), ptr("ctx_len"),
                              ptr("state_slot"), [ptr(f"block_table{g}") for g in range(len(self.max_pages))],
                              self.max_pages, [ptr(f"slots{g}") for g in range(len(self.max_pages))])
        ctx_lens = self._h("ctx_len")[:n_req].tolist()
        self._h("decode_order")[:n_req] = torch.tensor(sorted(range(n_req), key=lambda i: -ctx_lens[i]), dtype=torch.int32)
        if upload:
            self.upload()
        return StepContext(
            n=n, n_req=n_req, tokens=self._d("tokens", n), positions=self._d("positions", n),
            req_of_token=self._d("req_of_token", n), q_start=self._d("q_start", n_req + 1),
            ctx_len=self._d("ctx_len", n_req), state_slot=self._d("state_slot", n_req),
            logit_rows=self._d("logit_rows", len(rows)), n_logits=len(rows), logits_all=rows == list(range(n)),
            block_tables=[self._d(f"block_table{g}", n_req * mp).view(n_req, mp) for g, mp in enumerate(self.max_pages)],
            slot_maps=[self._d(f"slots{g}", n) for g in range(len(self.max_pages))],
            q_lens=n_new, ctx_lens=ctx_lens, req_ids=list(req_ids),
            state_slots=self._h("state_slot")[:n_req].tolist(),
            feed_src=self._d("feed_src", len(feed)) if feed else None,
            feed_dst=self._d("feed_dst", len(feed)) if feed else None,
            decode_order=self._d("decode_order", n_req), builder=self)
