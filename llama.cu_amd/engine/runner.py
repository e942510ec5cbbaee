"""The model runner: the model on the device, its caches, and the one step function.

``step`` is everything between a batch of (request, its next tokens) and the logits at
the wanted places.  It runs only the tokens it is given, as one batch, from the cache
that earlier steps left, whatever the mix: portions of prompts beside single decoded
tokens, cut anywhere.  (The reference's counterpart is ``ModelGroup::load_inputs`` +
``launch`` + ``OutputHead::launch``, llama.cu/src/exec/group.rs:89-157 and
llama.cu/src/exec/output_head.rs:55-116, which feeds whole prompts only and returns
sampled ids instead of logits.)
"""
from __future__ import annotations

import sys
from typing import Any, Dict, List, Optional, Sequence

import torch

from ..cache import CacheGroup, CacheManager, OutOfPages
from ..config import load_config
from ..kernels import ops
from ..parts import BuildContext, CacheNeed, DecoderModel, LayerCache, ModelSpec
from ..weights import load_weights, open_safetensors, random_tensors
from ..weights.loader import convert
from .batch import BatchBuilder, StepContext

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "f32": torch.float32,
          "fp32": torch.float32, torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


def free_bytes(device) -> int:
    """Memory of the card that this process can still fill: what the driver calls free, and what torch's
    allocator holds without a tensor in it."""
    free, _ = torch.cuda.mem_get_info(device)
    return int(free) + int(torch.cuda.memory_reserved(device)) - int(torch.cuda.memory_allocated(device))


def reserve_in_one_piece(device, nbytes: int) -> None:
    """Ask the driver for ``nbytes`` in ONE allocation and hand it to torch's allocator, which carves
    the tensors that follow (weights, their packed copies, the cache, the steps' buffers) out of it.  The
    card maps a large allocation with large pages; with the same tensors allocated one by one the
    weight-streaming kernels of the first sixty or so decode steps after a prefill ran 3 to 5 % slower
    (3.94 against 3.76 ms a step at 8 requests of the Llama-3-8B shape; later steps were equal).  Nothing
    depends on it but speed: too little memory for it, or a small model, and nothing is reserved."""
    if nbytes < (1 << 30):
        return
    held = int(torch.cuda.memory_reserved(device)) - int(torch.cuda.memory_allocated(device))
    nbytes = min(int(nbytes), int(0.95 * free_bytes(device)))
    if nbytes <= held:
        return                                      # the allocator holds that much already (an engine made before)
    try:
        torch.empty(nbytes, dtype=torch.uint8, device=device)      # freed at once: the allocator keeps the piece
    except RuntimeError:
        pass


def engine_bytes(spec: ModelSpec, expected, dtype: torch.dtype, device, page_size: int, max_tokens, num_pages, max_seqs: int,
                 max_batch_tokens: int, kv_fraction: float) -> int:
    """About how much memory an engine for ``spec`` will allocate (for reserve_in_one_piece)."""
    elem = torch.empty(0, dtype=dtype).element_size()
    weights = sum(int(torch.Size(t.shape).numel()) * elem for t in expected.values())
    matrices = sum(int(torch.Size(t.shape).numel()) * elem for t in expected.values() if len(t.shape) == 2)
    free = free_bytes(device)
    total = weights
    if dtype == torch.bfloat16 and free - matrices >= 0.3 * torch.cuda.mem_get_info(device)[1]:
        total += matrices                           # the packed copies
    needs = [n for n in DecoderModel(spec).cache_needs() if n is not None]
    token_bytes = sum(n.page_bytes(1, elem) for n in needs)
    if num_pages is not None:
        tokens = int(num_pages) * page_size
    elif max_tokens is not None:
        tokens = int(max_tokens)
    else:
        tokens = min(int((free - total) * kv_fraction) // max(token_bytes, 1), max_seqs * spec.max_positions)
    total += max(tokens, 0) * token_bytes
    widest = max([max(t.shape) for t in expected.values() if len(t.shape) == 2] + [1])
    total += 16 * int(max_batch_tokens) * widest * 4 + (256 << 20)        # a step's buffers and the library's workspace
    return total + total // 32                                             # and what the allocator's rounding adds


def require_gpu(device) -> torch.device:
    device = torch.device(device)
    if device.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError("llama.cu_amd runs on a GPU only (gfx950); no GPU is visible to torch "
                           "and there is no CPU fallback")
    return device


class ModelRunner:
    def __init__(self, spec: ModelSpec, tensors: Dict[str, torch.Tensor], dtype, device="cuda:0",
                 page_size: int = 16, max_tokens: Optional[int] = None, num_pages: Optional[int] = None,
                 max_seqs: int = 8, max_batch_tokens: int = 2048, max_model_len: Optional[int] = None,
                 kv_fraction: float = 0.85, use_graphs: bool = True, pack_weights: Optional[bool] = None,
                 poison_freed: bool = False):
        self.device = require_gpu(device)
        self.dtype = DTYPES[dtype]
        self.spec = spec
        self.page_size = int(page_size)
        if self.page_size % 8:
            raise ValueError(f"page_size {page_size} must be a multiple of 8")
        self.max_model_len = min(int(max_model_len or spec.max_positions), spec.max_positions)
        self.max_seqs, self.max_batch_tokens = int(max_seqs), int(max_batch_tokens)
        torch.cuda.set_device(self.device)
        ops.tune_for(self.device)
        self.model = DecoderModel(spec)
        if pack_weights is None:
            # the second, packed copy of the matrices is worth its memory only while most of the
            # card stays free for the cache: an 8B model takes it, a 70B model on one card does not
            matrices = sum(t.numel() * t.element_size() for t in tensors.values() if t.dim() == 2)
            total = torch.cuda.mem_get_info(self.device)[1]
            pack_weights = self.dtype == torch.bfloat16 and free_bytes(self.device) - matrices >= 0.3 * total
        self.pack_weights = bool(pack_weights)
        build = BuildContext(self.dtype, self.device, spec.max_positions, self.page_size, self.pack_weights)
        self.model.load(tensors, build)

        # cache groups: one per distinct pool that the layers' needs name (for keys and values in pages:
        # one per window); what a need is made of is the need's own business (parts.base.CacheNeed)
        needs = self.model.cache_needs()
        for i, need in enumerate(needs):
            if need is not None and not isinstance(need, CacheNeed):
                raise ValueError(f"run order entry {i}: {need!r} is no cache need (parts.base.CacheNeed)")
        pools = sorted({n.pool() for n in needs if n is not None and n.pool() is not None})
        page_of = [p[1] or self.page_size for p in pools]            # a pool's own page size, or the engine's
        for ps in page_of:
            if ps % 8:
                raise ValueError(f"page_size {ps} must be a multiple of 8")
        elem = torch.empty(0, dtype=self.dtype).element_size()
        tokens = int(max_tokens) if max_tokens is not None else None
        if num_pages is not None:
            tokens = int(num_pages) * self.page_size                  # the pool's size was given in the engine's pages
        if tokens is None:
            # what the free memory holds, and no more than every slot filled to the limit
            token_bytes = sum(n.page_bytes(1, elem) for n in needs if n is not None)
            by_memory = int(free_bytes(self.device) * kv_fraction) // max(token_bytes, 1)
            by_need = self.max_seqs * ((self.max_model_len + max(page_of + [self.page_size]) - 1) // self.page_size * self.page_size)
            tokens = max(self.page_size, min(by_memory, by_need))
        # every pool holds the same number of tokens, in pages of its own size
        self.num_pages = (tokens + self.page_size - 1) // self.page_size
        # a window keeps its pages one token longer than the next query needs: the engine runs one round ahead of
        # its sampler's results and cuts a request back by the token it computed beyond an end of sequence
        self.groups = [CacheGroup((tokens + ps - 1) // ps, ps, p[0], slack=1 if p[0] else 0) for p, ps in zip(pools, page_of)]
        # whether every need's state of fixed size can be cut back to a shorter length (the manager knows what its
        # pages and windows can); a request that cannot be cut back gives up what cannot and is computed again
        self.can_truncate = all(n.can_truncate for n in needs if n is not None)
        self.cache = CacheManager(self.groups, self.max_seqs, can_truncate=self.can_truncate)
        self.caches: List[LayerCache] = []
        for i, (entry, need) in enumerate(zip(spec.run_order, needs)):
            if entry.cache_of is not None:
                src = self.caches[entry.cache_of]
                self.caches.append(LayerCache(group=src.group, pages=src.pages, writes=False, state=src.state))
            elif need is None:
                self.caches.append(LayerCache())
            else:
                group = pools.index(need.pool()) if need.pool() is not None else -1
                pages, ps = (self.groups[group].num_pages, page_of[group]) if group >= 0 else (self.num_pages, self.page_size)
                try:
                    made = need.allocate(group, pages, ps, self.max_seqs, self.dtype, self.device)
                except torch.cuda.OutOfMemoryError:
                    # what torch's allocator holds without a tensor in it (the rest of a piece reserved for another
                    # engine, say) goes back to the driver, and the allocation is tried once more
                    torch.cuda.empty_cache()
                    made = need.allocate(group, pages, ps, self.max_seqs, self.dtype, self.device)
                self.caches.append(made)
        max_pages = [(self.max_model_len + g.page_size - 1) // g.page_size for g in self.groups]
        self.builder = BatchBuilder(self.cache, self.max_batch_tokens, self.max_seqs, max_pages, self.device)
        # a debugging aid: pages that were given back, or went to another request, since the last step are
        # filled with NaN before the step runs, so that a read of memory that its request does not own shows
        self.poison_freed = bool(poison_freed)
        self._owners: Optional[List[List[int]]] = None
        # captured steps: for steps of single tokens by batch size and key parts: (graph, its logits tensor)
        self.use_graphs = bool(use_graphs) and self.model.graph_safe
        self.tensors: Dict[str, torch.Tensor] = tensors      # by the names that files use (views of the load's one allocation)
        self._graphs: Dict[tuple, Any] = {}        # (batch size, key parts) -> (graph, its logits)
        self._seen: Dict[tuple, int] = {}
        self.graph_replays: Dict[tuple, int] = {}  # how often each was replayed
        self._step_graphs: Dict[tuple, Any] = {}   # the same for steps that are not all single tokens, by their sizes
        self.step_graph_replays: Dict[tuple, int] = {}
        self._last_use: Dict[tuple, int] = {}
        self._clock = 0
        self.last_run_was_replay = False

    # ------------------------------------------------------------ construction helpers
    @classmethod
    def from_folder(cls, folder: str, dtype="bfloat16", device="cuda:0", one_piece: bool = True, **kw) -> "ModelRunner":
        """The model of a folder (config.json picks the architecture; model.safetensors).  ``one_piece``: the
        engine's memory is asked of the driver in one allocation (reserve_in_one_piece)."""
        from .. import models  # noqa: F401  (registers the architectures)
        device = require_gpu(device)
        arch, cfg = load_config(folder)
        spec = arch.build_spec(cfg)
        files = open_safetensors(folder)
        model = DecoderModel(spec)
        if one_piece:
            reserve_in_one_piece(device, engine_bytes(spec, model.tensors(), DTYPES[dtype], device, int(kw.get("page_size", 16)),
                                                      kw.get("max_tokens"), kw.get("num_pages"), int(kw.get("max_seqs", 8)),
                                                      int(kw.get("max_batch_tokens", 2048)), float(kw.get("kv_fraction", 0.85))))
        tensors = load_weights(files, model.tensors(), DTYPES[dtype], device, groups=model.fused_groups(DTYPES[dtype], device),
                               log=lambda line: print(f"[llama.cu_amd] {line}", file=sys.stderr, flush=True),
                               ignored=arch.ignored_tensors)
        runner = cls(spec, tensors, dtype, device, **kw)
        runner.config = cfg
        runner.tensors = tensors
        return runner

    @classmethod
    def from_config(cls, cfg, seed: int, dtype="bfloat16", device="cuda:0", std: float = 0.02, stored=None,
                    one_piece: bool = True, **kw) -> "ModelRunner":
        """Random weights made on the device from ``seed`` (nothing is written or read): bit for
        bit the weights that ``write_random_model`` writes for the same seed.  ``stored``: the
        type that a file would hold them in, if not the compute type (``"bfloat16"`` with the
        float32 compute type gives the float32 engine weights that bfloat16 holds exactly)."""
        from .. import models  # noqa: F401
        from ..config import architecture_of
        device = require_gpu(device)
        spec = architecture_of(cfg.to_dict()).build_spec(cfg)
        expected = DecoderModel(spec).tensors()
        if one_piece:
            reserve_in_one_piece(device, engine_bytes(spec, expected, DTYPES[dtype], device, int(kw.get("page_size", 16)),
                                                      kw.get("max_tokens"), kw.get("num_pages"), int(kw.get("max_seqs", 8)),
                                                      int(kw.get("max_batch_tokens", 2048)), float(kw.get("kv_fraction", 0.85))))
        tensors = random_tensors(expected, seed, dtype=DTYPES[stored or dtype], std=std, device=device)
        tensors = {n: convert(t, expected[n], DTYPES[dtype]) for n, t in tensors.items()}
        runner = cls(spec, tensors, dtype, device, **kw)
        runner.config = cfg
        runner.tensors = tensors
        return runner

    def export_weights(self) -> Dict[str, torch.Tensor]:
        """The weights as the engine holds them, under the names that files use, copied to the host (for a
        plain model in a test, or to write a folder with ``weights.write_safetensors``)."""
        return {name: t.detach().to("cpu") for name, t in self.tensors.items()}

    # ------------------------------------------------------------ the step function
    def prepare(self, req_ids: Sequence[int], tokens: Sequence[Sequence[int]], want: Sequence[Sequence[int]],
                feed: Sequence[tuple] = ()) -> StepContext:
        """Give the requests their pages (new requests get a slot) and build the batch."""
        added = []
        reserved = []
        try:
            for rid, toks in zip(req_ids, tokens):
                if not self.cache.has(rid):
                    self.cache.add(rid)
                    added.append(rid)
                new_len = self.cache.length(rid) + len(toks)
                if new_len > self.max_model_len:
                    raise ValueError(f"request {rid}: {new_len} tokens exceed the context limit {self.max_model_len}")
                if not self.cache.reserve(rid, new_len):
                    raise OutOfPages(f"request {rid}: no free pages for {len(toks)} more tokens "
                                     f"({self.cache.free_pages(0)} pages free)")
                reserved.append(rid)
        except Exception:
            for rid in reserved:                       # give back what this call took
                if rid not in added:
                    self.cache.truncate(rid, self.cache.length(rid))
            for rid in added:
                self.cache.release(rid)
            raise
        if self.poison_freed:
            self._poison_pages_that_changed_hands()
        step = self.builder.build(req_ids, tokens, want, self.spec.vocab_size, feed, upload=False)
        self.model.prepare(step)                   # what the parts derive from the batch on the host joins the step's arrays
        self.builder.upload()
        return step

    def _poison_pages_that_changed_hands(self) -> None:
        """Called when a step's pages are reserved and nothing of it has run: every page that a request
        held at the last call and that is free now, or another request's (who has written nothing to it
        yet), is filled with NaN."""
        now = [self.cache.page_owners(g) for g in range(len(self.groups))]
        before, self._owners = self._owners, now
        if before is None:
            return
        for g in range(len(self.groups)):
            gone = [p for p, (a, b) in enumerate(zip(before[g], now[g])) if a >= 0 and a != b]
            if not gone:
                continue
            index = torch.tensor(gone, dtype=torch.long, device=self.device)
            for c in self.caches:
                if c.group == g and c.writes and c.pages is not None:
                    c.pages.index_fill_(0, index, float("nan"))

    GRAPH_AFTER = 2          # a kind of step is captured when it comes for the third time
    GRAPH_MAX_BATCH = 256
    GRAPH_MAX_TOKENS = 256   # steps that are not all single tokens are captured up to this many tokens (beyond, the
                             # GPU's step takes far longer than the host's launches, and a graph would hold much memory)
    GRAPH_MAX_KINDS = 64     # so many kinds of such steps are kept; the one replayed longest ago goes first
    SEEN_MAX_KINDS = 4096    # so many kinds of steps are counted on their way to a graph

    def run(self, step: StepContext) -> torch.Tensor:
        """The model on the batch.  Small steps are launch-bound (a step of the model is some two hundred to
        four hundred launches), so they are captured into HIP graphs and replayed: the batch arrays, and what
        the parts derive from them on the host (``Part.prepare``), live at fixed device addresses, so a replay
        reads the new step's tokens, positions, block tables and task lists.  A graph fits every step with the same
        sizes: for steps in which every request decodes one token the number of requests and the number of parts
        into which the decode attention cuts the keys; for any other step (a prompt portion beside decoding
        requests, say) the numbers of tokens, requests, single tokens and wanted rows, and what the parts' plans
        say fixes their launches (``signature``).  (The reference captures everything between two attentions per
        token-count bucket, llama.cu/src/exec/step.rs:82-96; here the whole step is one graph.)"""
        b = step.n_req
        self.last_run_was_replay = False
        if not self.use_graphs:
            return self.model.forward(step, self.caches)
        if step.decode_only:
            if not (step.n_logits == b and b <= self.GRAPH_MAX_BATCH):
                return self.model.forward(step, self.caches)
            # the number of key parts of the decode attention must not change between replays: a
            # graph is made for a batch size and a number of parts (which follows the longest
            # context rounded up to a power of two, so it changes rarely)
            step.attn_splits = self._decode_splits(b, step.max_ctx_len)
            return self._run_captured(self._graphs, (b, step.attn_splits), step, self.graph_replays)
        if step.n > self.GRAPH_MAX_TOKENS:
            return self.model.forward(step, self.caches)
        plans = tuple(sorted((k, v.signature) for k, v in step.scratch.items() if hasattr(v, "signature")))
        key = (step.n, b, step.n_logits, step.logits_all, plans)
        logits = self._run_captured(self._step_graphs, key, step, self.step_graph_replays)
        if len(self._step_graphs) > self.GRAPH_MAX_KINDS:
            oldest = min((k for k in self._step_graphs if k != key), key=lambda k: self._last_use.get(k, 0))
            del self._step_graphs[oldest]
            self._last_use.pop(oldest, None)
            self._seen.pop(oldest, None)                 # (it is counted anew if it comes again)
        return logits

    def _run_captured(self, graphs: Dict[tuple, Any], key: tuple, step: StepContext, replays: Dict[tuple, int]) -> torch.Tensor:
        """Replay the graph of ``key`` (capture it first if the key has come often enough; before that, run eagerly)."""
        self._clock += 1
        self._last_use[key] = self._clock
        entry = graphs.get(key)
        if entry is None:
            if len(self._seen) > self.SEEN_MAX_KINDS:    # a long-lived engine meets ever new kinds of steps: the counts of
                self._seen.clear()                       # those that never came a third time are not kept for ever
                self._last_use = {k: v for k, v in self._last_use.items() if k in self._graphs or k in self._step_graphs}
            self._seen[key] = self._seen.get(key, 0) + 1
            if self._seen[key] <= self.GRAPH_AFTER:
                return self.model.forward(step, self.caches)
            torch.cuda.synchronize(self.device)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                logits = self.model.forward(step, self.caches)
            entry = graphs[key] = (graph, logits)
        graph, logits = entry
        graph.replay()
        self.last_run_was_replay = True
        replays[key] = replays.get(key, 0) + 1
        return logits

    def _decode_splits(self, batch: int, max_ctx_len: int) -> int:
        """Into how many parts the layers' mixers want a decoding request's keys cut (the most any of
        them asks for; a mixer without keys asks for nothing)."""
        best = 1
        for layer in self.model.layers:
            best = max(best, int(layer.decode_splits(batch, max_ctx_len)))
        return best

    def step(self, req_ids: Sequence[int], tokens: Sequence[Sequence[int]],
             want: Optional[Sequence[Sequence[int]]] = None) -> torch.Tensor:
        """Run one batch: request ``req_ids[i]`` feeds ``tokens[i]`` (its next tokens, after
        what earlier steps fed).  Returns float32 logits ``[wanted, vocab]`` on the device, in
        the order of the requests and of ``want[i]`` (places among ``tokens[i]``; default: the
        last token of each request)."""
        if want is None:
            want = [[len(t) - 1] for t in tokens]
        ctx = self.prepare(req_ids, tokens, want)
        logits = self.run(ctx)
        for rid in req_ids:
            self.cache.commit(rid)
        return logits

    def end(self, req_id: int) -> None:
        """The request is finished: its pages and slot are given back."""
        if self.cache.has(req_id):
            self.cache.release(req_id)
