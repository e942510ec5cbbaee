"""The engine: requests in, tokens out.  A scheduler round is: plan the step, run it
through the runner's step function, sample where a request's known tokens end, hand
the tokens back to the scheduler, report what finished.

The reference's loop (llama.cu/src/exec/engine.rs:217-295) runs ahead of its caller and
learns of an end-of-sequence token a round or two late (llama.cu/src/lib.rs:175-184).  So
does this one by default (``run_ahead``): a round's sampled ids stay on the device, the next
round is planned with placeholders for them and takes them from there
(llama.cu/src/op/fast_embedding.cuh:1-15), and the host reads a round's ids while the next
one runs, so the GPU does not wait for the host between rounds.  What a request computed
beyond an end-of-sequence token that was learned late is cut away again.  With
``run_ahead=False`` every round is sampled and read before the next is planned.
"""
from __future__ import annotations

import time
from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Sequence, Union

import torch

from ..kernels import ops
from ..sampling import GREEDY, Sampler, SamplingParams, token_logprobs
from .config import EngineConfig
from .runner import ModelRunner
from .scheduler import Scheduler


@dataclass
class StepOutput:
    req: int
    token: Optional[int]          # the sampled token (None if the request ended without one)
    finished: Optional[str]       # None, "eos", "max_steps", "length", "aborted"
    logprob: Optional[float] = None   # log of the probability the model gave the token (an engine made with ``logprobs``)


@dataclass
class _Request:
    tokens: List[int]
    params: SamplingParams
    prompt_len: int
    ignore_eos: bool = False
    draw_id: int = 0                  # what its random draws are keyed by beside the seed (default: its id)
    unknown: Optional[int] = None     # index of a token that is sampled but not read yet
    done: bool = False                # its end has been reported (or it was aborted)
    turn: int = 0                     # counts continuations: a row of an earlier turn is stale


@dataclass
class _Flight:
    """A launched round whose sampled ids the host has not read."""
    rows: List[int]                   # the request of each sampled row
    index: List[int]                  # where the id goes in that request's tokens
    reasons: List[Optional[str]]      # an end by count, known at launch
    turns: List[int]                  # the request's turn at launch
    owners: List["_Request"]          # and the request itself (an id may come again after a drop)
    sampled: torch.Tensor             # the ids on the device
    host: torch.Tensor                # and where the copy to the host lands
    copied: torch.cuda.Event
    host_logprobs: Optional[torch.Tensor] = None


class Engine:
    def __init__(self, runner: ModelRunner, prefill_chunk: Optional[int] = None, eos_token_ids: Sequence[int] = (),
                 run_ahead: bool = True, logprobs: bool = False):
        """``logprobs``: every sampled token comes with the logarithm of the probability that the model gave it
        (``StepOutput.logprob``; one more small kernel and copy a round)."""
        self.runner = runner
        self.run_ahead = bool(run_ahead)
        self.logprobs = bool(logprobs)
        self._flight: Optional[_Flight] = None
        self._awaiting: set = set()    # ended by count at launch, token not read yet
        self.sched = Scheduler(runner.cache, runner.max_seqs, runner.max_batch_tokens,
                               prefill_chunk or runner.max_batch_tokens, runner.max_model_len)
        self.sampler = Sampler()
        self.eos = set(eos_token_ids) or set(runner.spec.eos_token_ids)
        self.requests: Dict[int, _Request] = {}
        self._next_id = 0
        self.steps = 0
        # measurement (``timeline = []`` switches it on): per launched round the host's time from the plan to the
        # last launch, the round's tokens and requests, whether it was replayed from a graph, and two events on
        # the stream around its work (the gap between one round's last and the next one's first is a GPU that waits)
        self.timeline: Optional[List[dict]] = None

    @classmethod
    def from_folder(cls, folder: str, config: Optional[EngineConfig] = None, **fields) -> "Engine":
        """The engine for a model folder.  ``config``: the engine's constants (``EngineConfig``); ``fields``
        replace single ones (``dtype="float32", max_seqs=4, ...``)."""
        ec = EngineConfig.of(config, **fields)
        engine = cls(ModelRunner.from_folder(folder, **ec.runner_kwargs()), ec.prefill_chunk, run_ahead=ec.run_ahead,
                     logprobs=ec.logprobs)
        engine.config = ec
        return engine

    @classmethod
    def from_config(cls, cfg, seed: int, config: Optional[EngineConfig] = None, std: float = 0.02, stored=None,
                    **fields) -> "Engine":
        """The engine for a model configuration with random weights made on the device from ``seed`` (``std``,
        ``stored``: as in ``ModelRunner.from_config``)."""
        ec = EngineConfig.of(config, **fields)
        engine = cls(ModelRunner.from_config(cfg, seed, std=std, stored=stored, **ec.runner_kwargs()), ec.prefill_chunk,
                     run_ahead=ec.run_ahead, logprobs=ec.logprobs)
        engine.config = ec
        return engine

    def export_weights(self):
        """The model's weights by the names that files use, on the host (``ModelRunner.export_weights``)."""
        return self.runner.export_weights()

    # ---------------------------------------------------------------- requests
    def add_request(self, tokens: Sequence[int], params: SamplingParams = GREEDY, max_steps: int = 1000,
                    req_id: Optional[int] = None, keep: bool = False, ignore_eos: bool = False,
                    draw_id: Optional[int] = None) -> int:
        """A new request; ``max_steps`` is the number of tokens to generate, the first
        included (llama.cu/src/exec/engine_manager.rs:118-122).  A random draw is a function of
        (the parameters' seed, ``draw_id``, the index of the drawn token); ``draw_id`` is the
        request's id unless given."""
        tokens = [int(t) for t in tokens]
        if not tokens:
            raise ValueError("a request needs at least one prompt token")
        vocab = self.runner.spec.vocab_size
        bad = [t for t in tokens if not 0 <= t < vocab]
        if bad:
            raise ValueError(f"token id {bad[0]} is outside the vocabulary of {vocab}")
        rid = self._next_id if req_id is None else int(req_id)
        self._next_id = max(self._next_id, rid + 1)
        self.sched.add(rid, tokens, max_steps, keep)
        self.requests[rid] = _Request(tokens, params, len(tokens), ignore_eos, draw_id=rid if draw_id is None else int(draw_id))
        return rid

    def continue_request(self, rid: int, tokens: Sequence[int], max_steps: int = 1000) -> None:
        """A finished request that kept its cache goes on with more tokens (a chat's next
        turn: llama.cu/xtask/src/chat/mod.rs:54-71 starts the same session again)."""
        tokens = [int(t) for t in tokens]
        self.sched.extend(rid, tokens, max_steps)
        r = self.requests[rid]
        r.tokens.extend(tokens)
        r.prompt_len = len(r.tokens)
        r.done = False
        r.turn += 1

    def abort(self, rid: int) -> None:
        self.sched.abort(rid)
        r = self.requests.get(rid)
        if r is not None:
            r.done = True
        self._awaiting.discard(rid)

    def drop(self, rid: int) -> None:
        """Forget a finished request and give back a cache it kept."""
        self.sched.drop(rid)
        self.requests.pop(rid, None)
        self._awaiting.discard(rid)

    @property
    def idle(self) -> bool:
        return self.sched.idle and self._flight is None

    # ---------------------------------------------------------------- one round
    def step(self) -> List[StepOutput]:
        """Run one round; returns the tokens that became known and the requests that ended.
        Running ahead, these are the tokens of the round before the one launched here."""
        if not self.run_ahead:
            return self._step_in_turn()
        launched = self._launch()
        outputs = self._collect(self._flight) if self._flight is not None else []
        self._flight = launched
        reported = {o.req for o in outputs if o.finished}
        for rid in self.sched.take_finished():
            if rid not in reported and rid not in self._awaiting:
                outputs.append(StepOutput(rid, None, self.sched.info(rid).reason))
        return outputs

    def _launch(self) -> Optional[_Flight]:
        """Plan and launch a round; the ids it samples stay on the device, and the requests
        get placeholders for them."""
        t_plan = time.perf_counter()
        plan = self.sched.plan()
        if not plan:
            return None
        first = None
        if self.timeline is not None:
            first = torch.cuda.Event(enable_timing=True)
            first.record()
        before = self._flight
        row_of = {rid: i for i, rid in enumerate(before.rows)} if before is not None else {}
        ids, toks, want, feed = [], [], [], []
        for j, e in enumerate(plan):
            r = self.requests[e.req]
            have = self.runner.cache.length(e.req)
            if have != e.start:
                raise RuntimeError(f"request {e.req}: the cache holds {have} tokens, the plan starts at {e.start}")
            last = e.start + e.count - 1
            if r.unknown is not None and e.start <= r.unknown <= last:
                if r.unknown != last or e.req not in row_of:
                    raise RuntimeError(f"request {e.req}: token {r.unknown} is not known and the round before does not give it")
                feed.append((row_of[e.req], j))
            ids.append(e.req)
            toks.append(r.tokens[e.start:e.start + e.count])
            want.append([e.count - 1] if e.want_logits else [])
        step = self.runner.prepare(ids, toks, want, feed)
        if feed:
            ops.feed_tokens(step.tokens, before.sampled, step.feed_src, step.feed_dst)
        logits = self.runner.run(step)
        self.sched.commit()
        self.steps += 1
        rows = [e for e in plan if e.want_logits]
        if not rows:
            return None
        params = [self.requests[e.req].params for e in rows]
        keys = [(self.requests[e.req].draw_id, len(self.requests[e.req].tokens)) for e in rows]
        sampled = self.sampler.sample_device(logits, params, keys)
        host = torch.empty(len(rows), dtype=torch.int32, pin_memory=True)
        host.copy_(sampled, non_blocking=True)
        host_lp = None
        if self.logprobs:
            host_lp = torch.empty(len(rows), dtype=torch.float32, pin_memory=True)
            host_lp.copy_(token_logprobs(logits, sampled), non_blocking=True)
        copied = torch.cuda.Event()
        copied.record()
        if first is not None:
            last = torch.cuda.Event(enable_timing=True)
            last.record()
            self.timeline.append({"host_ms": (time.perf_counter() - t_plan) * 1e3, "tokens": step.n, "requests": step.n_req,
                                  "graph": self.runner.last_run_was_replay, "first": first, "last": last})
        flight = _Flight([e.req for e in rows], [], [], [], [], sampled, host, copied, host_lp)
        for e in rows:
            r = self.requests[e.req]
            r.unknown = len(r.tokens)
            flight.index.append(r.unknown)
            flight.turns.append(r.turn)
            flight.owners.append(r)
            r.tokens.append(0)
            reason = self.sched.append(e.req, 0, False)
            flight.reasons.append(reason)
            if reason:
                self._awaiting.add(e.req)
        return flight

    def _collect(self, flight: _Flight) -> List[StepOutput]:
        """Read a round's ids, put them where the placeholders stand, and end the requests that
        an end-of-sequence token ends."""
        flight.copied.synchronize()
        outputs: List[StepOutput] = []
        lps = flight.host_logprobs.tolist() if flight.host_logprobs is not None else [None] * len(flight.rows)
        for rid, index, reason, turn, owner, tok, lp in zip(flight.rows, flight.index, flight.reasons, flight.turns,
                                                            flight.owners, flight.host.tolist(), lps):
            r = self.requests.get(rid)
            if r is not owner or r.done or r.turn != turn:
                continue                                    # ended earlier; this row ran for nothing
            r.tokens[index] = tok
            if r.unknown == index:
                r.unknown = None
            self.sched.set_token(rid, index, tok)
            if tok in self.eos and not r.ignore_eos:
                reason = self.sched.finish(rid, "eos", index + 1)
                del r.tokens[index + 1:]
                r.unknown = None
            if reason:
                r.done = True
                self._awaiting.discard(rid)
            outputs.append(StepOutput(rid, tok, reason, lp))
        return outputs

    def _step_in_turn(self) -> List[StepOutput]:
        plan = self.sched.plan()
        outputs: List[StepOutput] = []
        if plan:
            ids = [e.req for e in plan]
            toks = [self.requests[e.req].tokens[e.start:e.start + e.count] for e in plan]
            want = [[e.count - 1] if e.want_logits else [] for e in plan]
            for e in plan:
                have = self.runner.cache.length(e.req)
                if have != e.start:
                    raise RuntimeError(f"request {e.req}: the cache holds {have} tokens, the plan starts at {e.start}")
            logits = self.runner.run(self.runner.prepare(ids, toks, want))
            self.sched.commit()
            self.steps += 1
            rows = [e for e in plan if e.want_logits]
            if rows:
                params = [self.requests[e.req].params for e in rows]
                keys = [(self.requests[e.req].draw_id, len(self.requests[e.req].tokens)) for e in rows]
                sampled = self.sampler.sample(logits, params, keys)
                lps = [None] * len(sampled)
                if self.logprobs:
                    lps = token_logprobs(logits, ops.to_device(sampled, torch.int32, logits.device)).tolist()
                for e, tok, lp in zip(rows, sampled, lps):
                    r = self.requests[e.req]
                    r.tokens.append(tok)
                    reason = self.sched.append(e.req, tok, (tok in self.eos) and not r.ignore_eos)
                    outputs.append(StepOutput(e.req, tok, reason, lp))
        reported = {o.req for o in outputs if o.finished}
        for rid in self.sched.take_finished():
            if rid not in reported:
                outputs.append(StepOutput(rid, None, self.sched.info(rid).reason))
        return outputs

    # ---------------------------------------------------------------- whole generations
    def generate(self, prompts: Sequence[Sequence[int]], params: Union[SamplingParams, Sequence[SamplingParams]] = GREEDY,
                 max_steps: int = 1000, ignore_eos: bool = False,
                 on_token: Optional[Callable[[int, int], None]] = None) -> List[List[int]]:
        """Generate for every prompt (lists of token ids); returns the generated tokens of
        each, an end-of-sequence token included if one ended it.  The random draws of prompt ``i``
        are keyed by ``i``: the same call gives the same tokens however many requests the engine
        has served before.  If it raises, its requests are taken out of the engine again."""
        plist = [params] * len(prompts) if isinstance(params, SamplingParams) else list(params)
        if len(plist) != len(prompts):
            raise ValueError(f"{len(prompts)} prompts but {len(plist)} sets of sampling parameters")
        ids: List[int] = []
        try:
            for i, (p, sp) in enumerate(zip(prompts, plist)):
                ids.append(self.add_request(p, sp, max_steps, ignore_eos=ignore_eos, draw_id=i))
            out: Dict[int, List[int]] = {i: [] for i in ids}
            live = set(ids)
            while live:
                results = self.step()
                if not results and self.idle:
                    break
                for o in results:
                    if o.req not in out:
                        continue
                    if o.token is not None:
                        out[o.req].append(o.token)
                        if on_token:
                            on_token(ids.index(o.req), o.token)
                    if o.finished:
                        live.discard(o.req)
        except BaseException:
            # what this call put into the engine goes out again: the engine may serve other calls
            for i in ids:
                try:
                    self.abort(i)
                    self.drop(i)
                except Exception:
                    pass
            raise
        for i in ids:
            self.drop(i)
        return [out[i] for i in ids]
