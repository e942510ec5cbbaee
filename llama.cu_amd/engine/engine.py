"""The engine: requests in, tokens out.  A scheduler round is: plan the step, run it
through the runner's step function, sample where a request's known tokens end, hand
the tokens back to the scheduler, report what finished.

The reference's loop (llama.cu/src/exec/engine.rs:217-295) runs ahead of its caller and
learns of an end-of-sequence token a round or two late (llama.cu/src/lib.rs:175-184); this
one samples and checks for the end before it plans the next round.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence, Tuple, Union

import torch

from ..sampling import GREEDY, Sampler, SamplingParams
from .runner import ModelRunner
from .scheduler import PlanEntry, Scheduler


@dataclass
class StepOutput:
    req: int
    token: Optional[int]          # the sampled token (None if the request ended without one)
    finished: Optional[str]       # None, "eos", "max_steps", "length", "aborted"


@dataclass
class _Request:
    tokens: List[int]
    params: SamplingParams
    prompt_len: int
    ignore_eos: bool = False


class Engine:
    def __init__(self, runner: ModelRunner, prefill_chunk: Optional[int] = None, eos_token_ids: Sequence[int] = ()):
        self.runner = runner
        self.sched = Scheduler(runner.cache, runner.max_seqs, runner.max_batch_tokens,
                               prefill_chunk or runner.max_batch_tokens, runner.max_model_len)
        self.sampler = Sampler()
        self.eos = set(eos_token_ids) or set(runner.spec.eos_token_ids)
        self.requests: Dict[int, _Request] = {}
        self._next_id = 0
        self.steps = 0

    @classmethod
    def from_folder(cls, folder: str, dtype: str = "bfloat16", device: str = "cuda:0",
                    prefill_chunk: Optional[int] = None, **runner_kw) -> "Engine":
        return cls(ModelRunner.from_folder(folder, dtype=dtype, device=device, **runner_kw), prefill_chunk)

    @classmethod
    def from_config(cls, cfg, seed: int, dtype: str = "bfloat16", device: str = "cuda:0",
                    prefill_chunk: Optional[int] = None, **runner_kw) -> "Engine":
        return cls(ModelRunner.from_config(cfg, seed, dtype=dtype, device=device, **runner_kw), prefill_chunk)

    # ---------------------------------------------------------------- requests
    def add_request(self, tokens: Sequence[int], params: SamplingParams = GREEDY, max_steps: int = 1000,
                    req_id: Optional[int] = None, keep: bool = False, ignore_eos: bool = False) -> int:
        """A new request; ``max_steps`` is the number of tokens to generate, the first
        included (llama.cu/src/exec/engine_manager.rs:118-122)."""
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
        self.requests[rid] = _Request(tokens, params, len(tokens), ignore_eos)
        return rid

    def continue_request(self, rid: int, tokens: Sequence[int], max_steps: int = 1000) -> None:
        """A finished request that kept its cache goes on with more tokens (a chat's next
        turn: llama.cu/xtask/src/chat/mod.rs:54-71 starts the same session again)."""
        tokens = [int(t) for t in tokens]
        self.sched.extend(rid, tokens, max_steps)
        r = self.requests[rid]
        r.tokens.extend(tokens)
        r.prompt_len = len(r.tokens)

    def abort(self, rid: int) -> None:
        self.sched.abort(rid)

    def drop(self, rid: int) -> None:
        """Forget a finished request and give back a cache it kept."""
        self.sched.drop(rid)
        self.requests.pop(rid, None)

    @property
    def idle(self) -> bool:
        return self.sched.idle

    # ---------------------------------------------------------------- one round
    def step(self) -> List[StepOutput]:
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
                keys = [(e.req, len(self.requests[e.req].tokens)) for e in rows]
                sampled = self.sampler.sample(logits, params, keys)
                for e, tok in zip(rows, sampled):
                    r = self.requests[e.req]
                    r.tokens.append(tok)
                    reason = self.sched.append(e.req, tok, (tok in self.eos) and not r.ignore_eos)
                    outputs.append(StepOutput(e.req, tok, reason))
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
        each, an end-of-sequence token included if one ended it."""
        plist = [params] * len(prompts) if isinstance(params, SamplingParams) else list(params)
        ids = [self.add_request(p, sp, max_steps, ignore_eos=ignore_eos) for p, sp in zip(prompts, plist)]
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
        for i in ids:
            self.drop(i)
        return [out[i] for i in ids]
