"""The scheduler as Python sees it (the decisions are made in csrc/host/sched.cpp)."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import List, Sequence

from ..cache import CacheManager
from ..cache.manager import CacheError, _ints, _lib

REASONS = {0: None, 1: "eos", 2: "max_steps", 3: "length", 4: "aborted"}


@dataclass(frozen=True)
class PlanEntry:
    req: int
    start: int          # index of the portion's first token among the request's tokens
    count: int
    want_logits: bool   # the portion reaches the request's last known token


@dataclass(frozen=True)
class RequestInfo:
    n_tokens: int
    prompt_len: int
    computed: int
    generated: int
    reason: object
    preemptions: int


class Scheduler:
    def __init__(self, cache: CacheManager, max_num_seqs: int, max_batch_tokens: int, prefill_chunk: int,
                 max_model_len: int):
        self.cache = cache                      # kept alive: the C++ scheduler points into it
        self._lib = _lib()
        self._h = ctypes.c_void_p(self._lib.lcu_sched_create(cache._h, int(max_num_seqs), int(max_batch_tokens),
                                                             int(prefill_chunk), int(max_model_len)))
        if not self._h:
            raise CacheError("scheduler: bad configuration (all limits must be positive)")
        self._cap = max(int(max_num_seqs), 1) + 8

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.lcu_sched_destroy(h)

    def _st(self, st: int, what: str) -> None:
        if st:
            CacheManager._raise(st, what)

    def add(self, req: int, tokens: Sequence[int], max_new: int, keep: bool = False) -> None:
        self._st(self._lib.lcu_sched_add(self._h, ctypes.c_longlong(req), _ints(list(tokens)), len(tokens), int(max_new),
                                         int(keep)), f"add request {req}")

    def extend(self, req: int, tokens: Sequence[int], max_new: int) -> None:
        self._st(self._lib.lcu_sched_extend(self._h, ctypes.c_longlong(req), _ints(list(tokens)), len(tokens),
                                            int(max_new)), f"extend request {req}")

    def abort(self, req: int) -> None:
        self._st(self._lib.lcu_sched_abort(self._h, ctypes.c_longlong(req)), f"abort request {req}")

    def drop(self, req: int) -> None:
        self._st(self._lib.lcu_sched_drop(self._h, ctypes.c_longlong(req)), f"drop request {req}")

    def plan(self) -> List[PlanEntry]:
        """Decide the next step (pages for it are reserved)."""
        cap = self._cap
        ids = (ctypes.c_longlong * cap)()
        start, count, want = (ctypes.c_int * cap)(), (ctypes.c_int * cap)(), (ctypes.c_int * cap)()
        n = self._lib.lcu_sched_plan(self._h, ids, start, count, want, cap)
        if n < 0:
            raise CacheError("scheduler: plan larger than expected")
        return [PlanEntry(ids[i], start[i], count[i], bool(want[i])) for i in range(n)]

    def commit(self) -> None:
        """The planned step ran."""
        self._lib.lcu_sched_commit(self._h)

    def append(self, req: int, token: int, is_eos: bool):
        """A sampled token; returns the finish reason or None."""
        r = self._lib.lcu_sched_append(self._h, ctypes.c_longlong(req), int(token), int(bool(is_eos)))
        if r < 0:
            self._st(r, f"append to request {req}")
        return REASONS[r]

    def set_token(self, req: int, index: int, token: int) -> None:
        """The value of a token that was appended before it was known."""
        self._st(self._lib.lcu_sched_set_token(self._h, ctypes.c_longlong(req), int(index), int(token)),
                 f"set token {index} of request {req}")

    def finish(self, req: int, reason: str, n_tokens: int = -1):
        """End a request from outside, its tokens cut to ``n_tokens`` (an end of sequence
        learned after more was appended); returns the reason it now has."""
        code = {v: k for k, v in REASONS.items()}[reason]
        r = self._lib.lcu_sched_finish(self._h, ctypes.c_longlong(req), code, int(n_tokens))
        if r < 0:
            self._st(r, f"finish request {req}")
        return REASONS[r]

    def take_finished(self) -> List[int]:
        buf = (ctypes.c_longlong * 1024)()
        n = self._lib.lcu_sched_take_finished(self._h, buf, 1024)
        return list(buf[:n])

    def info(self, req: int) -> RequestInfo:
        out = (ctypes.c_int * 6)()
        self._st(self._lib.lcu_sched_info(self._h, ctypes.c_longlong(req), out), f"request {req}")
        return RequestInfo(out[0], out[1], out[2], out[3], REASONS[out[4]], out[5])

    def tokens(self, req: int) -> List[int]:
        n = self.info(req).n_tokens
        buf = (ctypes.c_int * max(n, 1))()
        self._lib.lcu_sched_tokens(self._h, ctypes.c_longlong(req), buf, n)
        return list(buf[:n])

    @property
    def n_waiting(self) -> int:
        return self._lib.lcu_sched_n_waiting(self._h)

    @property
    def n_running(self) -> int:
        return self._lib.lcu_sched_n_running(self._h)

    @property
    def idle(self) -> bool:
        return self.n_waiting == 0 and self.n_running == 0

    @property
    def preemptions(self) -> int:
        return self._lib.lcu_sched_preemptions(self._h)
