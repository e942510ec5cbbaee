"""The cache manager as Python sees it: a thin layer over the C++ manager
(csrc/host/cache.cpp), plus the device memory that the pages and state slots are.

Pages are handed out per *group*: layers whose caches grow and shrink alike (all keys;
or a window of them) share one pool of page ids and one block table per request, and
each such layer has a tensor of its own that those ids index.  State of fixed size per
request lives in slots; a request holds one slot index for all layers that keep state.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import List, Sequence

from ..kernels import build


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    """Not enough free pages (or state slots) for what was asked."""


@dataclass(frozen=True)
class CacheGroup:
    num_pages: int
    page_size: int
    window: int = 0      # 0: all tokens are kept
    slack: int = 0       # a window gives a page back only when a request cut back by up to this many tokens would not
                         # see it either (1 for an engine that runs one round ahead of its sampler's results)


_STATUS = {1: "not enough free pages", 2: "no free state slot", -1: "unknown request", -2: "request exists already",
           -3: "bad argument", -4: "a window has already given back pages below that length",
           -5: "the manager's tables are corrupt",
           -6: "the model keeps per-request state that cannot be cut back"}

_configured = False


def _lib() -> ctypes.CDLL:
    global _configured
    lib = build.load(build.HOST_LIBRARY)
    if not _configured:
        lib.lcu_cache_create.restype = ctypes.c_void_p
        lib.lcu_sched_create.restype = ctypes.c_void_p
        lib.lcu_sched_preemptions.restype = ctypes.c_longlong
        _configured = True
    return lib


def _ints(values: Sequence[int]):
    return (ctypes.c_int * len(values))(*values)


class CacheManager:
    def __init__(self, groups: Sequence[CacheGroup], n_slots: int, can_truncate: bool = True):
        """``can_truncate``: whether the state of fixed size that the model keeps for a request (if any) can be
        cut back to a shorter length; if not, ``truncate`` to less than a request holds raises, and
        ``truncate_or_reset`` sets the request to length 0 with its pages kept."""
        self.groups = list(groups)
        self.can_truncate = bool(can_truncate)
        self.n_slots = int(n_slots)
        self._lib = _lib()
        self._h = ctypes.c_void_p(self._lib.lcu_cache_create(
            len(self.groups), _ints([g.num_pages for g in self.groups]), _ints([g.page_size for g in self.groups]),
            _ints([g.window for g in self.groups]), _ints([g.slack for g in self.groups]), self.n_slots,
            int(self.can_truncate)))
        if not self._h:
            raise CacheError("cache manager: bad group description")

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.lcu_cache_destroy(h)

    @staticmethod
    def _raise(st: int, what: str):
        if st in (1, 2):
            raise OutOfPages(f"{what}: {_STATUS[st]}")
        raise CacheError(f"{what}: {_STATUS.get(st, st)}")

    def add(self, req: int) -> None:
        st = self._lib.lcu_cache_add(self._h, ctypes.c_longlong(req))
        if st:
            self._raise(st, f"add request {req}")

    def has(self, req: int) -> bool:
        return bool(self._lib.lcu_cache_has(self._h, ctypes.c_longlong(req)))

    def reserve(self, req: int, new_len: int) -> bool:
        """Pages for the request's tokens up to ``new_len`` in every group, all or nothing.
        False (and nothing changed) if the free pages do not suffice."""
        st = self._lib.lcu_cache_reserve(self._h, ctypes.c_longlong(req), int(new_len))
        if st == 1:
            return False
        if st:
            self._raise(st, f"reserve {new_len} tokens for request {req}")
        return True

    def commit(self, req: int) -> None:
        st = self._lib.lcu_cache_commit(self._h, ctypes.c_longlong(req))
        if st:
            self._raise(st, f"commit request {req}")

    def truncate(self, req: int, new_len: int) -> None:
        st = self._lib.lcu_cache_truncate(self._h, ctypes.c_longlong(req), int(new_len))
        if st:
            self._raise(st, f"truncate request {req} to {new_len}")

    def truncate_or_reset(self, req: int, new_len: int) -> bool:
        """``truncate`` where everything the request holds can be cut back (True).  Where something cannot (a state
        of fixed size, a window that has given back a page the shorter request would see), only that is given up:
        the request's length becomes 0, groups without a window keep their pages up to ``new_len``, and the request
        is to be computed again from its first token (False)."""
        st = self._lib.lcu_cache_truncate_or_reset(self._h, ctypes.c_longlong(req), int(new_len))
        if st not in (0, 3):
            self._raise(st, f"cut request {req} back to {new_len}")
        return st == 0

    def release(self, req: int) -> None:
        st = self._lib.lcu_cache_release(self._h, ctypes.c_longlong(req))
        if st:
            self._raise(st, f"release request {req}")

    def length(self, req: int) -> int:
        return self._lib.lcu_cache_len(self._h, ctypes.c_longlong(req))

    def reserved(self, req: int) -> int:
        return self._lib.lcu_cache_reserved(self._h, ctypes.c_longlong(req))

    def slot(self, req: int) -> int:
        return self._lib.lcu_cache_slot(self._h, ctypes.c_longlong(req))

    def free_pages(self, group: int = 0) -> int:
        return self._lib.lcu_cache_free_pages(self._h, group)

    def free_slots(self) -> int:
        return self._lib.lcu_cache_free_slots(self._h)

    def live_requests(self) -> int:
        return self._lib.lcu_cache_live(self._h)

    def table(self, req: int, group: int = 0) -> List[int]:
        """The request's block table in ``group``: physical page per logical page, -1 for a
        page that a window has passed and given back."""
        cap = 64
        while True:
            buf = (ctypes.c_int * cap)()
            n = self._lib.lcu_cache_table(self._h, ctypes.c_longlong(req), group, buf, cap)
            if n < 0:
                raise CacheError(f"table of request {req}: unknown request or group")
            if n <= cap:
                return list(buf[:n])
            cap = n

    def page_owners(self, group: int = 0) -> List[int]:
        """For every page of ``group`` the request that holds it, -1 for a free page."""
        n = self.groups[group].num_pages
        buf = (ctypes.c_longlong * max(n, 1))()
        if self._lib.lcu_cache_page_owners(self._h, group, buf, n) != n:
            raise CacheError(f"page owners of group {group}: unknown group")
        return list(buf[:n])

    def check(self) -> None:
        """Raise if a page or slot is lost, held twice, or both free and held."""
        why = ctypes.create_string_buffer(256)
        st = self._lib.lcu_cache_check(self._h, why, 256)
        if st:
            raise CacheError(f"cache manager invariant broken: {why.value.decode()}")

    def fill_batch(self, reqs: Sequence[int], n_new: Sequence[int], positions, req_of_token, q_start, ctx_len,
                   state_slot, block_tables, max_pages: Sequence[int], slots) -> None:
        """Write the batch arrays (addresses of int32 host buffers) for the requests ``reqs``
        feeding ``n_new[i]`` tokens each; their pages must be reserved."""
        n = len(reqs)
        ids = (ctypes.c_longlong * n)(*reqs)
        bt = (ctypes.c_void_p * len(self.groups))(*block_tables)
        sl = (ctypes.c_void_p * len(self.groups))(*slots)
        st = self._lib.lcu_cache_fill_batch(self._h, n, ids, _ints(list(n_new)), ctypes.c_void_p(positions),
                                            ctypes.c_void_p(req_of_token), ctypes.c_void_p(q_start),
                                            ctypes.c_void_p(ctx_len), ctypes.c_void_p(state_slot), bt,
                                            _ints(list(max_pages)), sl)
        if st:
            self._raise(st, "fill batch")
