"""The cache manager on the CPU: pages in groups, block tables, windows, state slots.
No page is lost, held twice or freed twice, under random orders of requests."""
import random

import pytest
import torch

import llama_cu_amd
from llama_cu_amd.cache import CacheError, CacheGroup, CacheManager, OutOfPages


def test_pages_follow_the_length():
    m = CacheManager([CacheGroup(10, 16)], 4)
    m.add(1)
    assert m.reserve(1, 1) and m.table(1) == [0]
    assert m.reserve(1, 16) and len(m.table(1)) == 1
    assert m.reserve(1, 17) and len(m.table(1)) == 2
    assert m.free_pages() == 8 and m.length(1) == 0 and m.reserved(1) == 17
    m.commit(1)
    assert m.length(1) == 17
    m.check()


def test_reserve_is_all_or_nothing():
    m = CacheManager([CacheGroup(4, 16), CacheGroup(2, 16)], 4)
    m.add(1)
    assert m.reserve(1, 32)
    assert not m.reserve(1, 33)            # the second group has no third page
    assert m.free_pages(0) == 2 and m.free_pages(1) == 0 and m.reserved(1) == 32
    m.check()


def test_release_gives_everything_back_and_pages_are_used_again():
    m = CacheManager([CacheGroup(4, 16)], 2)
    m.add(1); m.reserve(1, 40); m.commit(1)
    first = m.table(1)
    m.add(2); assert not m.reserve(2, 33)
    m.release(1)
    assert m.free_pages() == 4 and m.free_slots() == 1
    assert m.reserve(2, 33)
    assert set(m.table(2)) <= set(first)                 # the same pages again
    assert m.table(2)[0] == first[-1]                    # the one given back last is taken first
    with pytest.raises(CacheError):
        m.release(1)                                     # freed twice
    m.check()


def test_truncate_gives_tail_pages_back():
    """The reference shrinks a cache when its owner rolls ``pos`` back
    (llama.cu/src/exec/kv_cache.rs:34-50, llama.cu/xtask/src/service/cache_manager.rs:40-42)."""
    m = CacheManager([CacheGroup(8, 16)], 2)
    m.add(1); m.reserve(1, 100); m.commit(1)
    assert m.free_pages() == 1
    m.truncate(1, 33)
    assert m.length(1) == 33 and len(m.table(1)) == 3 and m.free_pages() == 5
    with pytest.raises(CacheError):
        m.truncate(1, 50)
    m.check()


def test_window_gives_passed_pages_back():
    m = CacheManager([CacheGroup(16, 16, window=0), CacheGroup(4, 16, window=20)], 2)
    m.add(1)
    used = []
    for new_len in range(1, 200):
        assert m.reserve(1, new_len), new_len            # 4 pages suffice for a window of 20 for ever
        m.commit(1)
        t = m.table(1, 1)
        # the next query, at position new_len, sees keys new_len - 19 .. new_len
        first_key = max(new_len - 19, 0)
        for p, page in enumerate(t):
            assert (page == -1) == (p < first_key // 16), (new_len, t)
        used.append(sum(1 for x in t if x >= 0))
        if new_len >= 160:
            break
    assert max(used) <= 3 and len(m.table(1, 0)) == 10 and all(x >= 0 for x in m.table(1, 0))
    with pytest.raises(CacheError, match="window"):
        m.truncate(1, 40)
    m.check()


def test_a_long_portion_in_a_windowed_group_holds_all_its_pages_for_the_step():
    m = CacheManager([CacheGroup(8, 16, window=20)], 2)
    m.add(1)
    assert m.reserve(1, 100)                              # every token of the portion is written and read in this step
    assert sum(1 for x in m.table(1) if x >= 0) == 7
    m.commit(1)
    assert sum(1 for x in m.table(1) if x >= 0) == 2       # then the window has passed the first five
    m.check()


def test_slots():
    m = CacheManager([CacheGroup(8, 16)], 2)
    m.add(10); m.add(11)
    assert {m.slot(10), m.slot(11)} == {0, 1}
    with pytest.raises(OutOfPages, match="slot"):
        m.add(12)
    with pytest.raises(CacheError, match="exists"):
        m.add(10)
    s = m.slot(10)
    m.release(10)
    m.add(12)
    assert m.slot(12) == s
    m.check()


def test_fill_batch_arrays():
    m = CacheManager([CacheGroup(8, 16), CacheGroup(8, 16, window=8)], 4)
    m.add(5); m.reserve(5, 30); m.commit(5)
    m.add(6)
    m.reserve(5, 31); m.reserve(6, 3)
    i32 = lambda n: torch.zeros(n, dtype=torch.int32)
    pos, rot, qs, ctx, slot = i32(4), i32(4), i32(3), i32(2), i32(2)
    bts = [torch.full((2, 3), -7, dtype=torch.int32) for _ in range(2)]
    sls = [i32(4), i32(4)]
    m.fill_batch([5, 6], [1, 3], pos.data_ptr(), rot.data_ptr(), qs.data_ptr(), ctx.data_ptr(), slot.data_ptr(),
                 [b.data_ptr() for b in bts], [3, 3], [s.data_ptr() for s in sls])
    assert pos.tolist() == [30, 0, 1, 2] and rot.tolist() == [0, 1, 1, 1]
    assert qs.tolist() == [0, 1, 4] and ctx.tolist() == [31, 3] and slot.tolist() == [m.slot(5), m.slot(6)]
    for g in range(2):
        t5, t6 = m.table(5, g), m.table(6, g)
        assert bts[g][0].tolist() == [x if x >= 0 else 0 for x in t5] + [0] * (3 - len(t5))
        assert bts[g][1].tolist() == t6 + [0] * (3 - len(t6))
        assert sls[g].tolist() == [t5[1] * 16 + 14, t6[0] * 16, t6[0] * 16 + 1, t6[0] * 16 + 2]
    assert m.table(5, 1)[0] == -1                          # the window of 8 has passed the first page
    with pytest.raises(CacheError):                        # tokens that have no pages
        m.fill_batch([6], [40], pos.data_ptr(), rot.data_ptr(), qs.data_ptr(), ctx.data_ptr(), slot.data_ptr(),
                     [b.data_ptr() for b in bts], [3, 3], [s.data_ptr() for s in sls])


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_the_invariants(seed):
    """Requests come, grow, shrink and go in random order, in a pool that is often full:
    after every operation every page is free or held exactly once, and what the requests
    hold is what their lengths need."""
    rng = random.Random(seed)
    groups = [CacheGroup(24, 16, 0), CacheGroup(10, 8, window=rng.choice([5, 17, 40]))]
    m = CacheManager(groups, 5)
    live = {}
    next_id = 0
    for _ in range(600):
        op = rng.random()
        if op < 0.2 and m.free_slots():
            m.add(next_id); live[next_id] = 0; next_id += 1
        elif op < 0.7 and live:
            r = rng.choice(list(live))
            new_len = live[r] + rng.choice([1, 1, 1, 2, 7, 16, 33])
            before = [m.free_pages(g) for g in range(2)]
            if m.reserve(r, new_len):
                m.commit(r); live[r] = new_len
            else:
                assert [m.free_pages(g) for g in range(2)] == before     # nothing changed
        elif op < 0.8 and live:
            r = rng.choice(list(live))
            new_len = rng.randint(0, live[r])
            try:
                m.truncate(r, new_len); live[r] = new_len
            except CacheError as e:
                assert "window" in str(e)
        elif live:
            r = rng.choice(list(live))
            m.release(r); del live[r]
        m.check()
        for r, n in live.items():
            assert m.length(r) == n
            t0 = m.table(r, 0)
            assert len(t0) == (n + 15) // 16 and all(x >= 0 for x in t0)
            w = groups[1].window
            t1 = m.table(r, 1)
            for p, page in enumerate(t1):
                if p * 8 + 7 >= max(n - w + 1, 0) and p * 8 < n:
                    assert page >= 0, (r, n, t1)             # what the next query sees is there
        held = [sum(sum(1 for x in m.table(r, g) if x >= 0) for r in live) for g in range(2)]
        assert [held[g] + m.free_pages(g) for g in range(2)] == [24, 10]
    for r in list(live):
        m.release(r)
    assert m.free_pages(0) == 24 and m.free_pages(1) == 10 and m.free_slots() == 5


def test_a_cache_with_state_that_cannot_be_cut_back_refuses_to_truncate():
    m = CacheManager([CacheGroup(8, 16)], 2, can_truncate=False)
    m.add(1); m.reserve(1, 40); m.commit(1)
    m.reserve(1, 70)
    m.truncate(1, 40)                      # giving back what was reserved and not written is no cut
    assert m.length(1) == 40 and m.reserved(1) == 40 and m.free_pages() == 5
    with pytest.raises(CacheError, match="cannot be cut back"):
        m.truncate(1, 39)
    assert m.length(1) == 40
    m.check()


def test_a_request_that_cannot_be_cut_back_gives_up_only_what_cannot_be_cut():
    """``truncate_or_reset``: where a plain ``truncate`` works it is one; where the state of fixed size cannot be
    cut back the request's length becomes 0 with its pages kept; where a window has given back a page that the
    shorter request would see, that group's pages go back to the pool and the other group's stay."""
    m = CacheManager([CacheGroup(8, 16)], 2, can_truncate=True)
    m.add(1); m.reserve(1, 40); m.commit(1)
    assert m.truncate_or_reset(1, 30) and m.length(1) == 30 and len(m.table(1)) == 2
    m = CacheManager([CacheGroup(8, 16)], 2, can_truncate=False)
    m.add(1); m.reserve(1, 40); m.commit(1)
    assert not m.truncate_or_reset(1, 30)
    assert m.length(1) == 0 and m.reserved(1) == 30 and len(m.table(1)) == 2 and m.free_pages() == 6
    assert m.reserve(1, 30) and m.free_pages() == 6        # computing it again asks the pool for nothing
    m.commit(1)
    assert m.length(1) == 30
    m.check()
    m = CacheManager([CacheGroup(8, 16), CacheGroup(8, 16, window=20)], 2)
    m.add(1); m.reserve(1, 70); m.commit(1)
    assert m.table(1, 1)[:3] == [-1, -1, -1]
    assert not m.truncate_or_reset(1, 60)                  # the query at 60 would see keys from 41: page 2 is gone
    assert m.length(1) == 0 and m.reserved(1) == 0
    assert len(m.table(1, 0)) == 4 and m.table(1, 1) == [] and m.free_pages(1) == 8 and m.free_pages(0) == 4
    assert m.reserve(1, 60) and m.free_pages(0) == 4 and m.free_pages(1) == 4
    m.commit(1)
    m.check()
    m.release(1)
    assert m.free_pages(0) == 8 and m.free_pages(1) == 8 and m.free_slots() == 2


def test_a_windows_slack_keeps_what_a_request_cut_back_by_that_much_would_see():
    for slack in (0, 1, 5):
        m = CacheManager([CacheGroup(8, 4, window=6, slack=slack)], 2)
        m.add(1)
        for n in range(1, 60):
            assert m.reserve(1, n)
            m.commit(1)
            t = m.table(1)
            first_key = max(n - slack - 5, 0)              # what the query at n - slack sees first
            for p, page in enumerate(t):
                assert (page == -1) == (p < first_key // 4), (slack, n, t)
            # cutting back by up to the slack works at every length; by more, not at every length
            for cut in range(0, slack + 1):
                if n - cut >= 0:
                    probe = CacheManager([CacheGroup(8, 4, window=6, slack=slack)], 2)
                    probe.add(1)
                    for k in range(1, n + 1):
                        probe.reserve(1, k); probe.commit(1)
                    probe.truncate(1, n - cut)
                    probe.check()
        m.check()
