"""The scheduler's decisions on the CPU, with a step function that does nothing: admission,
portions under the token budget, decoding, finishing, and what happens when pages run out."""
import random

import pytest

import llama_cu_amd
from llama_cu_amd.cache import CacheGroup, CacheManager
from llama_cu_amd.engine.scheduler import Scheduler


def make(pages=64, page=16, slots=8, seqs=8, budget=64, chunk=32, max_len=512):
    cache = CacheManager([CacheGroup(pages, page)], slots)
    return cache, Scheduler(cache, seqs, budget, chunk, max_len)


def run_round(s, next_token=lambda req, n: 1000 + n, eos=None, check=None):
    """One round with a step function that does nothing; returns the plan and who finished."""
    plan = s.plan()
    s.commit()
    if check:
        check(plan)
    done = {}
    for e in plan:
        if e.want_logits:
            tok = next_token(e.req, s.info(e.req).n_tokens)
            r = s.append(e.req, tok, tok == eos)
            if r:
                done[e.req] = r
    for rid in s.take_finished():
        done.setdefault(rid, s.info(rid).reason)
    return plan, done


def test_prompts_are_cut_into_portions_under_the_budget_first_come_first_served():
    cache, s = make(budget=64, chunk=32)
    s.add(0, list(range(50)), 5)
    s.add(1, list(range(10)), 5)
    s.add(2, list(range(100)), 5)
    plan, _ = run_round(s)
    assert [(e.req, e.start, e.count, e.want_logits) for e in plan] == [(0, 0, 32, False), (1, 0, 10, True), (2, 0, 22, False)]
    plan, _ = run_round(s)
    # the decoding request first, then portions in admission order
    assert [(e.req, e.start, e.count, e.want_logits) for e in plan] == [(1, 10, 1, True), (0, 32, 18, True), (2, 22, 32, False)]
    assert sum(e.count for e in plan) <= 64
    plan, _ = run_round(s)
    assert [(e.req, e.count) for e in plan] == [(0, 1), (1, 1), (2, 32)]
    cache.check()


def test_a_portion_may_be_as_small_as_the_budget_leaves():
    cache, s = make(budget=8, chunk=32)
    s.add(0, list(range(7)), 3)
    s.add(1, list(range(30)), 3)
    plan, _ = run_round(s)
    assert [(e.req, e.count) for e in plan] == [(0, 7), (1, 1)]
    plan, _ = run_round(s)
    assert [(e.req, e.start, e.count) for e in plan] == [(0, 7, 1), (1, 1, 7)]


def test_max_steps_counts_every_generated_token_the_first_included():
    """llama.cu/src/exec/engine_manager.rs:118-122: the budget goes down in the prefill round too."""
    cache, s = make()
    s.add(0, [1, 2, 3], 3)
    reasons = []
    for _ in range(5):
        _, done = run_round(s)
        reasons.append(done.get(0))
        if s.idle:
            break
    assert reasons == [None, None, "max_steps"]
    assert s.info(0).generated == 3 and s.info(0).n_tokens == 6
    assert cache.live_requests() == 0 and cache.free_pages() == 64


def test_eos_and_abort_and_context_limit():
    cache, s = make(max_len=40)
    s.add(0, [1] * 5, 100)
    s.add(1, [1] * 5, 100)
    s.add(2, [1] * 38, 100)
    s.add(3, [1] * 41, 100)                       # longer than the context: ends without running
    _, done = run_round(s, next_token=lambda r, n: 7 if r == 0 else 1, eos=7)
    assert done[0] == "eos" and done[3] == "length"
    s.abort(1)
    assert 1 in s.take_finished() and s.info(1).reason == "aborted"
    done = {}
    for _ in range(2):                            # request 2: the rest of its prompt, then the 40th token fills the context
        assert not done
        _, done = run_round(s)
    assert done == {2: "length"} and s.info(2).n_tokens == 40 and s.info(2).generated == 2
    assert cache.live_requests() == 0
    cache.check()


def test_running_requests_are_bounded():
    cache, s = make(seqs=2, slots=8)
    for i in range(4):
        s.add(i, [1, 2, 3], 2)
    plan, _ = run_round(s)
    assert [e.req for e in plan] == [0, 1] and s.n_waiting == 2
    plan, done = run_round(s)
    assert [e.req for e in plan] == [0, 1] and set(done) == {0, 1}
    plan, _ = run_round(s)
    assert [e.req for e in plan] == [2, 3]
    # state slots bound them too
    cache, s = make(seqs=8, slots=1)
    s.add(0, [1, 2, 3], 2); s.add(1, [1, 2, 3], 2)
    plan, _ = run_round(s)
    assert [e.req for e in plan] == [0]


def test_out_of_pages_a_decoding_request_preempts_the_one_admitted_last():
    cache, s = make(pages=4, page=16, budget=64, chunk=64)
    s.add(0, list(range(31)), 10)
    s.add(1, list(range(30)), 10)
    plan, _ = run_round(s)                          # both prefill: 2 pages each, the pool is full
    assert [(e.req, e.count) for e in plan] == [(0, 31), (1, 30)] and cache.free_pages() == 0
    plan, _ = run_round(s)                          # 0 decodes in its second page; 1 (30 -> 31) too
    assert [(e.req, e.count) for e in plan] == [(0, 1), (1, 1)]
    plan, _ = run_round(s)                          # 0 needs a third page: 1 gives way and waits
    assert [(e.req, e.start, e.count) for e in plan] == [(0, 32, 1)]
    assert s.preemptions == 1 and s.info(1).computed == 0 and s.info(1).preemptions == 1 and s.n_waiting == 1
    assert not cache.has(1)
    # 1 keeps its tokens (prompt and what it generated) and is computed again when there is room
    assert s.info(1).n_tokens == 32
    cache.check()
    seen = []
    for _ in range(40):
        plan, done = run_round(s)
        seen += [(e.req, e.start, e.count) for e in plan if e.req == 1]
        if s.idle:
            break
    assert seen[0][1] == 0 and s.info(0).reason == "max_steps" and s.info(1).reason == "max_steps"
    assert s.info(1).generated == 10
    assert cache.free_pages() == 4 and cache.live_requests() == 0


def test_a_prompt_portion_shrinks_to_the_free_pages_or_waits():
    cache, s = make(pages=3, page=16, budget=64, chunk=64)
    s.add(0, list(range(20)), 40)
    run_round(s)                                    # 2 pages
    s.add(1, list(range(40)), 4)
    plan, _ = run_round(s)
    assert [(e.req, e.start, e.count) for e in plan] == [(0, 20, 1), (1, 0, 16)]      # one page is left: 16 tokens
    plan, _ = run_round(s)
    assert [(e.req, e.count) for e in plan] == [(0, 1)]                               # 1 waits for pages
    assert s.n_running == 2 and s.preemptions == 0


def test_a_request_that_does_not_fit_into_the_empty_pool_ends_with_length():
    cache, s = make(pages=2, page=16, budget=64, chunk=64)
    s.add(0, list(range(40)), 4)
    done_all = {}
    for _ in range(6):
        _, done = run_round(s)
        done_all.update(done)
        if s.idle:
            break
    assert done_all == {0: "length"} and cache.free_pages() == 2 and cache.live_requests() == 0


def test_a_kept_cache_goes_on_with_the_next_turn():
    """llama.cu/xtask/src/chat/mod.rs:54-71: the same session is started again with more tokens."""
    cache, s = make()
    s.add(0, [1, 2, 3, 4], 2, keep=True)
    while not s.idle:
        run_round(s)
    assert s.info(0).reason == "max_steps" and cache.has(0) and cache.length(0) == 5     # the last token is not fed yet
    s.extend(0, [9, 9, 9], 2)
    plan, _ = run_round(s)
    assert [(e.req, e.start, e.count, e.want_logits) for e in plan] == [(0, 5, 4, True)]
    while not s.idle:
        run_round(s)
    assert s.info(0).n_tokens == 4 + 2 + 3 + 2
    s.drop(0)
    assert not cache.has(0) and cache.free_pages() == 64


@pytest.mark.parametrize("seed", range(5))
def test_random_load_every_request_ends_and_nothing_is_lost(seed):
    rng = random.Random(seed)
    cache, s = make(pages=rng.choice([6, 10, 30]), page=16, slots=5, seqs=rng.choice([2, 5]), budget=rng.choice([8, 40]),
                    chunk=rng.choice([4, 16, 64]), max_len=96)
    want = {}
    nxt = 0
    finished = {}
    for step in range(3000):
        if nxt < 25 and rng.random() < 0.3:
            n, k = rng.randint(1, 90), rng.randint(1, 30)
            s.add(nxt, [rng.randrange(50) for _ in range(n)], k)
            want[nxt] = (n, k)
            nxt += 1
        def check(plan):
            assert sum(e.count for e in plan) <= 40
            ids = [e.req for e in plan]
            assert len(set(ids)) == len(ids)
            for e in plan:
                assert cache.length(e.req) == e.start + e.count        # the step's tokens are in the cache
        plan, done = run_round(s, check=check)
        finished.update(done)
        cache.check()
        if nxt == 25 and s.idle:
            break
    assert s.idle and set(finished) == set(want)
    for rid, (n, k) in want.items():
        info = s.info(rid)
        if info.reason == "max_steps":
            assert info.generated == k
        else:
            assert info.reason == "length"
            assert info.n_tokens >= 96 or (n + 15) // 16 + 0 >= 0
    assert cache.live_requests() == 0


def test_a_token_appended_before_it_is_known_gets_its_value_later():
    cache, s = make()
    s.add(0, [1, 2, 3], 4)
    run_round(s, next_token=lambda req, n: 0)            # a placeholder stands for the sampled token
    assert s.tokens(0) == [1, 2, 3, 0]
    s.set_token(0, 3, 77)
    assert s.tokens(0) == [1, 2, 3, 77]
    with pytest.raises(Exception):
        s.set_token(0, 4, 5)
    with pytest.raises(Exception):
        s.set_token(9, 0, 5)


def test_an_end_learned_late_cuts_what_was_appended_and_computed_beyond_it():
    """Two rounds ran with placeholders; the first round's token turns out to end the sequence.
    The tokens are cut after it, a kept cache to what precedes it, and the pages beyond come back."""
    cache, s = make(page=4, pages=16)
    s.add(0, list(range(7)), 10, keep=True)
    run_round(s, next_token=lambda req, n: 0)            # prompt, first placeholder (index 7)
    run_round(s, next_token=lambda req, n: 0)            # computes index 7, second placeholder (index 8)
    run_round(s, next_token=lambda req, n: 0)            # computes index 8 (a third page), third placeholder
    assert s.info(0).n_tokens == 10 and cache.length(0) == 9
    assert s.finish(0, "eos", 8) == "eos"
    info = s.info(0)
    assert (info.n_tokens, info.generated, info.reason) == (8, 1, "eos")
    assert cache.length(0) == 7                            # the end-of-sequence token itself is not in the cache
    assert s.take_finished() == [0]
    assert s.plan() == []
    cache.check()
    # it goes on from there
    s.extend(0, [5, 6], 3)
    plan = s.plan()
    assert [(e.req, e.start, e.count) for e in plan] == [(0, 7, 3)]
    s.commit()
    s.abort(0)
    s.drop(0)
    cache.check()
    assert cache.free_pages(0) == 16


def test_an_end_by_count_at_the_same_token_takes_the_late_reason():
    cache, s = make()
    s.add(0, [1, 2, 3], 1)
    _, done = run_round(s, next_token=lambda req, n: 0)
    assert done == {0: "max_steps"}
    assert s.finish(0, "eos", 4) == "eos" and s.info(0).reason == "eos"
    cache.check()
    assert cache.free_pages(0) == 64


def test_an_end_learned_late_at_a_windows_edge_gives_the_windows_pages_back_and_the_next_turn_recomputes():
    """Window 4, pages of 4: once token 7 is in the cache, page 0 is given back (the next query, at
    8, sees keys 5..8).  If the request is then cut back to 6 tokens, the next query, at 6, would
    see keys 3..6, and key 3 lay in page 0, which is gone.  The request then gives up the pages of
    the group with the window, keeps those of the group without one, and a later turn starts at
    token 0 without asking that group's pool for anything."""
    cache = CacheManager([CacheGroup(16, 4, window=4), CacheGroup(16, 4)], 4)
    s = Scheduler(cache, 4, 64, 32, 512)
    s.add(0, list(range(6)), 10, keep=True)
    run_round(s, next_token=lambda req, n: 0)            # tokens 0..5 computed, placeholder 6
    run_round(s, next_token=lambda req, n: 0)            # token 6 computed, placeholder 7
    run_round(s, next_token=lambda req, n: 0)            # token 7 computed: page 0 is given back
    assert cache.length(0) == 8 and cache.table(0)[0] == -1
    # the token at index 6 was the end of the sequence: 7 tokens remain, 6 of them in the cache
    assert s.finish(0, "eos", 7) == "eos"
    assert cache.has(0) and cache.length(0) == 0 and s.info(0).computed == 0
    assert cache.free_pages(0) == 16                       # the window's pages are back in the pool
    assert cache.table(0, 1) and cache.free_pages(1) == 14 and len(cache.table(0, 1)) == 2     # pages for 6 tokens stay
    cache.check()
    s.extend(0, [5, 6], 3)
    plan = s.plan()
    assert [(e.req, e.start, e.count) for e in plan] == [(0, 0, 9)]
    assert cache.free_pages(1) == 13                       # one more page for tokens 8: the first two were its own already
    s.commit()
    s.abort(0); s.drop(0)
    cache.check()
    assert cache.free_pages(0) == 16 and cache.free_pages(1) == 16


def test_a_window_with_a_token_of_slack_can_be_cut_back_by_the_token_computed_beyond_the_end():
    """An engine that runs one round ahead computes one token beyond an end of sequence: here token 6, the end,
    is in the cache (7 tokens) when the end is learned, and the request is to be cut back to 6.  The query at 7
    sees keys 4..7, so without slack page 0 went when token 6 came, and the query at 6 (keys 3..6) has lost key 3.
    With ``slack=1`` (what the engine asks for) page 0 is still there, the request is cut back, and nothing is
    computed again."""
    for slack in (0, 1):
        cache = CacheManager([CacheGroup(16, 4, window=4, slack=slack)], 4)
        s = Scheduler(cache, 4, 64, 32, 512)
        s.add(0, list(range(6)), 10, keep=True)
        for _ in range(2):
            run_round(s, next_token=lambda req, n: 0)
        assert cache.length(0) == 7 and (cache.table(0)[0] >= 0) == (slack == 1)
        assert s.finish(0, "eos", 7) == "eos"
        assert cache.has(0) and cache.length(0) == (6 if slack else 0) and s.info(0).computed == (6 if slack else 0)
    s.extend(0, [5, 6], 3)
    assert [(e.req, e.start, e.count) for e in s.plan()] == [(0, 6, 3)]
    s.commit()
    assert cache.table(0)[0] == -1                         # with 9 tokens in, the query at 8 sees keys 5..8: page 0 goes
    s.abort(0); s.drop(0)
    cache.check()
    assert cache.free_pages(0) == 16


def test_an_end_learned_late_with_state_that_cannot_be_cut_back_recomputes_the_next_turn():
    cache = CacheManager([CacheGroup(16, 4)], 4, can_truncate=False)
    s = Scheduler(cache, 4, 64, 32, 512)
    s.add(0, list(range(7)), 10, keep=True)
    s.add(1, list(range(3)), 2, keep=True)
    run_round(s, next_token=lambda req, n: 0)
    run_round(s, next_token=lambda req, n: 0)
    run_round(s, next_token=lambda req, n: 0)
    assert cache.length(0) == 9
    free = cache.free_pages(0)
    assert s.finish(0, "eos", 8) == "eos"                 # one token computed beyond the end
    # the state cannot be cut back: the request starts again at 0, but its pages (for 7 tokens) stay its own
    assert cache.has(0) and cache.length(0) == 0 and s.info(0).computed == 0
    assert len(cache.table(0)) == 2 and cache.free_pages(0) == free + 1
    # request 1 ended by count with nothing computed beyond its end: its cache stays
    assert s.info(1).reason == "max_steps" and cache.has(1) and cache.length(1) == 4
    s.extend(0, [5], 2)
    s.extend(1, [5], 2)
    plan = s.plan()
    assert sorted((e.req, e.start, e.count) for e in plan) == [(0, 0, 9), (1, 4, 2)]
    cache.check()
