"""The scheduler's decisions (no GPU): admission, portions under a token budget, decoding,
finishing and freeing, and what happens when pages run out."""
import pytest

from torchlet_amd.cache.manager import CacheManager
from torchlet_amd.engine.request import Request, RequestState
from torchlet_amd.engine.scheduler import Scheduler
from torchlet_amd.parts.base import PagedNeed

NEED = PagedNeed(num_heads=1, head_dim=16)


def make(pages=20, page=4, slots=4, budget=16, max_positions=256):
    cache = CacheManager([(NEED, None, None)], page_size=page, num_pages=pages, max_requests=slots)
    return Scheduler(cache, max_tokens_per_step=budget, max_positions=max_positions), cache


def req(n, new=4, **kw):
    return Request(prompt_tokens=list(range(1, n + 1)), max_new_tokens=new, **kw)


def run_step(s, token=7):
    chosen = s.schedule()
    done = s.process_output(chosen, [token] * sum(c.samples for c in chosen))
    s.cache.check()
    return chosen, done


def test_validation_follows_the_reference_rules():
    s, _ = make(max_positions=20)
    with pytest.raises(ValueError, match="max_new_tokens"):
        s.add_request(req(3, new=0))
    with pytest.raises(ValueError, match="prompt token"):
        s.add_request(Request(prompt_tokens=[]))
    s.add_request(req(17, new=4))                       # 17 + 4 - 1 = 20 positions: fits
    with pytest.raises(ValueError, match="requires 21 cache positions"):
        s.add_request(req(17, new=5))
    s2, _ = make(pages=4, page=4)                       # 3 usable pages = 12 tokens
    with pytest.raises(ValueError, match="cache pages"):
        s2.add_request(req(10, new=4))                  # alone it could never fit


def test_prompt_is_cut_into_portions_under_the_budget_and_only_the_last_samples():
    s, cache = make(budget=16)
    r = req(40, new=2)
    s.add_request(r)
    seen = []
    while r.state != RequestState.FINISHED:
        chosen, _ = run_step(s)
        seen.append([(c.start, c.count, c.samples) for c in chosen])
    assert seen == [[(0, 16, False)], [(16, 16, False)], [(32, 8, True)], [(40, 1, True)]]
    assert r.output_tokens == [7, 7] and r.finish_reason == "length"
    assert cache.free_pages() == [19] and cache.free_slots() == 4


def test_decoding_goes_first_and_prompts_share_what_is_left():
    s, _ = make(budget=10, pages=40)
    a, b, c = req(3, new=8), req(4, new=8), req(30, new=2)
    for r in (a, b):
        s.add_request(r)
    chosen, _ = run_step(s)
    assert [(x.request, x.count, x.samples) for x in chosen] == [(a, 3, True), (b, 4, True)]
    s.add_request(c)
    chosen, _ = run_step(s)
    # two decode tokens first, the new prompt gets the remaining 8 of the budget
    assert [(x.request, x.start, x.count, x.samples) for x in chosen] == [(a, 3, 1, True), (b, 4, 1, True), (c, 0, 8, False)]
    chosen, _ = run_step(s)
    assert [(x.request, x.start, x.count) for x in chosen] == [(a, 4, 1), (b, 5, 1), (c, 8, 8)]


def test_stop_token_ends_without_being_kept_and_pages_return_at_once():
    s, cache = make()
    r = req(5, new=10, stop_token_ids=frozenset({9}))
    s.add_request(r)
    run_step(s, token=3)
    _, done = run_step(s, token=9)
    assert done == [r] and r.output_tokens == [3] and r.finish_reason == "stop" and r.state == RequestState.FINISHED
    assert cache.free_pages() == [19] and not s.has_work()
    assert s.drain_finished() == [r] and s.drain_finished() == []


def test_slots_limit_live_requests_and_waiting_is_first_come_first_served():
    s, _ = make(slots=2, budget=64)
    rs = [req(4, new=3) for _ in range(4)]
    for r in rs:
        s.add_request(r)
    chosen, _ = run_step(s)
    assert [c.request for c in chosen] == rs[:2] and s.waiting == rs[2:]
    run_step(s)
    _, done = run_step(s)
    assert done == rs[:2]
    chosen, _ = run_step(s)
    assert [c.request for c in chosen] == rs[2:]


def test_when_pages_run_out_the_youngest_is_preempted_and_recomputed():
    # 7 usable pages of 4 tokens.  Two requests of 8 prompt tokens (2 pages each) that decode
    # up to 12 new tokens: together they outgrow the pool.
    s, cache = make(pages=8, page=4, slots=4, budget=32)
    old, young = req(8, new=12), req(8, new=12)
    s.add_request(old)
    s.add_request(young)
    preempted_at = None
    steps = 0
    while s.has_work():
        chosen, _ = run_step(s)
        steps += 1
        assert any(c.request is old for c in chosen) or old.state == RequestState.FINISHED, "the oldest always moves"
        if young.preemptions and preempted_at is None:
            preempted_at = steps
            assert young.state == RequestState.WAITING and young.computed_tokens == 0
            assert s.waiting[0] is young and not cache.has(young.req_id)
            kept = list(young.output_tokens)
        assert steps < 200
    assert preempted_at is not None and s.num_preemptions >= 1
    assert len(old.output_tokens) == 12 and len(young.output_tokens) == 12
    assert young.output_tokens[: len(kept)] == kept            # what it had generated is kept and fed again
    assert cache.free_pages() == [7] and cache.free_slots() == 4


def test_recompute_feeds_prompt_plus_generated_tokens():
    r = req(3, new=9)
    r.output_tokens = [10, 11, 12]
    assert r.sequence_length == 6
    assert r.tokens(0, 6) == [1, 2, 3, 10, 11, 12] and r.tokens(2, 3) == [3, 10, 11] and r.tokens(4, 2) == [11, 12]


def test_nobody_can_move_raises_and_fail_all_resets():
    s, cache = make(pages=4, page=4, slots=2, budget=8)       # 12 tokens of cache
    a = req(6, new=7)                                         # alone it fits exactly (12 positions)
    s.add_request(a)
    run_step(s)
    # steal the free pages behind the scheduler's back: the lone request can neither grow nor be helped
    cache.add_request("thief")
    cache.reserve("thief", 4)
    for _ in range(2):
        run_step(s)
    with pytest.raises(RuntimeError, match="no request can make progress"):
        for _ in range(10):
            run_step(s)
    failed = s.fail_all(RuntimeError("boom"))
    assert a in failed and a.state == RequestState.FINISHED and isinstance(a.error, RuntimeError)
    assert cache.free_pages() == [3] and cache.free_slots() == 2 and not s.has_work()


def test_the_scheduler_looks_ahead_only_where_the_next_step_is_certain():
    """The step after a decode step, decided before that step's tokens are known."""
    s, cache = make(pages=9, page=4, slots=3, budget=8, max_positions=64)
    a, b = req(3, new=3), req(5, new=2)
    s.add_request(a)
    s.add_request(b)
    first = s.schedule()
    assert s.schedule_ahead(first) == []                         # prompts, not decoded tokens
    s.process_output(first, [10, 11])
    second = s.schedule()
    assert [(c.start, c.count, c.samples) for c in second] == [(3, 1, True), (5, 1, True)]
    late = req(1, new=2)
    s.add_request(late)
    assert s.schedule_ahead(second) == []                        # somebody waits: the next step is for schedule() to decide
    s.waiting.clear()
    ahead = s.schedule_ahead(second)                             # b ends with the token of `second`: only a goes on
    assert [(c.request is a, c.start, c.count, c.samples) for c in ahead] == [(True, 4, 1, True)]
    cache.check()
    s.process_output(second, [12, 13])
    assert b.finish_reason == "length" and a.output_tokens == [10, 12]
    s.process_output(ahead, [14])
    assert a.finish_reason == "length" and a.output_tokens == [10, 12, 14] and not s.has_work()
    cache.check()
    assert cache.free_pages() == [8] and cache.free_slots() == 3
    # the tokens after next need two pages and one is left: no step ahead, and no page taken for it
    s, cache = make(pages=4, page=4, slots=2, budget=8, max_positions=64)
    for r in (req(3, new=6), req(3, new=6)):
        s.add_request(r)
    s.process_output(s.schedule(), [5, 5])
    step = s.schedule()                                          # the tokens at position 3 fill the requests' first pages
    assert [(x.start, x.count) for x in step] == [(3, 1), (3, 1)] and cache.free_pages() == [1]
    assert s.schedule_ahead(step) == [] and cache.free_pages() == [1]
    cache.check()
    # a budget smaller than the running requests leaves somebody out: nothing to foresee
    s, cache = make(pages=20, page=4, slots=3, budget=3, max_positions=64)
    for r in (req(1, new=4), req(1, new=4), req(1, new=4)):
        s.add_request(r)
    s.process_output(s.schedule(), [7, 7, 7])
    s.max_tokens_per_step = 2
    chosen = s.schedule()
    assert len(s.running) == 3 and len(chosen) == 2 and not s.waiting and s.schedule_ahead(chosen) == []
