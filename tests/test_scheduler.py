"""The scheduler's decisions, with the real cache manager (no slabs) and no model.
The sequences of plans restate worker/tests/test_scheduler.py:29-182, adapted where this
scheduler cuts prompts (the reference never does)."""

import pytest

from distie_amd.cache import CacheManager
from distie_amd.engine.scheduler import BlockPoolExhausted, Scheduler, Request, Phase
from distie_amd.parts import PagedKV
from distie_amd.sampling import SamplingParams

EOS = 99


def make(pages, block=4, max_seqs=32, budget=2048, window=None, slots=8, max_model_len=None):
    needs = [PagedKV(1, 16), PagedKV(1, 16, window)] if window else [PagedKV(1, 16)]
    cache = CacheManager(needs, block, pages, slots, allocate=False)
    return Scheduler(cache, max_seqs, budget, max_model_len), cache


def seq(rid, prompt_len, max_new=8):
    return Request(request_id=rid, prompt_ids=list(range(1, prompt_len + 1)),
                    params=SamplingParams(max_new_tokens=max_new), eos_ids=(EOS,))


def run(sched, cache, tokens):
    """schedule, pretend the step ran (the step function advances the cache's counts), complete"""
    plan = sched.schedule()
    for item in plan.portions:
        cache.commit(item.request.request_id, len(item.token_ids))
    picks = [tokens if isinstance(tokens, int) else tokens[i] for i in range(len(plan.portions))]
    return plan, sched.complete(plan, picks)


def names(plan):
    return [i.request.request_id for i in plan.portions]


def test_fifo_and_prefill_then_decode():
    sched, cache = make(8)
    a, b = seq("a", 5), seq("b", 2)
    sched.submit(a)
    sched.submit(b)
    plan = sched.schedule()
    assert names(plan) == ["a", "b"]
    assert [len(i.token_ids) for i in plan.portions] == [5, 2]
    assert [i.begin for i in plan.portions] == [0, 0]
    assert all(i.samples for i in plan.portions)
    assert len(cache.request("a").tables[0]) == 2
    for i in plan.portions:
        cache.commit(i.request.request_id, len(i.token_ids))
    sched.complete(plan, [7, 8])
    plan = sched.schedule()
    assert [(i.token_ids, i.begin) for i in plan.portions] == [([7], 5), ([8], 2)]
    assert plan.is_decode


def test_max_seqs_and_token_budget_cut_prompts():
    sched, cache = make(16, max_seqs=2, budget=6)
    for rid in ("a", "b", "c"):
        sched.submit(seq(rid, 4))
    plan, _ = run(sched, cache, 7)
    # a whole, b's first two tokens: the budget of 6 is filled, b does not sample yet
    assert [(i.request.request_id, i.token_ids, i.samples) for i in plan.portions] == [("a", [1, 2, 3, 4], True), ("b", [1, 2], False)]
    assert sched.request("b").output_ids == []
    plan, _ = run(sched, cache, 7)
    # decoding first, then the prompt in flight
    assert [(i.request.request_id, i.token_ids, i.begin, i.samples) for i in plan.portions] == \
        [("a", [7], 4, True), ("b", [3, 4], 2, True)]
    plan, _ = run(sched, cache, 7)
    assert names(plan) == ["a", "b"] and sched.num_waiting == 1      # max_seqs keeps c waiting


def test_long_prompt_is_cut_under_the_budget():
    sched, cache = make(16, budget=4)
    sched.submit(seq("a", 10))
    sizes = []
    for _ in range(3):
        plan, out = run(sched, cache, 7)
        sizes.append((plan.num_tokens, plan.portions[0].begin, plan.portions[0].samples))
    assert sizes == [(4, 0, False), (4, 4, False), (2, 8, True)]
    assert out[0].token_id == 7
    assert all(p.num_tokens <= 4 for p in [plan])


def test_every_step_stays_within_the_budget_and_decodes_come_first():
    sched, cache = make(64, budget=8)
    sched.submit(seq("a", 3, max_new=20))
    run(sched, cache, 7)
    sched.submit(seq("b", 30, max_new=2))
    for _ in range(6):
        plan, _ = run(sched, cache, 7)
        assert plan.num_tokens <= 8
        assert plan.portions[0].request.request_id == "a" and len(plan.portions[0].token_ids) == 1


def test_waits_for_blocks():
    sched, cache = make(2)
    sched.submit(seq("a", 7, max_new=1))
    sched.submit(seq("b", 4, max_new=2))
    plan = sched.schedule()
    assert names(plan) == ["a"] and cache.free_pages() == [0]
    cache.commit("a", 7)
    emitted = sched.complete(plan, [7])
    assert emitted[0].finished and emitted[0].request.finish_reason == "length"
    assert names(sched.schedule()) == ["b"]


def test_request_that_can_never_fit_is_refused():
    sched, _ = make(2)
    with pytest.raises(BlockPoolExhausted):
        sched.submit(seq("a", 6, max_new=4))
    sched2, _ = make(100, max_model_len=12)
    with pytest.raises(ValueError, match="model length"):
        sched2.submit(seq("a", 6, max_new=7))


def test_rejects_duplicate_and_empty():
    sched, _ = make(4)
    sched.submit(seq("a", 2))
    with pytest.raises(ValueError):
        sched.submit(seq("a", 2))
    with pytest.raises(ValueError):
        sched.submit(Request(request_id="b", prompt_ids=[]))


def test_eos_and_cap_free_blocks():
    sched, cache = make(4)
    sched.submit(seq("a", 2, max_new=5))
    sched.submit(seq("b", 2, max_new=1))
    plan, emitted = run(sched, cache, [EOS, 3])
    assert [(e.request.request_id, e.finished, e.request.finish_reason) for e in emitted] == \
        [("a", True, "stop"), ("b", True, "length")]
    assert cache.free_pages() == [4] and cache.slots.num_free == 8
    assert not sched.has_work()


def test_ignore_eos():
    sched, cache = make(4)
    s = Request("a", [1, 2], SamplingParams(max_new_tokens=3, ignore_eos=True), eos_ids=(EOS,))
    sched.submit(s)
    _, emitted = run(sched, cache, EOS)
    assert not emitted[0].finished


def test_newest_is_preempted_and_recomputed_without_reemitting():
    sched, cache = make(2)
    a, b = seq("a", 3, max_new=4), seq("b", 3, max_new=4)
    sched.submit(a)
    sched.submit(b)
    run(sched, cache, [10, 20])
    run(sched, cache, [11, 21])       # 5 tokens each: page 1 is full
    plan = sched.schedule()
    # a needs a second page; the pool is empty, so b (newest) is preempted
    assert names(plan) == ["a"]
    assert b.phase is Phase.QUEUED and "b" not in cache
    assert b.output_ids == [20, 21] and b.preemptions == 1 and b.num_computed == 0
    cache.commit("a", 1)
    assert [e.token_id for e in sched.complete(plan, [12])] == [12]
    cache.check()


def test_recompute_prefills_prompt_plus_output():
    sched, cache = make(3)
    a, b = seq("a", 3, max_new=2), seq("b", 3)
    sched.submit(a)
    sched.submit(b)
    run(sched, cache, [10, 20])
    plan, _ = run(sched, cache, [11, 21])     # a finishes on the cap and frees its pages
    assert len(plan.portions) == 2 and cache.free_pages() == [2]
    sched.give_way(b)
    item = sched.schedule().portions[0]
    assert (item.request.request_id, item.token_ids, item.begin, item.samples) == ("b", [1, 2, 3, 20, 21], 0, True)


def test_queue_front_after_preemption_and_no_readmission_in_that_step():
    sched, cache = make(2)
    for rid in ("a", "b"):
        sched.submit(seq(rid, 3, max_new=4))
    run(sched, cache, [1, 2])
    run(sched, cache, [1, 2])
    sched.submit(seq("c", 1, max_new=4))
    plan = sched.schedule()
    assert names(plan) == ["a"]
    assert [s.request_id for s in sched.queued()] == ["b", "c"]


def test_needy_request_preempts_itself_when_it_is_the_newest():
    sched, cache = make(3)
    a, b = seq("a", 4, max_new=8), seq("b", 4, max_new=8)
    sched.submit(a)
    sched.submit(b)
    run(sched, cache, 5)                      # one page each, one page free
    plan = sched.schedule()
    # both need a second page: a (older) takes the free one, b is the newest and goes itself
    assert names(plan) == ["a"] and sched.queued()[0] is b and b.preemptions == 1
    assert cache.free_pages() == [1]
    cache.check()


def test_abort_running_frees_on_next_schedule():
    sched, cache = make(4)
    sched.submit(seq("a", 2))
    plan = sched.schedule()
    sched.abort("a")
    cache.commit("a", 2)
    assert sched.complete(plan, [5]) == []        # aborted in flight: nothing emitted
    assert sched.schedule().portions == ()
    assert cache.free_pages() == [4] and not sched.has_work()


def test_abort_waiting_and_unknown():
    sched, cache = make(1)
    sched.submit(seq("a", 3, max_new=1))
    sched.submit(seq("b", 3, max_new=1))
    sched.abort("b")
    sched.abort("missing")
    assert names(sched.schedule()) == ["a"] and sched.num_waiting == 0


def test_failed_step_ends_its_requests_and_frees():
    sched, cache = make(4)
    sched.submit(seq("a", 2))
    plan = sched.schedule()
    failed = sched.fail(plan, RuntimeError("boom"))
    assert [s.request_id for s in failed] == ["a"] and failed[0].finish_reason == "error"
    assert cache.free_pages() == [4] and not sched.has_work()


def test_windowed_group_lets_long_requests_decode_in_few_pages():
    sched, cache = make(8, block=4, window=4, budget=8)
    sched.submit(seq("a", 6, max_new=20))
    for _ in range(15):
        run(sched, cache, 7)
        cache.check()
    full, windowed = cache.free_pages()
    assert full == 8 - 5 and windowed >= 8 - 2      # 20 cached: 5 pages in full, at most 2 in the window group


def test_the_step_after_is_planned_ahead_only_when_that_is_plain():
    sched, cache = make(8, block=4)
    a, b, c = seq("a", 3, max_new=2), seq("b", 2, max_new=5), seq("c", 9, max_new=5)
    sched.submit(a)
    sched.submit(b)
    plan = sched.schedule()
    for item in plan.portions:
        cache.commit(item.request.request_id, len(item.token_ids))
    # both decode from here on, nothing waits: the next step can be planned before the tokens are known
    ahead = sched.schedule_ahead(plan)
    assert names(ahead) == ["a", "b"] and ahead.feeds == (0, 1)
    assert [(i.token_ids, i.begin, i.samples) for i in ahead.portions] == [([sched.PENDING], 3, True), ([sched.PENDING], 2, True)]
    sched.complete(plan, [7, 8])
    for item in ahead.portions:
        cache.commit(item.request.request_id, 1)
    # a reaches its length with the token that is pending now: it is not in the step after
    after = sched.schedule_ahead(ahead)
    assert names(after) == ["b"] and after.feeds == (1,)
    out = sched.complete(ahead, [5, 6])
    assert [(e.request.request_id, e.finished) for e in out] == [("a", True), ("b", False)]
    cache.commit("b", 1)
    # b ends with an end-of-sequence token: its row of the step after was computed for nothing
    again = sched.schedule_ahead(after)
    assert names(again) == ["b"]
    out = sched.complete(after, [EOS])
    assert out[0].finished and b.finish_reason == "stop"
    assert sched.complete(again, [4]) == [] and b.output_ids == [8, 6, EOS]
    cache.check()
    assert cache.free_pages() == [8]
    # a request that waits is admitted by the step planned ahead if a seat, a slot and its pages are free now
    sched.submit(seq("d", 2))
    plan = sched.schedule()
    for item in plan.portions:
        cache.commit(item.request.request_id, len(item.token_ids))
    sched.submit(c)
    ahead = sched.schedule_ahead(plan)
    assert names(ahead) == ["d", "c"] and ahead.feeds == (0,)
    assert [(i.token_ids, i.begin, i.samples) for i in ahead.portions] == [([sched.PENDING], 2, True), (list(range(1, 10)), 0, True)]
    sched.complete(plan, [1])
    for item in ahead.portions:
        cache.commit(item.request.request_id, len(item.token_ids))
    sched.complete(ahead, [2, 3])
    assert c.output_ids == [3] and c.num_computed == 9
    # a prompt in portions goes on in the step planned ahead; a waiting request without pages stays out of it
    small, cache2 = make(3, block=4, budget=4)
    e, f = seq("e", 7, max_new=3), seq("f", 8, max_new=3)
    small.submit(e)
    small.submit(f)
    plan = small.schedule()
    assert [(i.request.request_id, i.token_ids, i.samples) for i in plan.portions] == [("e", [1, 2, 3, 4], False)]   # f: no pages
    for item in plan.portions:
        cache2.commit(item.request.request_id, len(item.token_ids))
    ahead = small.schedule_ahead(plan)
    assert [(i.request.request_id, i.token_ids, i.begin, i.samples) for i in ahead.portions] == [("e", [5, 6, 7], 4, True)]
    assert ahead.feeds == () and small.num_waiting == 1
    small.complete(plan, [None])
    for item in ahead.portions:
        cache2.commit(item.request.request_id, len(item.token_ids))
    after = small.schedule_ahead(ahead)
    assert names(after) == ["e"] and after.feeds == (0,)
    small.complete(ahead, [1])
    # a page that is not there: no planning ahead, the plain schedule decides who gives way
    tight, cache4 = make(2, block=4)
    tight.submit(seq("j", 4, max_new=4))
    tight.submit(seq("k", 3, max_new=1))
    plan = tight.schedule()
    assert names(plan) == ["j", "k"]
    for item in plan.portions:
        cache4.commit(item.request.request_id, len(item.token_ids))
    assert tight.schedule_ahead(plan) is None             # j needs a second page, none is free
    tight.complete(plan, [1, 2])
    # a request waits and those that go on fill every seat: the step after is planned without it; the seat of a
    # request that ends with the pending token is free one step later
    two, cache3 = make(8, block=4, max_seqs=2)
    for s_ in (seq("g", 2, max_new=2), seq("h", 3, max_new=9), seq("i", 2, max_new=9)):
        two.submit(s_)
    plan = two.schedule()
    assert names(plan) == ["g", "h"]
    for item in plan.portions:
        cache3.commit(item.request.request_id, len(item.token_ids))
    ahead = two.schedule_ahead(plan)
    assert names(ahead) == ["g", "h"]
    two.complete(plan, [1, 2])
    for item in ahead.portions:
        cache3.commit(item.request.request_id, 1)
    after = two.schedule_ahead(ahead)
    assert names(after) == ["h"] and after.feeds == (1,)      # g ends with the pending token; its seat is still taken
    two.complete(ahead, [3, 4])
    cache3.commit("h", 1)
    last = two.schedule_ahead(after)
    assert names(last) == ["h", "i"] and last.feeds == (0,)   # now i has g's seat
    two.complete(after, [5])


def drive(sched, cache, lookahead, token=5, limit=2000):
    """The engine's loop without a model: schedule, the step function's commit, plan the next step ahead
    if asked, complete. -> steps run."""
    steps, ahead = 0, None
    while sched.has_work():
        plan, ahead = ahead, None
        if plan is not None and not any(p.request.phase is Phase.SEATED for p in plan.portions):
            plan = None
        if plan is None:
            plan = sched.schedule()
            assert plan.portions
            for item in plan.portions:
                cache.commit(item.request.request_id, len(item.token_ids))
        if lookahead:
            ahead = sched.schedule_ahead(plan)
            if ahead is not None:
                for item in ahead.portions:
                    cache.commit(item.request.request_id, len(item.token_ids))
        sched.complete(plan, [token] * len(plan.portions))
        cache.check()
        steps += 1
        assert steps < limit
    return steps


def test_who_gave_way_does_not_come_straight_back_through_a_step_planned_ahead():
    """A pool so tight that the newest of three requests must give way while the older two decode: with steps
    planned ahead it is seated again no sooner than the plain schedule would seat it (not in the step planned
    right behind the one it gave way in, and only where a page stays free for each older request), so it gives
    way as often as without look-ahead."""
    def preemptions(lookahead, pages, block, prompts, lengths):
        sched, cache = make(pages, block=block, max_seqs=len(prompts))
        reqs = [seq(str(i), n, max_new=m) for i, (n, m) in enumerate(zip(prompts, lengths))]
        for r in reqs:
            sched.submit(r)
        drive(sched, cache, lookahead)
        assert all(r.phase is Phase.ENDED and len(r.output_ids) == m for r, m in zip(reqs, lengths))
        assert cache.free_pages() == [pages]
        return sum(r.preemptions for r in reqs)

    # (found by a random search: without the two conditions the look-ahead preempts once more than the plain
    # schedule in each of these)
    for case in ((7, 4, [2, 4, 7, 4, 10, 1], [20, 8, 8, 8, 13, 13]), (8, 4, [9, 7, 5, 4, 11, 5], [18, 5, 2, 20, 17, 4]),
                 (15, 2, [2, 6, 10, 8, 2, 5], [7, 20, 18, 16, 12, 9])):
        plain, ahead = preemptions(False, *case), preemptions(True, *case)
        assert plain > 0 and ahead <= plain, (case, plain, ahead)
    # the step planned behind a step in which somebody gave way seats nobody
    sched, cache = make(4, block=4, max_seqs=3)
    a, b = seq("a", 8, max_new=6), seq("b", 4, max_new=6)
    sched.submit(a)
    sched.submit(b)
    plan = sched.schedule()
    for item in plan.portions:
        cache.commit(item.request.request_id, len(item.token_ids))
    sched.complete(plan, [5, 5])
    plan = sched.schedule()               # a takes the last page for its ninth token, b finds none for its fifth
    assert names(plan) == ["a"] and plan.gave_way and b.preemptions == 1
    cache.commit("a", 1)
    ahead = sched.schedule_ahead(plan)
    assert names(ahead) == ["a"] and sched.queued() == [b]
