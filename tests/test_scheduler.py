"""The scheduler's decisions (CPU): the reference's two cases, the token budget, decode first,
shortened portions, preemption when pages run out, refusal of what can never fit."""
import pytest

from pulse_infer_amd.cache import CacheManager, PagedKVSpec
from pulse_infer_amd.engine.request import InferenceRequest, RequestState
from pulse_infer_amd.engine.scheduler import ContinuousBatchScheduler, SchedulerError
from pulse_infer_amd.sampling.params import SamplingParams


def test_request_chunk_state_machine():
    """reference: tests/scheduler/test_continuous_batch_scheduler.cpp:10-38"""
    r = InferenceRequest(0, [11, 12, 13], max_new_tokens=2)
    assert r.state == RequestState.WAITING and r.is_prefill
    assert r.get_next_chunk_tokens(2) == [11, 12] and r.get_next_chunk_positions(2) == [0, 1]
    r.start_running()
    r.add_computed_tokens(2)
    assert r.get_next_chunk_tokens(2) == [13] and r.get_next_chunk_positions(2) == [2]
    r.add_computed_tokens(1)
    assert not r.is_prefill and not r.has_pending_input and r.get_next_chunk_size(2) == 0
    assert r.add_sampled_token(21, [99]) is True
    assert r.has_pending_input and r.get_next_chunk_tokens(2) == [21] and r.get_next_chunk_positions(2) == [3]
    r.add_computed_tokens(1)
    assert r.add_sampled_token(99, [99]) is False
    assert r.is_finished and r.generated_tokens == [21, 99] and r.finish_reason == "eos"
    with pytest.raises(RuntimeError):
        r.add_computed_tokens(1)
    with pytest.raises(ValueError):
        InferenceRequest(1, [1], 5).add_computed_tokens(2)


def test_max_new_tokens_and_ignore_eos():
    r = InferenceRequest(0, [1], 2, SamplingParams(ignore_eos=True))
    assert r.add_sampled_token(9, [9]) is True
    assert r.add_sampled_token(9, [9]) is False and r.finish_reason == "length"
    q = InferenceRequest(1, [1], 5)
    assert q.add_sampled_token(-1, []) is False and q.finish_reason == "no_token"


def _finish_step(s, batch, finished=()):
    for p in batch.portions:
        p.request.add_computed_tokens(len(p.tokens))
    s.update_after_step(list(finished))


def test_a_finished_request_frees_a_batch_slot():
    """reference: tests/scheduler/test_continuous_batch_scheduler.cpp:40-66"""
    s = ContinuousBatchScheduler(max_batch_size=2, max_sequences=32, chunk_size=4)
    ids = [s.add_request([1, 2, 3], 4) for _ in range(3)]
    b1 = s.schedule_next_batch()
    assert [r.request_id for r in b1.requests] == ids[:2]
    _finish_step(s, b1, finished=[ids[0]])
    for r in b1.requests[1:]:
        r.add_sampled_token(5, [])
    b2 = s.schedule_next_batch()
    assert [r.request_id for r in b2.requests] == ids[1:]
    st = s.get_stats()
    assert (st.num_running, st.num_waiting, st.num_finished, st.total_requests) == (2, 0, 1, 3)


def _cache(pages, page_size=4, slots=8):
    return CacheManager([PagedKVSpec(1, 8)], page_size=page_size, num_pages=pages, max_requests=slots)


def test_token_budget_decode_first_and_portions_cut_anywhere():
    c = _cache(64)
    s = ContinuousBatchScheduler(8, 8, chunk_size=16, max_num_batched_tokens=10, cache=c, max_positions=256)
    a = s.add_request(list(range(7)), 8)
    b1 = s.schedule_next_batch()
    assert [(p.request.request_id, len(p.tokens), p.samples) for p in b1.portions] == [(a, 7, True)]
    _finish_step(s, b1)
    s.get_request(a).add_sampled_token(3, [])
    b = s.add_request(list(range(30)), 4)
    d = s.add_request(list(range(5)), 4)
    b2 = s.schedule_next_batch()
    # the decoding request first with one token, the rest of the budget (9) to the next prompt, nothing for the third
    assert [(p.request.request_id, len(p.tokens), p.start, p.samples) for p in b2.portions] == [(a, 1, 7, True), (b, 9, 0, False)]
    assert b2.num_tokens() == 10
    _finish_step(s, b2)
    s.get_request(a).add_sampled_token(3, [])
    b3 = s.schedule_next_batch()
    assert [(p.request.request_id, len(p.tokens), p.start) for p in b3.portions] == [(a, 1, 8), (b, 9, 9)]
    _finish_step(s, b3)
    s.get_request(a).add_sampled_token(3, [])
    b4 = s.schedule_next_batch()
    assert [(p.request.request_id, len(p.tokens), p.start) for p in b4.portions] == [(a, 1, 9), (b, 9, 18)]
    _finish_step(s, b4)
    s.get_request(a).add_sampled_token(3, [])
    b5 = s.schedule_next_batch()
    # b's last 3 prompt tokens end its prompt (sampled), and the third request gets what is left of the budget
    assert [(p.request.request_id, len(p.tokens), p.samples) for p in b5.portions] == [(a, 1, True), (b, 3, True), (d, 5, True)]
    c.check()


def test_admission_waits_for_pages_and_shortens_running_prefill():
    c = _cache(pages=4)            # 16 tokens
    s = ContinuousBatchScheduler(4, 4, chunk_size=8, cache=c, max_positions=64)
    a = s.add_request(list(range(12)), 2)
    b = s.add_request(list(range(6)), 2)
    b1 = s.schedule_next_batch()
    # a takes 8 tokens (2 pages); b's 6 tokens need 2 pages: they fit
    assert [(p.request.request_id, len(p.tokens)) for p in b1.portions] == [(a, 8), (b, 6)]
    _finish_step(s, b1)
    s.get_request(b).add_sampled_token(1, [])
    e = s.add_request(list(range(3)), 2)
    b2 = s.schedule_next_batch()
    # no page is free: b decodes inside its page; a's next portion is not possible; e is not admitted
    assert [(p.request.request_id, len(p.tokens)) for p in b2.portions] == [(b, 1)]
    assert s.num_waiting() == 1 and not b2.preempted
    _finish_step(s, b2)
    s.get_request(b).add_sampled_token(1, [])     # second token: b is finished (max_new_tokens = 2)
    s.update_after_step([b])
    b3 = s.schedule_next_batch()
    assert [(p.request.request_id, len(p.tokens)) for p in b3.portions] == [(a, 4), (e, 3)]
    c.check()


def test_preemption_of_the_newest_when_a_decode_needs_a_page():
    c = _cache(pages=4)
    s = ContinuousBatchScheduler(4, 4, chunk_size=8, cache=c, max_positions=64)
    a = s.add_request(list(range(8)), 5)
    b = s.add_request(list(range(8)), 5)
    b1 = s.schedule_next_batch()
    assert len(b1.portions) == 2 and c.free_pages() == [0]
    _finish_step(s, b1)
    for rid in (a, b):
        s.get_request(rid).add_sampled_token(7, [])
    b2 = s.schedule_next_batch()
    # a needs a fifth page: b, admitted last, is preempted and waits at the front
    assert [r.request_id for r in b2.preempted] == [b]
    assert [(p.request.request_id, len(p.tokens)) for p in b2.portions] == [(a, 1)]
    rb = s.get_request(b)
    assert rb.state == RequestState.PREEMPTED and rb.num_computed_tokens == 0 and rb.generated_tokens == [7]
    assert s.waiting[0] is rb and s.get_stats().num_preemptions == 1
    c.check()
    _finish_step(s, b2, finished=[a])
    b3 = s.schedule_next_batch()
    # b runs again from its first token: prompt and the token it had generated (a portion of the chunk's 8 tokens,
    # extended by the ninth since the step's budget has room), then sampling goes on
    assert [(p.request.request_id, p.tokens, p.samples) for p in b3.portions] == [(b, list(range(8)) + [7], True)]
    _finish_step(s, b3)
    s.get_request(b).add_sampled_token(9, [])
    b4 = s.schedule_next_batch()
    assert [(p.tokens, p.start, p.samples) for p in b4.portions] == [([9], 9, True)]
    c.check()


def test_budget_that_is_left_extends_the_portions_in_order():
    """Every prefilling request gets its portion of at most a chunk first; what the budget still holds then goes to
    the same portions in their order, as far as tokens, pages and budget reach."""
    c = _cache(pages=64)
    s = ContinuousBatchScheduler(4, 4, chunk_size=8, max_num_batched_tokens=40, cache=c, max_positions=256)
    a = s.add_request(list(range(100)), 2)
    b1 = s.schedule_next_batch()
    assert [(p.request.request_id, len(p.tokens), p.start, p.samples) for p in b1.portions] == [(a, 40, 0, False)]
    _finish_step(s, b1)
    b = s.add_request(list(range(30)), 2)
    d = s.add_request(list(range(5)), 2)
    b2 = s.schedule_next_batch()
    # a chunk each for a and b, all of d; the 19 left go to a
    assert [(p.request.request_id, len(p.tokens), p.start, p.samples) for p in b2.portions] == \
        [(a, 8 + 19, 40, False), (b, 8, 0, False), (d, 5, 0, True)]
    assert b2.num_tokens() == 40 and b2.portions[0].tokens == list(range(40, 67))
    _finish_step(s, b2)
    s.get_request(d).add_sampled_token(1, [])
    b3 = s.schedule_next_batch()
    # d decodes first; a and b a chunk each; 23 left: a takes 23 of the 25 tokens it still has
    assert [(p.request.request_id, len(p.tokens), p.start) for p in b3.portions] == [(d, 1, 5), (a, 31, 67), (b, 8, 8)]
    _finish_step(s, b3)
    s.get_request(d).add_sampled_token(1, [])
    s.update_after_step([d])
    b4 = s.schedule_next_batch()
    # a ends its prompt with 2 tokens (sampled); what is left extends b to the end of its prompt (14 tokens)
    assert [(p.request.request_id, len(p.tokens), p.samples) for p in b4.portions] == [(a, 2, True), (b, 14, True)]
    c.check()
    # pages decide too: an extension is cut where the pool ends, and nobody is preempted for it
    c2 = _cache(pages=5)          # 20 tokens
    s2 = ContinuousBatchScheduler(4, 4, chunk_size=4, max_num_batched_tokens=64, cache=c2, max_positions=256)
    x = s2.add_request(list(range(19)), 1)
    y = s2.add_request(list(range(3)), 1)
    b5 = s2.schedule_next_batch()
    assert [(p.request.request_id, len(p.tokens)) for p in b5.portions] == [(x, 16), (y, 3)] and not b5.preempted
    c2.check()


def test_portions_stay_at_the_chunk_size_when_extension_is_off():
    """``extend_portions=False``: the reference's meaning of the chunk size, no portion longer than it whatever the
    budget has left; and a request that is admitted as computed goes on from there."""
    c = _cache(pages=64)
    s = ContinuousBatchScheduler(4, 4, chunk_size=8, max_num_batched_tokens=40, cache=c, max_positions=256,
                                 extend_portions=False)
    a = s.add_request(list(range(30)), 2)
    b = s.add_request(list(range(5)), 2)
    sizes = []
    while s.get_request(a).is_prefill:
        batch = s.schedule_next_batch()
        sizes.append([(p.request.request_id, len(p.tokens)) for p in batch.portions])
        _finish_step(s, batch, finished=[b] if len(sizes) == 1 else [])
    assert sizes == [[(a, 8), (b, 5)], [(a, 8)], [(a, 8)], [(a, 6)]]
    d = s.add_request(list(range(21)), 3)
    with pytest.raises(SchedulerError, match="cannot count as computed"):
        s.admit_as_computed(d, 21)
    s.admit_as_computed(d, 20)
    assert c.computed(d) == 20 and len(c.table(0, d)) == 5 and s.get_request(d).state == RequestState.RUNNING
    batch = s.schedule_next_batch()
    assert [(p.request.request_id, p.tokens, p.start, p.samples) for p in batch.portions if p.request.request_id == d] == \
        [(d, [20], 20, True)]
    with pytest.raises(SchedulerError, match="not waiting"):
        s.admit_as_computed(d, 3)
    c.check()


def test_what_can_never_fit_is_refused():
    c = _cache(pages=2)
    s = ContinuousBatchScheduler(2, 2, chunk_size=8, cache=c, max_positions=16)
    with pytest.raises(SchedulerError, match="positions"):
        s.add_request(list(range(10)), 8)
    with pytest.raises(SchedulerError, match="cache pages"):
        s.add_request(list(range(8)), 2)           # 9 tokens = 3 pages of 4
    ok = s.add_request(list(range(7)), 2)          # 8 tokens = 2 pages
    assert s.get_request(ok) is not None
    with pytest.raises(ValueError):
        s.add_request([], 2)


def test_a_lone_request_that_outgrows_the_pool_is_an_error_not_a_hang():
    c = _cache(pages=2)
    s = ContinuousBatchScheduler(2, 2, chunk_size=8, cache=None, max_positions=64)
    a = s.add_request(list(range(8)), 5)
    s.cache = c                                    # past the admission check, to reach the running-time decision
    _finish_step(s, s.schedule_next_batch())
    s.get_request(a).add_sampled_token(1, [])
    with pytest.raises(SchedulerError, match="too small"):
        s.schedule_next_batch()


def test_prompts_that_hold_each_others_pages_do_not_stall():
    """Three long prompts admitted together fill the pool while all of them are still in their prompts: none can get
    another page.  The newest gives way (twice if need be) and every request finishes with what it generates alone."""
    c = _cache(pages=8)            # 32 tokens
    s = ContinuousBatchScheduler(4, 4, chunk_size=4, cache=c, max_positions=64)
    ids = [s.add_request(list(range(20)), 2) for _ in range(3)]     # each needs 6 pages in the end
    steps, preempted, done = 0, 0, set()
    while s.has_work():
        batch = s.schedule_next_batch()
        assert not batch.empty()
        preempted += len(batch.preempted)
        finished = []
        for p in batch.portions:
            p.request.add_computed_tokens(len(p.tokens))
            if p.samples and not p.request.add_sampled_token(5, []):
                finished.append(p.request.request_id)
        s.update_after_step(finished)
        done.update(finished)
        c.check()
        steps += 1
        assert steps < 200, "the scheduler goes round in circles"
    assert done == set(ids) and preempted >= 1
    assert all(s.get_request(i).generated_tokens == [5, 5] for i in ids)
    assert c.free_pages() == [8]


@pytest.mark.parametrize("seed", range(60))
def test_random_workloads_always_finish(seed):
    """Random pools (one group with all keys, sometimes a windowed one beside it), portions, budgets, batch limits and
    requests that arrive while others run: every step schedules something, the cache stays consistent, every
    request ends with exactly the tokens it was allowed, and nothing is left in the pool."""
    import random
    rng = random.Random(seed)
    page = rng.choice([1, 4, 16])
    specs = [PagedKVSpec(1, 8)] + ([PagedKVSpec(1, 8, window=rng.choice([3, 10, 40]))] if rng.random() < 0.4 else [])
    longest = rng.choice([12, 40, 90])
    pages = (longest + 8 + page - 1) // page + rng.choice([0, 1, 3, 20])
    slots = rng.choice([1, 2, 4, 8])
    c = CacheManager(specs, page_size=page, num_pages=pages, max_requests=slots)
    budget = rng.choice([None, 5, 17, 64])
    s = ContinuousBatchScheduler(rng.choice([1, 2, 4, 8]), rng.choice([1, 2, 8]), chunk_size=rng.choice([1, 3, 8, 32]),
                                 max_num_batched_tokens=budget, cache=c, max_positions=256)
    eos = [7]
    todo = [(rng.randint(1, longest), rng.randint(0, 8)) for _ in range(rng.randint(1, 12))]
    ids, allowed = [], {}

    def add():
        n, new = todo.pop()
        rid = s.add_request([rng.randint(0, 6) for _ in range(n)], new,
                            SamplingParams(ignore_eos=rng.random() < 0.5))
        ids.append(rid)
        allowed[rid] = new

    for _ in range(min(len(todo), rng.randint(1, 4))):
        add()
    steps = 0
    while s.has_work() or todo:
        if todo and (not s.has_work() or rng.random() < 0.3):
            add()
        batch = s.schedule_next_batch()
        assert not batch.empty()
        if budget is not None:
            assert batch.num_tokens() <= budget
        finished = []
        for p in batch.portions:
            assert c.reserved(p.request.request_id) >= p.start + len(p.tokens)
            p.request.add_computed_tokens(len(p.tokens))
            c.advance(p.request.request_id, p.start + len(p.tokens))
            if p.samples:
                if not p.request.can_generate_more:
                    p.request.finish("length")
                    finished.append(p.request.request_id)
                elif not p.request.add_sampled_token(rng.choice([1, 2, 7]), eos):
                    finished.append(p.request.request_id)
        s.update_after_step(finished)
        c.check()
        steps += 1
        assert steps < 5000, "the scheduler goes round in circles"
    for rid in ids:
        r = s.get_request(rid)
        assert r.is_finished and len(r.generated_tokens) <= allowed[rid]
        if r.finish_reason == "length":
            assert len(r.generated_tokens) == allowed[rid]
    assert c.free_pages() == [pages] * len(specs) and c.slots.num_free == slots
