"""The serving loop's bookkeeping on the CPU: the loop one step ahead with the device side replaced by a stand-in
(tokens from a table, no kernels), so that what the loop does with a step in flight can be tested where a failure is
forced from the host; and the protocols by which parts and cache specs answer the step function."""
import pytest

from pulse_infer_amd.cache import CacheManager, PagedKVSpec, StateSpec
from pulse_infer_amd.engine.engine import ContinuousBatchEngine, _InFlight
from pulse_infer_amd.engine.scheduler import ContinuousBatchScheduler, SchedulerError


class _Landed:
    def synchronize(self):
        pass


class _Tokens(list):
    def tolist(self):
        return list(self)


class LoopOnly(ContinuousBatchEngine):
    """The engine's loop over a scheduler and a cache manager, with ``_launch`` drawing tokens from a function of
    (request id, index) instead of running a model."""

    def __init__(self, draw, pages=64, page_size=4, batch=4, chunk=8, eos=()):
        self.cache = CacheManager([PagedKVSpec(1, 8)], page_size=page_size, num_pages=pages, max_requests=batch)
        self.scheduler = ContinuousBatchScheduler(batch, batch, chunk, None, cache=self.cache, max_positions=4096)
        self.eos_token_ids = list(eos)
        self.last_batch = None
        self.draw = draw
        self.launched = 0

    def add_request(self, prompt_tokens, max_new_tokens, sampling=None):
        return self.scheduler.add_request(prompt_tokens, max_new_tokens, sampling)

    def _launch(self, batch, before):
        self.launched += 1
        for p in batch.portions:
            self.cache.advance(p.request.request_id, p.start + len(p.tokens))
        sampled = [p for p in batch.portions if p.samples]
        live = [(row, p.request) for row, p in enumerate(sampled) if p.request.can_generate_more]
        flight = _InFlight(batch, sampled, live)
        if live:
            # what a request draws depends on how many it has drawn; the step before may still hold one of them
            flight.landing = _Tokens(self.draw(q.request_id, q.num_generated) for _, q in live)
            flight.rows = {q.request_id: i for i, (_, q) in enumerate(live)}
            flight.landed = _Landed()
        return flight


def draw(request_id, index):
    return 100 + 10 * request_id + index          # never 0, the place-holder's value


def test_the_loop_one_step_ahead_on_the_cpu_stand_in():
    engine = LoopOnly(draw, eos=[113])
    ids = [engine.add_request([1, 2, 3, 4, 5][:n], new) for n, new in ((5, 6), (3, 9), (1, 0), (4, 2))]
    engine.run_until_complete()
    got = [engine.get_request(i) for i in ids]
    assert got[0].generated_tokens == [100 + k for k in range(6)] and got[0].finish_reason == "length"
    assert got[1].generated_tokens == [110, 111, 112, 113] and got[1].finish_reason == "eos"
    assert engine.get_result(ids[1]) == [110, 111, 112]
    assert got[2].generated_tokens == [] and got[2].finish_reason == "length"
    assert got[3].generated_tokens == [130, 131]
    engine.cache.check()
    assert not engine.cache.requests


@pytest.mark.parametrize("fail_at", [2, 3, 5])
def test_an_error_while_a_step_is_in_flight_leaves_no_placeholder(fail_at):
    """The scheduler raises while the step before is queued and its requests carry place-holders (token 0, a finish by
    length that only the place-holder's count gave): the step's tokens are taken before the error goes on, so every
    token is a drawn one and every finish reason is the one the tokens give."""
    engine = LoopOnly(draw, eos=[111, 121])
    ids = [engine.add_request([7] * n, new) for n, new in ((5, 6), (3, 2), (2, 9))]
    schedule = engine.scheduler.schedule_next_batch
    calls = []

    def failing():
        calls.append(1)
        if len(calls) == fail_at:
            raise SchedulerError("forced by the test")
        return schedule()

    engine.scheduler.schedule_next_batch = failing
    with pytest.raises(SchedulerError, match="forced"):
        engine.run_until_complete()
    assert engine.launched == fail_at - 1
    for i in ids:
        request = engine.get_request(i)
        assert 0 not in request.generated_tokens, (i, request.generated_tokens)
        assert request.generated_tokens == [100 + 10 * i + k for k in range(request.num_generated)]
        if request.generated_tokens and request.generated_tokens[-1] in (111, 121):
            assert request.is_finished and request.finish_reason == "eos"      # (also where its length ended it too)
        elif request.is_finished:
            assert request.finish_reason == "length" and request.num_generated == request.max_new_tokens


def test_a_part_says_whether_it_records_as_an_attribute_or_a_method():
    from pulse_infer_amd.parts.base import Part, says

    class Silent(Part):
        pass

    class ByAttribute(Part):
        records_cleanly = True

    class ByMethod(Part):
        def records_cleanly(self):
            return True

    class NoByMethod(Part):
        def records_cleanly(self):
            return False

    assert not says(Silent(), "records_cleanly") and not says(object(), "records_cleanly")
    assert says(ByAttribute(), "records_cleanly") and says(ByMethod(), "records_cleanly")
    assert not says(NoByMethod(), "records_cleanly")


def test_a_model_with_a_block_that_does_not_say_stays_eager():
    """A block kind that inherits ``Part`` and says nothing about recording: the model answers no (it used to be an
    error when the step function was made)."""
    from pulse_infer_amd.models.causal_lm import CausalLM
    from pulse_infer_amd.models.spec import RunSpec
    from pulse_infer_amd.parts.base import EntryMeta, Part

    class Clean(Part):
        records_cleanly = True

    class Quiet(Part):
        pass

    class Spec:
        order = [RunSpec(0), RunSpec(1)]

    def model(blocks):
        m = object.__new__(CausalLM)
        m.spec, m.mode, m.blocks, m.positions, m._clean = Spec(), "bfloat16", blocks, {"p": Clean()}, None
        m.embedding = m.final_norm = m.head = Clean()
        return m

    entries = [EntryMeta("r", 0, 5, 1, 0)]
    assert model([Clean(), Clean()]).recordable(entries)
    assert not model([Clean(), Quiet()]).recordable(entries)
    assert not model([Clean(), Clean()]).recordable(entries * 65)            # more rows than its own products take
    m32 = model([Clean(), Clean()])
    m32.mode = "float32"
    assert not m32.recordable(entries)


def test_a_cache_spec_of_another_kind_goes_through_the_manager():
    """A spec class the manager has never heard of (one row of some width per token, in pages) gets a pool, block
    tables, window release and views like the built-in one: the manager asks the spec, it does not look at its type."""
    from dataclasses import dataclass

    made = {}

    @dataclass(frozen=True)
    class RowSpec:
        width: int
        window: int = None
        per_token = True

        def bytes_per_token(self, element_size):
            return self.width * element_size

        def allocate(self, runs, units, page_size, device, dtype):
            made[self] = (runs, units, page_size)
            return [[None] * units for _ in range(runs)]

        def view(self, storage, index, group, page_size, writable):
            return ("rows", storage[index], group, page_size, writable)

        def tensors(self, storage):
            return []

    kv, rows, win = PagedKVSpec(2, 16), RowSpec(24), RowSpec(24, window=6)
    m = CacheManager([kv, rows, None, win, rows, StateSpec((3,))], page_size=4, num_pages=8, max_requests=2)
    assert [g.spec for g in m.groups] == [kv, rows, win] and [g.runs for g in m.groups] == [[0], [1, 4], [3]]
    assert m.storage_bytes(2) == 8 * 4 * (2 * 2 * 16 * 2 + 2 * 24 * 2 + 24 * 2)
    m.groups[1].storage = rows.allocate(2, 8, 4, "cpu", None)
    m.groups[2].storage = win.allocate(1, 8, 4, "cpu", None)
    assert made[rows] == (2, 8, 4)
    assert m.view(4, writable=False) == ("rows", m.groups[1].storage[1], 1, 4, False) and m.view(2) is None
    m.add_request("a")
    m.reserve("a", 13)
    m.advance("a", 13)
    assert len(m.table(1, "a")) == 4 and m.table(2, "a")[:2] == [-1, -1]      # the window gave its first pages back
    m.check()
    m.free_request("a")
    assert all(g.pool.num_held == 0 for g in m.groups)
    with pytest.raises(TypeError, match="no cache spec"):
        CacheManager([object()], page_size=4, num_pages=2, max_requests=1)
