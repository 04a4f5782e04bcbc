"""Continuous batching with chunked prefill under a token budget.

The queues and the first-come-first-served admission are the reference's
(reference: include/pulse/scheduler/continuous_batch_scheduler.hpp:27-147):
every step takes all running requests, then admits waiting ones while the batch
has room (``max_batch_size`` requests) and fewer than ``max_sequences`` run.
What the reference leaves out is decided here:

* **token budget** — a step computes at most ``max_num_batched_tokens`` tokens:
  decoding requests come first with one token each, what is left goes to
  prefilling requests in order of arrival, each at most ``chunk_size`` tokens,
  cut anywhere; if budget is left when every one of them has its portion, the
  portions are extended in the same order (a lone long prompt runs in steps
  of the whole budget) unless ``extend_portions`` is off, which keeps every
  portion at ``chunk_size`` tokens at most, as the reference's are.
* **pages** — every portion is reserved in the cache before the step; a request
  is admitted only if its first portion fits.  When a running request cannot
  get the page it needs, the most recently admitted running request is
  preempted: its pages and slot are given back, it returns to the front of the
  waiting queue and is later computed again from its first token (prompt and
  generated tokens alike), which reproduces what it had.  A prefill portion is
  shortened rather than preempting anyone; only when every running request is
  still in its prompt and none can get a page (they hold each other's) does the
  newest give way too.  A request that could never fit the pool or the model's
  positions is refused at ``add_request``.
  (The reference aborts the whole run when pages run out,
  src/runtime/block_manager.cpp:44-46, src/scheduler/continuous_batch_engine.cpp:98-101.)
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Sequence

from .. import log
from ..cache.manager import CacheManager
from ..sampling.params import SamplingParams
from .request import InferenceRequest, RequestState


class SchedulerError(RuntimeError):
    pass


@dataclass
class ScheduledPortion:
    request: InferenceRequest
    tokens: List[int]
    start: int
    samples: bool  # the portion ends the request's pending input: its last row is sampled from


@dataclass
class ScheduledBatch:
    portions: List[ScheduledPortion] = field(default_factory=list)
    preempted: List[InferenceRequest] = field(default_factory=list)
    admitted: List[InferenceRequest] = field(default_factory=list)

    @property
    def requests(self) -> List[InferenceRequest]:
        return [p.request for p in self.portions]

    def batch_size(self) -> int:
        return len(self.portions)

    def num_tokens(self) -> int:
        return sum(len(p.tokens) for p in self.portions)

    def empty(self) -> bool:
        return not self.portions


@dataclass
class Stats:
    num_running: int = 0
    num_waiting: int = 0
    num_finished: int = 0
    total_requests: int = 0
    num_steps: int = 0
    num_preemptions: int = 0
    tokens_computed: int = 0
    tokens_generated: int = 0
    pages_high_water: int = 0


class ContinuousBatchScheduler:
    def __init__(self, max_batch_size: int, max_sequences: int, chunk_size: int = 256,
                 max_num_batched_tokens: Optional[int] = None, cache: Optional[CacheManager] = None,
                 max_positions: Optional[int] = None, extend_portions: bool = True):
        """``chunk_size`` is what the reference calls so (every prompt gets a portion of that many tokens in every
        step, continuous_batch_scheduler.hpp:27-147) as long as ``extend_portions`` is off.  With it on (the default)
        ``chunk_size`` is a portion's share of a step when several prompts want one: what the step's budget
        (``max_num_batched_tokens``, by default ``max_batch_size`` chunks) still has when every prompt has its share
        goes to the same portions in order, so a prompt that has a step to itself runs in portions of the whole
        budget."""
        if max_batch_size <= 0 or max_sequences <= 0 or chunk_size <= 0:
            raise ValueError("max_batch_size, max_sequences and chunk_size must be positive")
        self.max_batch_size = int(max_batch_size)
        self.max_sequences = int(max_sequences)
        self.chunk_size = int(chunk_size)
        self.max_num_batched_tokens = int(max_num_batched_tokens) if max_num_batched_tokens else \
            self.max_batch_size * self.chunk_size
        if self.max_num_batched_tokens <= 0:
            raise ValueError("max_num_batched_tokens must be positive")
        self.cache = cache
        self.max_positions = max_positions
        self.extend_portions = bool(extend_portions)
        self.next_request_id = 0
        self.waiting: Deque[InferenceRequest] = deque()
        self.running: List[InferenceRequest] = []
        self.request_map: Dict[int, InferenceRequest] = {}
        self.num_steps = 0
        self.num_preemptions = 0
        self.tokens_computed = 0

    # ------------------------------------------------------------------ intake
    def add_request(self, prompt_tokens: Sequence[int], max_new_tokens: int,
                    sampling: Optional[SamplingParams] = None) -> int:
        request = InferenceRequest(self.next_request_id, prompt_tokens, max_new_tokens, sampling)
        # the last sampled token is never fed back, so a request holds at most prompt + max_new - 1 tokens
        longest = request.prompt_len + max(0, request.max_new_tokens - 1)
        if self.max_positions is not None and longest > self.max_positions:
            raise SchedulerError(f"request needs {longest} positions, the model allows {self.max_positions}")
        if self.cache is not None:
            for g, need in zip(self.cache.groups, self.cache.pages_needed_new(longest)):
                if g.window is None and need > g.pool.num_pages:
                    raise SchedulerError(f"request needs {need} cache pages of {g.page_size} tokens, "
                                         f"the pool has {g.pool.num_pages}")
        self.next_request_id += 1
        self.waiting.append(request)
        self.request_map[request.request_id] = request
        return request.request_id

    def admit_as_computed(self, request_id: int, computed: int) -> None:
        """Admit a waiting request at once and let the first ``computed`` tokens of its stream count as computed: pages
        are reserved for them and the cursor stands behind them, but no step has run them, so their keys and values are
        whatever the pages hold.  For measurements at a given context (a decode step does the same work over a cache
        that only looks computed); never for requests whose output matters."""
        request = self.request_map[request_id]
        if request not in self.waiting or request.num_computed_tokens != 0:
            raise SchedulerError(f"request {request_id} is not waiting at its start")
        if not 0 < computed < request.total_input_tokens:
            raise SchedulerError(f"request {request_id}: {computed} tokens cannot count as computed, it has "
                                 f"{request.total_input_tokens} and must run one at least")
        if len(self.running) >= self.max_sequences:
            raise SchedulerError(f"{self.max_sequences} requests are running already")
        self.waiting.remove(request)
        if self.cache is not None:
            self.cache.add_request(request_id)
            self.cache.reserve(request_id, computed)
            self.cache.advance(request_id, computed)
        request.start_running()
        request.num_computed_tokens = computed
        self.running.append(request)

    # --------------------------------------------------------------- decisions
    def _fits(self, request: InferenceRequest, length: int) -> bool:
        return self.cache is None or self.cache.can_reserve(
            request.request_id if self.cache.has_request(request.request_id) else None, length)

    def _reserve(self, request: InferenceRequest, length: int) -> None:
        if self.cache is not None:
            self.cache.reserve(request.request_id, length)

    def _largest_fitting(self, request: InferenceRequest, want: int) -> int:
        """The longest portion <= want whose pages are free right now."""
        if self.cache is None:
            return want
        base = request.num_computed_tokens
        lo, hi = 0, want
        while lo < hi:  # can_reserve is monotone in the length
            mid = (lo + hi + 1) // 2
            if self._fits(request, base + mid):
                lo = mid
            else:
                hi = mid - 1
        return lo

    def _preempt(self, victim: InferenceRequest, batch: ScheduledBatch) -> None:
        log.debug(f"request {victim.request_id} gives its pages back after {victim.num_computed_tokens} tokens "
                  f"(preemption {self.num_preemptions + 1})")
        self.running.remove(victim)
        if self.cache is not None and self.cache.has_request(victim.request_id):
            self.cache.free_request(victim.request_id)
        victim.preempt()
        self.waiting.appendleft(victim)
        batch.preempted.append(victim)
        batch.portions = [p for p in batch.portions if p.request is not victim]
        self.num_preemptions += 1

    def schedule_next_batch(self) -> ScheduledBatch:
        batch = ScheduledBatch()
        while True:
            self._fill(batch)
            if not batch.empty() or not (self.running or self.waiting):
                return batch
            if len(self.running) > 1:
                # every running request waits for pages that the others hold (all of them still in their prompts):
                # the newest gives way, as when a decoding request needs a page
                self._preempt(self.running[-1], batch)
                continue
            raise SchedulerError("nothing can be scheduled although requests remain: the cache pool cannot hold "
                                 "the first portion of the next request")

    def _fill(self, batch: ScheduledBatch) -> None:
        """One pass of the three phases, adding to ``batch``."""
        budget = self.max_num_batched_tokens
        # who decodes and who is in a prompt (or is being recomputed), looked at once: in order of admission
        decoding: List[InferenceRequest] = []
        prompting: List[InferenceRequest] = []
        for request in self.running:
            pending = request.num_pending_tokens
            if pending == 1 and not request.is_prefill:
                decoding.append(request)
            elif pending >= 1:
                prompting.append(request)

        # 1. running requests that decode: one token each, preempting the newest when pages run out
        for request in decoding:
            if request.state is not RequestState.RUNNING:  # preempted a moment ago
                continue
            if budget <= 0 or batch.batch_size() >= self.max_batch_size:
                break
            need = request.num_computed_tokens + 1
            gives_way = False
            while not self._fits(request, need):
                victim = self.running[-1]
                if victim is request:
                    if len(self.running) == 1:
                        raise SchedulerError(f"request {request.request_id} cannot get a cache page although "
                                             "nothing else is running; the pool is too small for it")
                    gives_way = True  # it is the newest itself
                    break
                self._preempt(victim, batch)
            if gives_way:
                self._preempt(request, batch)
                continue
            self._reserve(request, need)
            batch.portions.append(ScheduledPortion(request, request.get_next_chunk_tokens(1),
                                                   request.num_computed_tokens, True))
            budget -= 1

        # 2. running requests with more than one pending token (prefill, or recomputation after preemption)
        for request in prompting:
            if request.state is not RequestState.RUNNING:
                continue
            if budget <= 0 or batch.batch_size() >= self.max_batch_size:
                break
            want = min(self.chunk_size, request.num_pending_tokens, budget)
            count = self._largest_fitting(request, want)
            if count <= 0:
                continue
            self._reserve(request, request.num_computed_tokens + count)
            batch.portions.append(ScheduledPortion(request, request.get_next_chunk_tokens(count),
                                                   request.num_computed_tokens,
                                                   count == request.num_pending_tokens))
            budget -= count

        # 3. admit waiting requests, first come first served
        while (self.waiting and budget > 0 and batch.batch_size() < self.max_batch_size
               and len(self.running) < self.max_sequences):
            request = self.waiting[0]
            if self.cache is not None and self.cache.slots.num_free == 0:
                break
            want = min(self.chunk_size, request.num_pending_tokens, budget)
            count = self._largest_fitting(request, want)
            # admit only with room for the whole first portion (or all that the budget allows)
            if count < want:
                break
            self.waiting.popleft()
            if self.cache is not None:
                self.cache.add_request(request.request_id)
            request.start_running()
            self.running.append(request)
            batch.admitted.append(request)
            self._reserve(request, request.num_computed_tokens + count)
            batch.portions.append(ScheduledPortion(request, request.get_next_chunk_tokens(count),
                                                   request.num_computed_tokens,
                                                   count == request.num_pending_tokens))
            budget -= count

        # 4. what is left of the budget (fewer requests in their prompts than it has room for) extends this step's
        #    prompt portions, in their order: a lone long prompt then runs in steps of the whole budget, whose
        #    matrix products are far more efficient than those of a chunk's rows
        for i, portion in enumerate(batch.portions if self.extend_portions else ()):
            if budget <= 0:
                break
            if portion.samples:   # it brings all that its request has pending
                continue
            request, have = portion.request, len(portion.tokens)
            more = min(request.num_pending_tokens - have, budget)
            if more <= 0:
                continue
            count = self._largest_fitting(request, have + more)
            if count <= have:
                continue
            self._reserve(request, request.num_computed_tokens + count)
            batch.portions[i] = ScheduledPortion(request, request.get_next_chunk_tokens(count),
                                                 request.num_computed_tokens, count == request.num_pending_tokens)
            budget -= count - have

    def update_after_step(self, finished_ids: Sequence[int], count_step: bool = True) -> None:
        """Take finished requests out of the running list and give their cache back
        (reference: continuous_batch_scheduler.hpp:75-89).  ``count_step`` False: requests whose end became known
        after the step had been counted (a loop that learns a step's tokens while the next step runs); such a
        request may have been preempted meanwhile and wait in the queue, from which it is taken too."""
        if count_step:
            self.num_steps += 1
        for request_id in finished_ids:
            request = self.request_map.get(request_id)
            if request is None:
                continue
            if request in self.running:
                self.running.remove(request)
            elif request in self.waiting:
                self.waiting.remove(request)
            else:
                continue
            if not request.is_finished:
                request.finish()
            if self.cache is not None and self.cache.has_request(request_id):
                self.cache.free_request(request_id)

    # ----------------------------------------------------------------- queries
    def get_request(self, request_id: int) -> Optional[InferenceRequest]:
        return self.request_map.get(request_id)

    def has_work(self) -> bool:
        return bool(self.running) or bool(self.waiting)

    def num_running(self) -> int:
        return len(self.running)

    def num_active_sequences(self) -> int:
        return len(self.running)

    def num_waiting(self) -> int:
        return len(self.waiting)

    def set_chunk_size(self, chunk_size: int) -> None:
        self.chunk_size = int(chunk_size)

    def get_stats(self) -> Stats:
        finished = [r for r in self.request_map.values() if r.is_finished]
        return Stats(
            num_running=len(self.running), num_waiting=len(self.waiting), num_finished=len(finished),
            total_requests=len(self.request_map), num_steps=self.num_steps, num_preemptions=self.num_preemptions,
            tokens_computed=self.tokens_computed,
            tokens_generated=sum(r.num_generated for r in self.request_map.values()),
            pages_high_water=max((g.pool.high_water for g in self.cache.groups), default=0) if self.cache else 0)
