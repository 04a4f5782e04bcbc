"""The serving loop: scheduler -> step function -> sampler -> scheduler.

``ContinuousBatchEngine`` keeps the reference engine's interface
(reference: include/pulse/scheduler/continuous_batch_engine.hpp:14-35,
src/scheduler/continuous_batch_engine.cpp:66-305) with token ids in place of
text: ``add_request``, ``run_until_complete``, ``get_result``, ``get_request``,
``get_stats``.  ``LLM`` is the Python entry point on top of it.
"""
from __future__ import annotations

import time
from typing import Any, Dict, List, Optional, Sequence

import torch

from .. import log
from ..models.factory import build_model, load_model
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .request import InferenceRequest
from .runner import ModelRunner, StepEntry
from .scheduler import ContinuousBatchScheduler, ScheduledBatch, Stats

DEFAULT_MAX_SEQUENCES = 32  # reference: src/scheduler/continuous_batch_engine.cpp:73


class _InFlight:
    """A step that has been queued: who draws a token in it, where the tokens will be, and where they belong."""

    def __init__(self, batch: ScheduledBatch, sampled: list, live: list):
        self.batch, self.sampled, self.live = batch, sampled, live
        self.tokens: Optional[torch.Tensor] = None    # int32 on the device, one a drawing request
        self.rows: Dict[int, int] = {}                # request id -> its row of ``tokens``
        self.landing: Optional[torch.Tensor] = None   # pinned host memory the tokens are copied to
        self.landed: Optional[torch.cuda.Event] = None
        self.places: list = []                        # (request, index in its generated tokens, row)


class ContinuousBatchEngine:
    def __init__(self, model: Any, max_batch_size: int, chunk_size: int, *, page_size: int = 16,
                 num_pages: int = 1024, max_sequences: int = DEFAULT_MAX_SEQUENCES,
                 max_num_batched_tokens: Optional[int] = None, eos_token_ids: Sequence[int] = (),
                 banned_tokens: Optional[Sequence[int]] = None, seed: int = 0, extend_portions: bool = True):
        self.model = model
        slots = max(max_sequences, max_batch_size)
        self.runner = ModelRunner(model, page_size=page_size, num_pages=num_pages, max_requests=slots)
        self.scheduler = ContinuousBatchScheduler(
            max_batch_size, max_sequences, chunk_size, max_num_batched_tokens, cache=self.runner.cache,
            max_positions=model.spec.max_positions, extend_portions=extend_portions)
        self.sampler = Sampler(model.vocab_size, slots, model.device, banned_tokens)
        self.eos_token_ids = list(eos_token_ids)
        self.seed = int(seed)
        self.last_batch: Optional[ScheduledBatch] = None
        self._landing: List[Optional[torch.Tensor]] = [None, None]   # pinned buffers for a step's tokens, in turn
        self._turn = 0

    # ------------------------------------------------------------------ intake
    def add_request(self, prompt_tokens: Sequence[int], max_new_tokens: int,
                    sampling: Optional[SamplingParams] = None) -> int:
        vocab = self.model.vocab_size
        for tok in prompt_tokens:
            if not 0 <= int(tok) < vocab:
                raise ValueError(f"prompt token id {tok} is outside the vocabulary of {vocab}")
        return self.scheduler.add_request(prompt_tokens, max_new_tokens, sampling)

    def admit_as_computed(self, request_id: int, computed: int) -> None:
        """For measurements at a given context: the request is admitted at once and its first ``computed`` tokens count
        as computed, with whatever its pages hold for keys and values
        (``ContinuousBatchScheduler.admit_as_computed``).  What it generates means nothing."""
        self.scheduler.admit_as_computed(request_id, computed)
        request = self.scheduler.get_request(request_id)
        self.sampler.start_request(self.runner.cache.slot_of(request_id), request.sampling,
                                   request.prompt_tokens + request.generated_tokens)

    # -------------------------------------------------------------------- loop
    def step(self) -> ScheduledBatch:
        """One scheduling decision, one model step, one sampling call."""
        batch = self.scheduler.schedule_next_batch()
        self.last_batch = batch
        if batch.empty():
            return batch
        cache = self.runner.cache
        for request in batch.admitted:
            self.sampler.start_request(cache.slot_of(request.request_id), request.sampling,
                                       request.prompt_tokens + request.generated_tokens)
        entries = [StepEntry(p.request.request_id, p.tokens, [len(p.tokens) - 1] if p.samples else [])
                   for p in batch.portions]
        logits = self.runner.step(entries)
        self.scheduler.tokens_computed += batch.num_tokens()
        finished: List[int] = []
        sampled = [p for p in batch.portions if p.samples]
        for p in batch.portions:
            p.request.add_computed_tokens(len(p.tokens))
        live = []
        for row, p in enumerate(sampled):
            if not p.request.can_generate_more:  # nothing more to generate (max_new_tokens == 0)
                p.request.finish("length")
                finished.append(p.request.request_id)
            else:
                live.append((row, p.request))
        if live:
            rows = logits if len(live) == logits.shape[0] else logits[[r for r, _ in live]]
            requests = [q for _, q in live]
            tokens = self.sampler.sample(
                rows, [q.sampling for q in requests], [cache.slot_of(q.request_id) for q in requests],
                [q.num_generated for q in requests], [self.seed + q.request_id for q in requests])
            noted_slots, noted_tokens = [], []
            for q, tok in zip(requests, tokens):
                if q.sampling.presence_penalty > 0.0 and tok >= 0:
                    noted_slots.append(cache.slot_of(q.request_id))
                    noted_tokens.append(tok)
                if not q.add_sampled_token(tok, self.eos_token_ids):
                    finished.append(q.request_id)
            self.sampler.note_tokens(noted_slots, noted_tokens)
        self.scheduler.update_after_step(finished)
        return batch

    # ------------------------------------------------------- the loop, one step ahead
    # ``step`` leaves the GPU idle while the host takes a step's tokens, decides the next step and fills its arrays.
    # ``run_until_complete`` therefore runs one step ahead: step k is decided and queued while step k - 1 is still
    # computed, with the tokens of step k - 1 fed to it on the device, and only then are those tokens waited for.
    # What a step's tokens can change in the step after it is little: a request that drew an end-of-sequence id
    # (or had no token left to draw) has one token too many computed, which is dropped; that it ends by its length
    # is known without the token.  Every request draws what it draws with ``step``.
    def _launch(self, batch: ScheduledBatch, before: Optional["_InFlight"]) -> "_InFlight":
        """Queue a step and its sampling; nothing is waited for."""
        cache = self.runner.cache
        fed = before.rows if before is not None else {}
        for request in batch.admitted:
            slot = cache.slot_of(request.request_id)
            tokens = request.prompt_tokens + request.generated_tokens
            if request.request_id in fed:   # (preempted and admitted again at once: its last token is on the device)
                self.sampler.start_request(slot, request.sampling, tokens[:-1])
                if request.sampling.presence_penalty > 0.0:
                    row = fed[request.request_id]
                    self.sampler.note_on_device(self._ints([slot]), before.tokens[row:row + 1])
            else:
                self.sampler.start_request(slot, request.sampling, tokens)
        entries, places, rows, at = [], [], [], 0
        for p in batch.portions:
            entries.append(StepEntry(p.request.request_id, p.tokens, [len(p.tokens) - 1] if p.samples else []))
            at += len(p.tokens)
            if p.request.request_id in fed and p.start + len(p.tokens) == p.request.total_input_tokens:
                places.append(at - 1)       # the portion ends with the token that the step before drew
                rows.append(fed[p.request.request_id])
        logits = self.runner.step(entries, feed=(before.tokens, places, rows) if places else None)
        self.scheduler.tokens_computed += batch.num_tokens()
        sampled = [p for p in batch.portions if p.samples]
        live = [(row, p.request) for row, p in enumerate(sampled) if p.request.can_generate_more]
        flight = _InFlight(batch, sampled, live)
        if live:
            picked = logits if len(live) == logits.shape[0] else logits[[r for r, _ in live]]
            requests = [q for _, q in live]
            slots = [cache.slot_of(q.request_id) for q in requests]
            flight.tokens = self.sampler.launch(
                picked, [q.sampling for q in requests], slots, [q.num_generated for q in requests],
                [self.seed + q.request_id for q in requests])
            if any(q.sampling.presence_penalty > 0.0 for q in requests):
                self.sampler.note_on_device(
                    self._ints([s if q.sampling.presence_penalty > 0.0 else -1 for s, q in zip(slots, requests)]),
                    flight.tokens)
            flight.rows = {q.request_id: i for i, q in enumerate(requests)}
            turn = self._turn = 1 - self._turn
            if self._landing[turn] is None or self._landing[turn].numel() < len(live):
                self._landing[turn] = torch.empty(max(64, len(live)), dtype=torch.int32, pin_memory=True)
            flight.landing = self._landing[turn][:len(live)]
            flight.landing.copy_(flight.tokens, non_blocking=True)
            flight.landed = torch.cuda.Event()
            flight.landed.record()
        return flight

    def _ints(self, values: List[int]) -> torch.Tensor:
        return self.runner._staging.upload_values(values)

    def _assume(self, flight: "_InFlight") -> None:
        """What a queued step does to its requests as far as it is known without its tokens: the cursors move,
        every drawing request has one token more (its value follows), and who reaches its length ends."""
        finished: List[int] = []
        for p in flight.batch.portions:
            if not p.request.is_finished:      # (ended meanwhile by the token it drew in the step before)
                p.request.add_computed_tokens(len(p.tokens))
        drawing = {id(q) for _, q in flight.live}
        for p in flight.sampled:
            if id(p.request) not in drawing and not p.request.is_finished:   # nothing more to generate
                p.request.finish("length")
                finished.append(p.request.request_id)
        for row, (_, q) in enumerate(flight.live):
            if q.is_finished:
                continue
            if not q.add_sampled_token(0, ()):      # (any valid id holds the place)
                finished.append(q.request_id)
            flight.places.append((q, len(q.generated_tokens) - 1, row))
        self.scheduler.update_after_step(finished)

    def _settle(self, flight: "_InFlight") -> None:
        """The tokens of a step have arrived: they take their places, and who drew an end ends."""
        if flight.landed is None:
            return
        flight.landed.synchronize()
        tokens = flight.landing.tolist()
        finished: List[int] = []
        for q, index, row in flight.places:
            tok = tokens[row]
            q.generated_tokens[index] = tok
            reason = None
            if tok == -1:
                reason = "no_token"
            elif tok in self.eos_token_ids and not q.sampling.ignore_eos:
                reason = "eos"
            if reason is None:
                continue
            if q.is_finished:
                q.finish_reason = reason     # it reached its length with this token; the token's reason comes first
            else:
                q.finish(reason)
                finished.append(q.request_id)
        if finished:
            self.scheduler.update_after_step(finished, count_step=False)

    def run_until_complete(self, print_progress: bool = False, one_step_ahead: bool = True,
                           max_steps: Optional[int] = None) -> int:
        """Run until every request has finished, or for ``max_steps`` steps (all of them waited for when it returns;
        what remains goes on with the next call).  Returns the number of steps run."""
        step = 0
        flight: Optional[_InFlight] = None
        try:
            while True:
                if step % 10 == 0 and self.scheduler.has_work() and (print_progress or log.enabled("debug")):
                    s = self.scheduler.get_stats()
                    (log.info if print_progress else log.debug)(
                        f"step {step}: {s.num_running} requests running, {s.num_waiting} waiting, "
                        f"{s.num_finished} finished")
                more = max_steps is None or step < max_steps
                if not one_step_ahead:
                    if not more or not self.scheduler.has_work() or self.step().empty():
                        break
                    step += 1
                    continue
                batch = self.scheduler.schedule_next_batch() if more and self.scheduler.has_work() else None
                self.last_batch = batch if batch is not None else self.last_batch
                queued = self._launch(batch, flight) if batch is not None and not batch.empty() else None
                if flight is not None:
                    settling, flight = flight, None
                    self._settle(settling)
                if queued is None:     # nothing left, or nothing that can be scheduled (as ``step`` returning an empty batch)
                    break
                self._assume(queued)
                flight = queued
                step += 1
        finally:
            # Only an error leaves a step in flight here (the scheduler's, a kernel's, an interrupt, between the step's
            # launch and the arrival of its tokens): the tokens are still taken, so that no request keeps a
            # place-holder for a token, or a finish reason that only the place-holder gave it.
            if flight is not None:
                try:
                    self._settle(flight)
                except Exception:      # (the device may be what failed; the error under way says more than this one)
                    pass
        if print_progress or log.enabled("debug"):
            s = self.scheduler.get_stats()
            (log.info if print_progress else log.debug)(
                f"{s.num_finished} of {s.total_requests} requests finished after {step} steps "
                f"({s.num_preemptions} preemptions, {self.runner.graph_records} steps recorded, "
                f"{self.runner.graph_replays} replayed)")
        return step

    # ----------------------------------------------------------------- results
    def get_result(self, request_id: int) -> List[int]:
        """The generated ids of a finished request, cut before the first end-of-sequence id
        (reference: src/scheduler/continuous_batch_engine.cpp:114-130); empty while it still runs."""
        request = self.scheduler.get_request(request_id)
        if request is None or not request.is_finished:
            return []
        out: List[int] = []
        for tok in request.generated_tokens:
            if not request.sampling.ignore_eos and tok in self.eos_token_ids:
                break
            out.append(tok)
        return out

    def get_request(self, request_id: int) -> Optional[InferenceRequest]:
        return self.scheduler.get_request(request_id)

    def get_stats(self) -> Stats:
        return self.scheduler.get_stats()


class LLM:
    """Python entry point: a model folder in, generated token ids out."""

    def __init__(self, model: Any, config: Any = None, *, max_batch_size: int = 8, chunk_size: int = 256,
                 page_size: int = 16, num_pages: Optional[int] = None, max_sequences: int = DEFAULT_MAX_SEQUENCES,
                 max_num_batched_tokens: Optional[int] = None, seed: int = 0, extend_portions: bool = True):
        self.model = model
        self.config = config
        if num_pages is None:
            # room for max_sequences contexts of up to 4096 tokens, bounded by the model's positions
            per_request = min(model.spec.max_positions, 4096)
            num_pages = max(64, max_sequences * ((per_request + page_size - 1) // page_size))
        eos = list(getattr(config, "eos_token_ids", []) or [])
        self.engine = ContinuousBatchEngine(
            model, max_batch_size, chunk_size, page_size=page_size, num_pages=num_pages, max_sequences=max_sequences,
            max_num_batched_tokens=max_num_batched_tokens, eos_token_ids=eos, seed=seed,
            extend_portions=extend_portions)

    @classmethod
    def from_pretrained(cls, model_dir: str, dtype: str = "bfloat16", device: str = "cuda:0",
                        config_overrides: Optional[Dict[str, Any]] = None, strict: bool = False, **engine_options):
        """``strict``: a tensor in the folder that no part of the model asks for is an error (else a warning)."""
        config, model = load_model(model_dir, mode=dtype, device=device, config_overrides=config_overrides,
                                   strict=strict)
        return cls(model, config, **engine_options)

    @classmethod
    def from_config_random(cls, config: Any, weights_seed: int = 0, init: Any = "fan_in", dtype: str = "bfloat16",
                           device: str = "cuda:0", **engine_options):
        """Random weights made on the GPU, without a file (for sizes not worth writing to disk)."""
        from ..models.causal_lm import expected_tensors
        from ..weights.random_init import RandomSource

        source = RandomSource(expected_tensors(config.model_spec()), weights_seed, init, torch.bfloat16, device=device)
        model = build_model(config, source, mode=dtype, device=device)
        return cls(model, config, **engine_options)

    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int = 32, temperature: float = 0.0,
                 top_k: int = 0, top_p: float = 0.0, presence_penalty: float = 0.0, seed: Optional[int] = None,
                 ignore_eos: bool = False, sampling: Optional[Sequence[SamplingParams]] = None) -> List[List[int]]:
        ids = []
        for i, prompt in enumerate(prompts):
            params = sampling[i] if sampling is not None else SamplingParams(
                temperature=temperature, top_k=top_k, top_p=top_p, presence_penalty=presence_penalty,
                seed=None if seed is None else seed + i, ignore_eos=ignore_eos)
            ids.append(self.engine.add_request(prompt, max_new_tokens, params))
        self.engine.run_until_complete()
        return [self.engine.get_result(i) for i in ids]

    def step_raw(self, entries: Sequence[Dict[str, Any]], end: Sequence[Any] = ()) -> torch.Tensor:
        """Run one step of given tokens: entries are {"id", "tokens", "want"}; float32 logits [wanted, vocab]."""
        runner = self.engine.runner
        batch = []
        for item in entries:
            rid = ("raw", item["id"])
            if not runner.cache.has_request(rid):
                runner.add_request(rid)
            runner.reserve(rid, runner.cache.computed(rid) + len(item["tokens"]))
            batch.append(StepEntry(rid, list(item["tokens"]), list(item.get("want", []))))
        logits = runner.step(batch)
        for rid in end:
            runner.free_request(("raw", rid))
        return logits
