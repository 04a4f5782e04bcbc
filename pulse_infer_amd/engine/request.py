"""One generation request and its life: WAITING -> RUNNING -> FINISHED, with a
detour through PREEMPTED when its pages were taken back.

Names and meanings follow the reference's ``InferenceRequest``
(reference: include/pulse/scheduler/inference_request.hpp:15-199): a request
holds its prompt and generated tokens and counts how many of them the model has
computed; while that count is below the prompt length it is in prefill, after
that exactly one token (the last sampled one) is pending per step.
"""
from __future__ import annotations

import enum
import time
from typing import List, Optional, Sequence

from ..sampling.params import SamplingParams


class RequestState(enum.Enum):
    WAITING = "waiting"
    RUNNING = "running"
    PREEMPTED = "preempted"
    FINISHED = "finished"


class InferenceRequest:
    def __init__(self, request_id: int, prompt_tokens: Sequence[int], max_new_tokens: int,
                 sampling: Optional[SamplingParams] = None):
        if len(prompt_tokens) == 0:
            raise ValueError("a request needs at least one prompt token")
        if max_new_tokens < 0:
            raise ValueError("max_new_tokens must not be negative")
        self.request_id = request_id
        self.prompt_tokens: List[int] = [int(t) for t in prompt_tokens]
        self.generated_tokens: List[int] = []
        self.max_new_tokens = int(max_new_tokens)
        self.sampling = sampling or SamplingParams()
        self.state = RequestState.WAITING
        self.num_computed_tokens = 0
        self.num_preemptions = 0
        self.finish_reason: Optional[str] = None
        self.arrival_time = time.monotonic()
        self.start_time: Optional[float] = None
        self.finish_time: Optional[float] = None

    # ----------------------------------------------------------------- queries
    @property
    def prompt_len(self) -> int:
        return len(self.prompt_tokens)

    @property
    def num_generated(self) -> int:
        return len(self.generated_tokens)

    @property
    def total_input_tokens(self) -> int:
        return self.prompt_len + self.num_generated

    @property
    def is_finished(self) -> bool:
        return self.state == RequestState.FINISHED

    @property
    def is_prefill(self) -> bool:
        return self.num_computed_tokens < self.prompt_len

    @property
    def has_pending_input(self) -> bool:
        return not self.is_finished and self.num_computed_tokens < self.total_input_tokens

    @property
    def can_generate_more(self) -> bool:
        return not self.is_finished and self.num_generated < self.max_new_tokens

    @property
    def num_pending_tokens(self) -> int:
        return 0 if self.is_finished else self.total_input_tokens - self.num_computed_tokens

    def token_at(self, index: int) -> int:
        return self.prompt_tokens[index] if index < self.prompt_len else self.generated_tokens[index - self.prompt_len]

    # ------------------------------------------------------------------ chunks
    def get_next_chunk_size(self, chunk_size: int = 256) -> int:
        """How many tokens the next step computes: a portion of what is pending, one token in plain decoding."""
        return max(0, min(int(chunk_size), self.num_pending_tokens))

    def get_next_chunk_tokens(self, chunk_size: int = 256) -> List[int]:
        n = self.get_next_chunk_size(chunk_size)
        start, end = self.num_computed_tokens, self.num_computed_tokens + n
        split = self.prompt_len    # prompt tokens, then generated ones (two slices, not a call a token)
        if end <= split:
            return self.prompt_tokens[start:end]
        if start >= split:
            return self.generated_tokens[start - split:end - split]
        return self.prompt_tokens[start:] + self.generated_tokens[:end - split]

    def get_next_chunk_positions(self, chunk_size: int = 256) -> List[int]:
        n = self.get_next_chunk_size(chunk_size)
        return list(range(self.num_computed_tokens, self.num_computed_tokens + n))

    # ------------------------------------------------------------- transitions
    def start_running(self) -> None:
        self.state = RequestState.RUNNING
        if self.start_time is None:
            self.start_time = time.monotonic()

    def finish(self, reason: str = "stopped") -> None:
        self.state = RequestState.FINISHED
        self.finish_reason = self.finish_reason or reason
        self.finish_time = time.monotonic()

    def preempt(self) -> None:
        """Its cache is gone: everything it holds is computed again when it runs next."""
        self.state = RequestState.PREEMPTED
        self.num_computed_tokens = 0
        self.num_preemptions += 1

    def add_computed_tokens(self, count: int) -> None:
        if count <= 0:
            raise ValueError("Computed token count must be positive")
        if self.is_finished:
            raise RuntimeError("Request already finished")
        if self.num_computed_tokens + count > self.total_input_tokens:
            raise ValueError("Computed token count exceeds available inputs")
        self.num_computed_tokens += count

    def add_sampled_token(self, token: int, eos_token_ids: Sequence[int]) -> bool:
        """Append a sampled token; False when the request is finished by it
        (end-of-sequence id, -1, or ``max_new_tokens`` reached)."""
        if self.is_finished:
            return False
        self.generated_tokens.append(int(token))
        if token == -1:
            self.finish("no_token")
        elif not self.sampling.ignore_eos and token in eos_token_ids:
            self.finish("eos")
        elif self.num_generated >= self.max_new_tokens:
            self.finish("length")
        return not self.is_finished
