"""One generation request: a growing token stream and a cursor into it.

The stream is the prompt followed by the tokens sampled so far; the cursor
(``num_computed_tokens``) says how much of it the model has run, i.e. how many
keys of the request are in the cache.  Everything the scheduler asks follows
from those two: what is pending is ``stream[cursor:]``, the request is in its
prompt while the cursor lies inside the prompt, and in plain decoding exactly
one token (the last sampled one) is pending.  Preemption moves the cursor back
to zero; the stream stays, so recomputation reproduces the same cache.

Life: WAITING -> RUNNING -> FINISHED, with a detour through PREEMPTED when its
pages were taken back.  The public names are those of the reference's request
object, which the scheduler and the engine's callers use
(reference: include/pulse/scheduler/inference_request.hpp:15-199); PREEMPTED,
``finish_reason``, ``num_preemptions`` and portions that cross from the prompt
into generated tokens are this engine's.
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
        self.sampling = sampling or SamplingParams()
        self.max_new_tokens = int(max_new_tokens)
        # the stream and the cursor
        self.prompt_tokens: List[int] = [int(t) for t in prompt_tokens]
        self.generated_tokens: List[int] = []
        self.num_computed_tokens = 0
        # life
        self.state = RequestState.WAITING
        self.finish_reason: Optional[str] = None
        self.num_preemptions = 0
        self.arrival_time = time.monotonic()
        self.start_time: Optional[float] = None
        self.finish_time: Optional[float] = None

    # ------------------------------------------------------------ the stream
    @property
    def prompt_len(self) -> int:
        return len(self.prompt_tokens)

    @property
    def num_generated(self) -> int:
        return len(self.generated_tokens)

    @property
    def total_input_tokens(self) -> int:
        """Length of the stream: every token that is, or will be, an input of the model."""
        return len(self.prompt_tokens) + len(self.generated_tokens)

    def token_at(self, index: int) -> int:
        split = len(self.prompt_tokens)
        return self.prompt_tokens[index] if index < split else self.generated_tokens[index - split]

    def _stream(self, start: int, end: int) -> List[int]:
        """stream[start:end] as at most two slices (the prompt's part, the generated part)."""
        split = len(self.prompt_tokens)
        if end <= split:
            return self.prompt_tokens[start:end]
        if start >= split:
            return self.generated_tokens[start - split:end - split]
        return self.prompt_tokens[start:] + self.generated_tokens[:end - split]

    # ------------------------------------------------------------ the cursor
    @property
    def num_pending_tokens(self) -> int:
        return 0 if self.is_finished else self.total_input_tokens - self.num_computed_tokens

    @property
    def has_pending_input(self) -> bool:
        return self.num_pending_tokens > 0

    @property
    def is_prefill(self) -> bool:
        return self.num_computed_tokens < len(self.prompt_tokens)

    def get_next_chunk_size(self, chunk_size: int = 256) -> int:
        """Tokens the next step runs: what is pending, at most ``chunk_size`` (one token in plain decoding)."""
        return max(0, min(int(chunk_size), self.num_pending_tokens))

    def get_next_chunk_tokens(self, chunk_size: int = 256) -> List[int]:
        at = self.num_computed_tokens
        return self._stream(at, at + self.get_next_chunk_size(chunk_size))

    def get_next_chunk_positions(self, chunk_size: int = 256) -> List[int]:
        at = self.num_computed_tokens
        return list(range(at, at + self.get_next_chunk_size(chunk_size)))

    def add_computed_tokens(self, count: int) -> None:
        """Move the cursor over ``count`` tokens that a step has just run."""
        if self.is_finished:
            raise RuntimeError(f"request {self.request_id} is finished; no step can have run tokens of it")
        pending = self.total_input_tokens - self.num_computed_tokens
        if not 0 < count <= pending:
            raise ValueError(f"request {self.request_id}: a step ran {count} tokens, between 1 and the {pending} "
                             f"pending ones were possible")
        self.num_computed_tokens += count

    # --------------------------------------------------------------- sampling
    @property
    def can_generate_more(self) -> bool:
        return not self.is_finished and len(self.generated_tokens) < self.max_new_tokens

    def add_sampled_token(self, token: int, eos_token_ids: Sequence[int]) -> bool:
        """Append a sampled token to the stream; False when that token ends the request: -1 (no token was
        allowed), an end-of-sequence id (kept in the stream, cut from the result later), or the last of
        ``max_new_tokens``.  A finished request takes no token."""
        if self.is_finished:
            return False
        self.generated_tokens.append(int(token))
        reason = None
        if token == -1:
            reason = "no_token"
        elif token in eos_token_ids and not self.sampling.ignore_eos:
            reason = "eos"
        elif len(self.generated_tokens) >= self.max_new_tokens:
            reason = "length"
        if reason is None:
            return True
        self.finish(reason)
        return False

    # ------------------------------------------------------------------- life
    @property
    def is_finished(self) -> bool:
        return self.state is RequestState.FINISHED

    def start_running(self) -> None:
        self.state = RequestState.RUNNING
        if self.start_time is None:
            self.start_time = time.monotonic()

    def preempt(self) -> None:
        """Its cache is gone: the cursor goes back to the start, and the whole stream is run again later."""
        self.state = RequestState.PREEMPTED
        self.num_computed_tokens = 0
        self.num_preemptions += 1

    def finish(self, reason: str = "stopped") -> None:
        self.state = RequestState.FINISHED
        if self.finish_reason is None:
            self.finish_reason = reason
        self.finish_time = time.monotonic()
