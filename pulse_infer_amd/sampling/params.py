"""How one request chooses its tokens.

The options and their meaning are the reference CLI sampler's
(reference: demo/qwen3_infer.cpp:230-423): temperature <= 0 is greedy; ``top_k``
> 0 keeps the k largest; ``top_p`` in (0, 1) keeps the most likely tokens up to
that mass; ``presence_penalty`` is subtracted from every token already in the
prompt or the output (the reference fixes 1.5, demo/qwen3_infer.cpp:469).
``seed`` makes the draws of this request reproducible whatever else is batched
with it (the reference seeds one generator from the system, :633-634).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 0.0
    presence_penalty: float = 0.0
    seed: Optional[int] = None
    ignore_eos: bool = False

    def __post_init__(self) -> None:
        if self.top_k < 0:
            raise ValueError(f"top_k must not be negative, got {self.top_k}")
        if not 0.0 <= self.top_p <= 1.0:
            raise ValueError(f"top_p must lie in [0, 1], got {self.top_p}")
        if self.presence_penalty < 0.0:
            raise ValueError(f"presence_penalty must not be negative, got {self.presence_penalty}")

    @property
    def greedy(self) -> bool:
        return not self.temperature > 0.0


_MASK = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform_for(seed: int, counter: int) -> float:
    """A number in [0, 1) that depends only on (seed, counter): the counter-th draw of a request."""
    z = _splitmix64(_splitmix64(seed & _MASK) ^ ((counter * 0xD1342543DE82EF95) & _MASK))
    return (z >> 40) / float(1 << 24)
