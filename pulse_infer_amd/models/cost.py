"""What one step of a model costs, from its ``ModelSpec`` alone: arithmetic, the weights it has to read, and
what it reads of its caches.  Each part states its own share (``Part.step_cost``), so a model with another mixer
or feed-forward is priced by the same function; benchmarks build their rooflines on it.
"""
from __future__ import annotations

from typing import List, Tuple

from ..parts.base import BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, StepCost
from .spec import ModelSpec


def step_cost(spec: ModelSpec, entries: List[Tuple[int, int]], wanted: int, weight_bytes: int = 2,
              cache_bytes: int = 2) -> StepCost:
    """The cost of one step of ``entries`` = (tokens already in the cache, tokens of this step) per request, with
    logits wanted at ``wanted`` places.  ``weight_bytes`` / ``cache_bytes``: bytes of a stored element.

    Weights count once a step (every run of the order that names a layer again reads them again); the embedding
    table counts its gathered rows only; the head counts its whole matrix and the arithmetic of the wanted rows."""
    cost = EMBEDDINGS.get(spec.embedding.kind).step_cost(spec.embedding.params, entries, weight_bytes, cache_bytes)
    for run in spec.order:
        layer = spec.layers[run.layer]
        block = BLOCKS.get(layer.block.kind)
        mixer = MIXERS.get(layer.mixer.kind).step_cost(layer.mixer.params, entries, weight_bytes, cache_bytes)
        cost = cost + mixer
        cost = cost + FEED_FORWARDS.get(layer.ffn.kind).step_cost(layer.ffn.params, entries, weight_bytes, cache_bytes)
        for place in getattr(block, "NORM_PLACES", ()):
            norm = layer.norm(place)
            cost = cost + NORMS.get(norm.kind).step_cost(norm.params, entries, weight_bytes, cache_bytes)
    cost = cost + NORMS.get(spec.final_norm.kind).step_cost(spec.final_norm.params, [(0, wanted)], weight_bytes,
                                                             cache_bytes)
    return cost + HEADS.get(spec.head.kind).step_cost(spec.head.params, [(0, wanted)], weight_bytes, cache_bytes)
