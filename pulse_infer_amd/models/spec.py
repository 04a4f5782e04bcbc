"""An architecture written down as data.

A ``ModelSpec`` lists the layers of a decoder (each a choice of block
arrangement, mixer, feed-forward and norm, every one with its own sizes and
constants), the position encodings they refer to, and the order in which the
layers run.  The order is a list of ``RunSpec``: it may name a layer twice
(the weights are shared, each run has a cache of its own) or let a run read
the cache that an earlier run wrote.  Nothing in here knows which model it
describes; configuration classes produce it, ``CausalLM`` consumes it.
"""
from __future__ import annotations

from dataclasses import dataclass, field, replace
from typing import Any, Dict, List, Optional


@dataclass(frozen=True)
class PartSpec:
    """One part: the registered kind and the parameters it is built with."""

    kind: str
    params: Dict[str, Any] = field(default_factory=dict)

    def __hash__(self) -> int:  # params are small, flat dictionaries
        return hash((self.kind, tuple(sorted((k, repr(v)) for k, v in self.params.items()))))


@dataclass(frozen=True)
class LayerSpec:
    """One decoder layer: which parts it is made of and where its weights are.

    ``norms`` names a norm for every place the block arrangement has one ("mixer_norm" and "ffn_norm" for the
    pre-norm block; another arrangement may name more): each is a ``PartSpec`` of its own, so the norms of a layer
    may differ in kind and in constants.  The block's parameters say under which tensor prefix each of them loads.
    """

    prefix: str
    mixer: PartSpec
    ffn: PartSpec
    norms: Dict[str, PartSpec]
    block: PartSpec = field(default_factory=lambda: PartSpec("prenorm", {"mixer_norm": "input_layernorm",
                                                                         "ffn_norm": "post_attention_layernorm"}))

    def norm(self, place: str) -> PartSpec:
        try:
            return self.norms[place]
        except KeyError:
            raise KeyError(f"layer '{self.prefix}' names no norm for '{place}' (it has {sorted(self.norms)})") from None

    def with_parts(self, **changes: Any) -> "LayerSpec":
        """A copy with some of its fields replaced."""
        return replace(self, **changes)

    def __hash__(self) -> int:
        return hash((self.prefix, self.mixer, self.ffn, tuple(sorted(self.norms.items())), self.block))


@dataclass(frozen=True)
class RunSpec:
    """One entry of the execution order.

    ``layer`` indexes ``ModelSpec.layers``.  ``cache_of`` is the index (in the
    order) of an earlier run whose cache this run reads instead of owning one.
    """

    layer: int
    cache_of: Optional[int] = None


@dataclass
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    embedding: PartSpec
    layers: List[LayerSpec]
    order: List[RunSpec]
    final_norm: PartSpec
    head: PartSpec
    final_norm_prefix: str = "model.norm"
    # position encodings by name; mixers refer to them through params["position"]
    positions: Dict[str, PartSpec] = field(default_factory=dict)

    def validate(self) -> None:
        if not self.layers:
            raise ValueError("a model needs at least one layer")
        for index, run in enumerate(self.order):
            if not 0 <= run.layer < len(self.layers):
                raise ValueError(f"order[{index}] names layer {run.layer}, the model has {len(self.layers)}")
            if run.cache_of is not None:
                if not 0 <= run.cache_of < index:
                    raise ValueError(f"order[{index}].cache_of must name an earlier run, got {run.cache_of}")
                if self.order[run.cache_of].cache_of is not None:
                    raise ValueError(f"order[{index}].cache_of names run {run.cache_of}, which owns no cache")
