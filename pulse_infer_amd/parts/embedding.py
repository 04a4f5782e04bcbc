"""Token embedding and output head.

Embedding: row gather into the float32 residual (reference: src/layer/embedding.cpp:132-153).
Head: logits = n W^T in float32, for the wanted rows only; W is ``lm_head.weight`` when the
checkpoint holds it, else the embedding table when the configuration ties them
(reference: src/model/qwen3/model.cpp:1009-1021, :1322-1371).
"""
from __future__ import annotations

from typing import Any, Dict, List, Tuple

import torch

from ..ops import kernels
from ..weights.store import TensorSpec
from .base import EMBEDDINGS, HEADS, BuildContext, Part, StepCost
from .linear import Linear


@EMBEDDINGS.register("embedding")
class TokenEmbedding(Part):
    records_cleanly = True

    @classmethod
    def weight_specs(cls, params: Dict[str, Any]) -> Dict[str, TensorSpec]:
        return {params["name"]: TensorSpec((params["vocab_size"], params["hidden_size"]), kind="embedding",
                                           fan_in=params["hidden_size"])}

    @classmethod
    def step_cost(cls, params: Dict[str, Any], entries: List[Tuple[int, int]], weight_bytes: int,
                  cache_bytes: int) -> StepCost:
        """Only the gathered rows of the table are read."""
        rows = sum(count for _, count in entries)
        return StepCost(weight_bytes=float(rows) * params["hidden_size"] * weight_bytes)

    def __init__(self, params: Dict[str, Any], build: BuildContext):
        self.vocab = int(params["vocab_size"])
        self.hidden = int(params["hidden_size"])
        self.table = build.loader.get(params["name"])
        self.bad_id = torch.zeros(1, dtype=torch.int32, device=build.device)

    def forward(self, ids: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        """The step function checks ids on the host before it runs.  A caller that comes another way and brings an
        id outside the table gets a row of NaN, which reaches that token's logits (no token is chosen from them),
        never a silent row of zeros; ``saw_bad_id`` tells, at the price of a synchronisation."""
        kernels.embed_gather(ids, self.table, out, self.bad_id)
        return out

    def saw_bad_id(self, clear: bool = True) -> bool:
        seen = bool(self.bad_id.item())
        if seen and clear:
            self.bad_id.zero_()
        return seen


@HEADS.register("lm_head")
class OutputHead(Part):
    records_cleanly = True

    @classmethod
    def step_cost(cls, params: Dict[str, Any], entries: List[Tuple[int, int]], weight_bytes: int,
                  cache_bytes: int) -> StepCost:
        """The whole matrix (tied or its own) is read once; ``entries`` holds the wanted rows as one entry."""
        rows = sum(count for _, count in entries)
        size = float(params["vocab_size"]) * params["hidden_size"]
        return StepCost(flops=2.0 * rows * size, weight_bytes=size * weight_bytes)

    @classmethod
    def weight_specs(cls, params: Dict[str, Any]) -> Dict[str, TensorSpec]:
        # with tied embeddings the head's own tensor may be absent; if present it is used
        return {params["name"]: TensorSpec((params["vocab_size"], params["hidden_size"]), fan_in=params["hidden_size"],
                                           optional=bool(params.get("tied", False)))}

    def __init__(self, params: Dict[str, Any], build: BuildContext, embedding: TokenEmbedding):
        self.vocab = int(params["vocab_size"])
        if build.loader.has(params["name"]):
            weight = build.loader.get(params["name"])
        elif params.get("tied", False):
            weight = embedding.table
        else:
            raise KeyError(f"'{params['name']}' is missing and the configuration does not tie it to the embedding")
        self.linear = Linear(weight, build.mode)

    def forward(self, x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        """out: float32 [R, vocab]."""
        return self.linear.forward(x, out)
