"""A decoder-only language model assembled from a ``ModelSpec``.

It owns the parts (embedding, one block per layer, final norm, head, position
encodings) and runs them in the spec's order for one step: embedding of the
step's tokens, every run of the order over the same float32 residual, final
norm on the rows whose logits are wanted only, and the head in float32
(reference flow: src/model/qwen3/model.cpp:1283-1371, which computes the head on
all rows in the model's storage type).
"""
from __future__ import annotations

from typing import Any, Dict, List, Optional

import torch

from ..parts.base import (BLOCKS, EMBEDDINGS, HEADS, NORMS, POSITIONS, BuildContext, EntryMeta, ResidualStream,
                          StepContext, Workspace, joined, says)
from ..weights.store import TensorSpec, WeightLoader
from .spec import ModelSpec

ACT_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def expected_tensors(spec: ModelSpec) -> Dict[str, TensorSpec]:
    """Every tensor the model loads, by checkpoint name."""
    out: Dict[str, TensorSpec] = {}
    out.update(EMBEDDINGS.get(spec.embedding.kind).weight_specs(spec.embedding.params))
    for layer in spec.layers:
        out.update(BLOCKS.get(layer.block.kind).layer_weight_specs(layer))
    for name, ts in NORMS.get(spec.final_norm.kind).weight_specs(spec.final_norm.params).items():
        out[joined(spec.final_norm_prefix, name)] = ts
    for name, ts in HEADS.get(spec.head.kind).weight_specs(spec.head.params).items():
        out.setdefault(name, ts)
    return out


class CausalLM:
    def __init__(self, spec: ModelSpec, source: Any, mode: str = "bfloat16", device: Any = "cuda:0",
                 strict: bool = False, options: Optional[Dict[str, Any]] = None):
        if mode not in ACT_DTYPES:
            raise ValueError(f"unknown run dtype '{mode}', choose from {sorted(ACT_DTYPES)}")
        spec.validate()
        self.spec = spec
        self.mode = mode
        self.device = torch.device(device)
        self.act_dtype = ACT_DTYPES[mode]
        self.workspace = Workspace(self.device)
        self.options = dict(options or {})
        loader = WeightLoader(source, expected_tensors(spec), mode, self.device, strict=strict)
        build = BuildContext(loader=loader, mode=mode, device=self.device, act_dtype=self.act_dtype,
                             workspace=self.workspace, options=dict(options or {}))
        for name, part in spec.positions.items():
            params = dict(part.params)
            params.setdefault("name", name)
            build.positions[name] = POSITIONS.get(part.kind)(params, build)
        self.positions = build.positions
        self.embedding = EMBEDDINGS.get(spec.embedding.kind)(spec.embedding.params, build)
        self.blocks = [BLOCKS.get(layer.block.kind)(layer, build) for layer in spec.layers]
        self.final_norm = NORMS.get(spec.final_norm.kind)(spec.final_norm.params, spec.final_norm_prefix, build)
        self.head = HEADS.get(spec.head.kind)(spec.head.params, build, self.embedding)
        self.vocab_size = spec.vocab_size
        self.hidden_size = spec.hidden_size
        self._clean: Optional[bool] = None

    # ------------------------------------------------------------------- caches
    def run_cache_specs(self) -> List[Any]:
        """Per run of the order: the cache spec it owns (None when it owns none)."""
        out = []
        for run in self.spec.order:
            out.append(None if run.cache_of is not None else self.blocks[run.layer].cache_spec())
        return out

    # ---------------------------------------------------------------- recording
    MAX_RECORDED_ROWS = 64      # up to here every product of a step of single tokens can be this package's own kernel;
                                # a shape whose step does call the vendor library (seen when it is first run for
                                # recording) stays eager

    def records_cleanly(self) -> bool:
        """Whether every part of the model says that its launches do not depend on a step's values
        (``Part.records_cleanly``, an attribute or a method)."""
        if self._clean is None:
            parts: List[Any] = [self.embedding, self.final_norm, self.head]
            parts += [self.blocks[run.layer] for run in self.spec.order]
            parts += list(self.positions.values())
            self._clean = all(says(part, "records_cleanly") for part in parts)
        return self._clean

    def recordable(self, entries: List[EntryMeta]) -> bool:
        """Whether a step of these entries (one token each, every one wanting its logits: the form the step function
        can replay) may be recorded as a graph and replayed with other values."""
        return self.mode == "bfloat16" and len(entries) <= self.MAX_RECORDED_ROWS and self.records_cleanly()

    # --------------------------------------------------------------------- step
    def forward(self, ctx: StepContext, cache_views: List[Any]) -> torch.Tensor:
        """Run the step's tokens through every run of the order; float32 logits [wanted, vocab]."""
        ws = ctx.workspace
        h = ws.buffer("model.residual", ctx.num_tokens, self.hidden_size, torch.float32)
        self.embedding.forward(ctx.token_ids, h)
        stream = ResidualStream(h)
        order = self.spec.order
        for index, run in enumerate(order):
            # who reads the residual once this block is through: the block behind it (the final norm after the last
            # one gathers the wanted rows and stays a kernel of its own)
            follower = self.blocks[order[index + 1].layer] if index + 1 < len(order) else None
            stream.after_block = follower.entry_norm() if hasattr(follower, "entry_norm") else None
            self.blocks[run.layer].forward(stream, ctx, cache_views[index])
        logits = torch.empty((ctx.num_wanted, self.vocab_size), dtype=torch.float32, device=self.device)
        if ctx.num_wanted == 0:
            return logits
        x = ws.buffer("model.final", ctx.num_wanted, self.hidden_size, self.act_dtype)
        self.final_norm.apply(stream.h, stream.pending_for(self.final_norm), x, rows=ctx.want_rows)
        self.head.forward(x, logits)
        return logits
