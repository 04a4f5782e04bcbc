"""Arrangements of mixer, feed-forward and norms around the residual stream.

``prenorm``: h <- h + mixer(norm_a(h)); h <- h + ffn(norm_b(h))
(reference: src/model/qwen3/model.cpp:779-923).  The additions are deferred into
the next norm's kernel through ``ResidualStream``.
"""
from __future__ import annotations

from typing import Any, Dict, Optional

from ..models.spec import LayerSpec
from ..weights.store import TensorSpec
from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, BuildContext, Part, ResidualStream, StepContext, joined, says


@BLOCKS.register("prenorm")
class PreNormBlock(Part):
    NORM_PLACES = ("mixer_norm", "ffn_norm")   # the norms this arrangement has; a layer names a spec for each

    @classmethod
    def layer_weight_specs(cls, layer: LayerSpec) -> Dict[str, TensorSpec]:
        """All tensors of one layer, by full name."""
        p = layer.block.params
        out: Dict[str, TensorSpec] = {}
        for which in cls.NORM_PLACES:
            norm = layer.norm(which)
            for name, spec in NORMS.get(norm.kind).weight_specs(norm.params).items():
                out[joined(joined(layer.prefix, p[which]), name)] = spec
        for part, registry in ((layer.mixer, MIXERS), (layer.ffn, FEED_FORWARDS)):
            sub = joined(layer.prefix, part.params.get("prefix", ""))
            for name, spec in registry.get(part.kind).weight_specs(part.params).items():
                out[joined(sub, name)] = spec
        return out

    def __init__(self, layer: LayerSpec, build: BuildContext):
        p = layer.block.params
        made = {}
        for which in self.NORM_PLACES:
            norm = layer.norm(which)
            made[which] = NORMS.get(norm.kind)(norm.params, joined(layer.prefix, p[which]), build)
        self.mixer_norm, self.ffn_norm = made["mixer_norm"], made["ffn_norm"]
        self.mixer = MIXERS.get(layer.mixer.kind)(layer.mixer.params,
                                                  joined(layer.prefix, layer.mixer.params.get("prefix", "")), build)
        self.ffn = FEED_FORWARDS.get(layer.ffn.kind)(layer.ffn.params,
                                                     joined(layer.prefix, layer.ffn.params.get("prefix", "")), build)
        self.act_dtype = build.act_dtype

    def cache_spec(self) -> Optional[Any]:
        return self.mixer.cache_spec()

    def records_cleanly(self) -> bool:
        """Whether a step of this block may be recorded as a graph and replayed: every part of it says so."""
        return all(says(part, "records_cleanly")
                   for part in (self.mixer, self.ffn, self.mixer_norm, self.ffn_norm))

    def _input(self, stream: ResidualStream, norm: Any, part: Any, ctx: StepContext) -> Any:
        """norm(h) for ``part``: left to the part's first product where that is possible, else computed here."""
        if getattr(part, "accepts_lazy_input", False):
            lazy = stream.lazy(norm)
            if lazy is not None:
                return lazy
        x = ctx.workspace.buffer("block.normed", ctx.num_tokens, stream.h.shape[1], self.act_dtype)
        return stream.normed(norm, x)

    def entry_norm(self) -> Any:
        """The norm that reads the residual first in this block."""
        return self.mixer_norm

    @staticmethod
    def _scale_of(norm: Any) -> Any:
        return norm.column_scale() if norm is not None and hasattr(norm, "column_scale") else None

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: Any) -> None:
        x = self._input(stream, self.mixer_norm, self.mixer, ctx)
        # a part that says so may add its result into the residual itself and return None (or the new rows' statistics,
        # for which it is told the column factors of the norm that reads the residual next)
        if getattr(self.mixer, "accepts_residual", False):
            stream.push(self.mixer.forward(x, ctx, cache, residual=stream.h, next_scale=self._scale_of(self.ffn_norm)))
        else:
            stream.push(self.mixer.forward(x, ctx, cache))
        x = self._input(stream, self.ffn_norm, self.ffn, ctx)
        if getattr(self.ffn, "accepts_residual", False):
            stream.push(self.ffn.forward(x, ctx, residual=stream.h, next_scale=self._scale_of(stream.after_block)))
        else:
            stream.push(self.ffn.forward(x, ctx))
