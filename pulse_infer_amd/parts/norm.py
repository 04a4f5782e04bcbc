"""RMSNorm: y = x / sqrt(mean(x^2) + eps) * w, float32 inside, one rounding
(reference: src/ops/kernels/cuda/rmsnorm_kernel.cu:97-157; layer: src/layer/rmsnorm.cpp:9-157)."""
from __future__ import annotations

from typing import Any, Dict, Optional

import torch

from ..ops import kernels
from ..weights.store import TensorSpec
from .base import NORMS, BuildContext, LazyNorm, Part, RowStats


@NORMS.register("rmsnorm")
class RMSNorm(Part):
    @classmethod
    def weight_specs(cls, params: Dict[str, Any]) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((params["size"],), kind="norm")}

    def __init__(self, params: Dict[str, Any], prefix: str, build: BuildContext):
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.weight = build.loader.get(f"{prefix}.weight")

    records_cleanly = True
    takes_parts = True   # delta may be [parts, T, H] float32: the kernel adds the parts in order

    def apply(self, h: torch.Tensor, delta: Optional[torch.Tensor], out: torch.Tensor,
              rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """out = norm(h + delta) * w; h keeps the sum unless rows are gathered."""
        kernels.add_rmsnorm(h, delta, self.weight, self.eps, out, rows=rows)
        return out

    def column_scale(self) -> Optional[torch.Tensor]:
        """The factor of every column: whoever writes the rows that this norm reads next may multiply it in as it
        writes a rounded copy of them (``RowStats``), and leave the rest of the norm to the consumer."""
        return self.weight

    def lazy(self, h: torch.Tensor, stats: RowStats) -> Optional[LazyNorm]:
        """This norm as an input that its consumer finishes: the rows already carry this norm's weight, and dividing
        a row by a number commutes with a linear product."""
        if stats.rounded is None or stats.scaled_by is not self.weight:
            return None
        return LazyNorm(stats.rounded, stats.sumsq, self.eps, h, self)
