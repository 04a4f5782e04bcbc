"""Gated feed-forward: down( act(gate(x)) * up(x) ), no biases
(reference: src/model/qwen3/model.cpp:893-913; silu: src/ops/kernels/cuda/silu_kernel.cu:82-97).
gate and up are one product with the row-stacked weight; activation and product are one
kernel in float32 with one rounding."""
from __future__ import annotations

from typing import Any, Dict, Optional

import torch

from ..ops import kernels
from ..weights.store import TensorSpec
from .base import FEED_FORWARDS, BuildContext, LazyNorm, Part, StepContext
from .linear import Linear


SLAB = 16  # rows of a weight slab of the few-rows product


@FEED_FORWARDS.register("gated_mlp")
class GatedMLP(Part):
    @classmethod
    def weight_specs(cls, params: Dict[str, Any]) -> Dict[str, TensorSpec]:
        hidden, inter = params["hidden_size"], params["intermediate_size"]
        return {
            "gate_proj.weight": TensorSpec((inter, hidden), fan_in=hidden),
            "up_proj.weight": TensorSpec((inter, hidden), fan_in=hidden),
            "down_proj.weight": TensorSpec((hidden, inter), fan_in=inter),
        }

    def __init__(self, params: Dict[str, Any], prefix: str, build: BuildContext):
        self.hidden = int(params["hidden_size"])
        self.inter = int(params["intermediate_size"])
        activation = params.get("activation", "silu")
        if activation != "silu":
            raise ValueError(f"gated_mlp has no kernel for activation '{activation}' (only 'silu')")
        load = build.loader
        gate, up = load.get(f"{prefix}.gate_proj.weight"), load.get(f"{prefix}.up_proj.weight")
        # gate and up rows alternate in slabs of 16 where the sizes allow it, so that one workgroup of the
        # few-rows product holds a gate slab and its up slab and can apply SwiGLU itself (a layout choice)
        self.slab = SLAB if (build.mode == "bfloat16" and gate.dtype == torch.bfloat16 and up.dtype == torch.bfloat16
                             and self.inter % SLAB == 0) else 0
        if self.slab:
            stacked = torch.stack([gate.view(-1, SLAB, self.hidden), up.view(-1, SLAB, self.hidden)], dim=1)
            self.gate_up = Linear(stacked.reshape(2 * self.inter, self.hidden).contiguous(), build.mode)
        else:
            self.gate_up = Linear(load.get_concat([f"{prefix}.gate_proj.weight", f"{prefix}.up_proj.weight"]), build.mode)
        del gate, up
        self.down = Linear(load.get(f"{prefix}.down_proj.weight"), build.mode)
        self.act_dtype = build.act_dtype

    accepts_residual = True
    accepts_lazy_input = True   # the first product may take rows that are not normalised yet and scale its result
    records_cleanly = True

    def forward(self, x, ctx: StepContext, residual: Optional[torch.Tensor] = None,
                next_scale: Optional[torch.Tensor] = None):
        tokens = x.shape[0]
        ws = ctx.workspace
        z = ws.buffer("mlp.act", tokens, self.inter, self.act_dtype)
        if isinstance(x, LazyNorm) and not (self.slab and self.gate_up.takes_lazy(x)):
            x = x.materialize(ws.buffer("mlp.normed", tokens, self.hidden, self.act_dtype))
        if isinstance(x, LazyNorm):
            self.gate_up.forward(x, z, swiglu=True)
        elif (self.slab and tokens <= kernels.SKINNY_FAST_ROWS and kernels.gemm_skinny_ok(x, self.gate_up.weight)):
            self.gate_up.forward(x, z, swiglu=True)
        elif (self.slab and self.gate_up.takes_mid(x) and (2 * self.inter) % 32 == 0
              and kernels.gemm_mid_takes(tokens, 2 * self.inter, self.hidden)):
            self.gate_up.forward(x, z, swiglu=True)   # 17 to 64 rows: X shared through LDS, SwiGLU in the epilogue
        elif self.slab and self.gate_up.takes_tiles(x, swiglu=True):
            self.gate_up.forward(x, z, swiglu=True)   # many rows: output tiles on the matrix cores, SwiGLU on the way out
        else:
            gu = ws.buffer("mlp.gate_up", tokens, 2 * self.inter, self.act_dtype)
            self.gate_up.forward(x, gu, own=False)   # (the shapes that come here at 17 to 64 rows are those the library wins)
            kernels.swiglu(gu, z, slab=self.slab)
        out = ws.buffer("mlp.out", tokens, self.hidden, self.act_dtype)
        if residual is not None:
            return self.down.add_into(z, residual, out, ws, next_scale)
        return self.down.forward(z, out)
