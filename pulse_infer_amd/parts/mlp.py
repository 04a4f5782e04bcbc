"""Gated feed-forward: down( act(gate(x)) * up(x) ), no biases
(reference: src/model/qwen3/model.cpp:893-913; silu: src/ops/kernels/cuda/silu_kernel.cu:82-97).
gate and up are one product with the row-stacked weight; activation and product are one
kernel in float32 with one rounding."""
from __future__ import annotations

from typing import Any, Dict

import torch

from ..ops import kernels
from ..weights.store import TensorSpec
from .base import FEED_FORWARDS, BuildContext, Part, StepContext
from .linear import Linear


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
        self.gate_up = Linear(load.get_concat([f"{prefix}.gate_proj.weight", f"{prefix}.up_proj.weight"]), build.mode)
        self.down = Linear(load.get(f"{prefix}.down_proj.weight"), build.mode)
        self.act_dtype = build.act_dtype

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        tokens = x.shape[0]
        ws = ctx.workspace
        gu = ws.buffer("mlp.gate_up", tokens, 2 * self.inter, self.act_dtype)
        self.gate_up.forward(x, gu)
        z = ws.buffer("mlp.act", tokens, self.inter, self.act_dtype)
        kernels.swiglu(gu, z)
        out = ws.buffer("mlp.out", tokens, self.hidden, self.act_dtype)
        return self.down.forward(z, out)
