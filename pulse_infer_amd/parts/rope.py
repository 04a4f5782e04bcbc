"""Rotary position encoding: pairs of channels rotated by position * theta^(-2i/rotary_dim).

The reference rotates ADJACENT pairs (x[2i], x[2i+1])
(src/ops/kernels/cuda/rope_kernel.cu:100-126); ``pairing: "half"`` rotates
(x[i], x[i + rotary_dim/2]) instead.  Channels beyond ``rotary_dim`` pass unchanged.
Once per step this part makes the cos/sin tables for the step's positions (angles in
float64, tables float32); the mixer's fused kernel applies them to q and k.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict

import torch

from ..ops import kernels
from .base import POSITIONS, BuildContext, Part, StepContext

PAIRINGS = {"interleaved": 0, "half": 1}


@dataclass
class RotationTables:
    cos: torch.Tensor   # float32 [T, rotary_dim / 2]
    sin: torch.Tensor
    rotary_dim: int
    pairing: int


@POSITIONS.register("rope")
class RotaryEmbedding(Part):
    records_cleanly = True

    def __init__(self, params: Dict[str, Any], build: BuildContext):
        self.theta = float(params["theta"])
        self.rotary_dim = int(params["rotary_dim"])
        self.head_dim = int(params.get("head_dim", self.rotary_dim))
        pairing = params.get("pairing", "interleaved")
        if pairing not in PAIRINGS:
            raise ValueError(f"unknown rotary pairing '{pairing}', choose from {sorted(PAIRINGS)}")
        if self.rotary_dim <= 0 or self.rotary_dim % 2 or self.rotary_dim > self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even, positive and at most head_dim {self.head_dim}")
        if not self.theta > 0:
            raise ValueError(f"rope theta must be positive, got {self.theta}")
        self.pairing = PAIRINGS[pairing]
        half = self.rotary_dim // 2
        exponent = torch.arange(half, dtype=torch.float64) * (2.0 / self.rotary_dim)
        self.inv_freq = torch.pow(torch.tensor(self.theta, dtype=torch.float64), -exponent).to(build.device)
        self.name = params.get("name", "rope")

    def prepare(self, ctx: StepContext) -> RotationTables:
        half = self.rotary_dim // 2
        cos = ctx.workspace.buffer(f"{self.name}.cos", ctx.num_tokens, half, torch.float32)
        sin = ctx.workspace.buffer(f"{self.name}.sin", ctx.num_tokens, half, torch.float32)
        kernels.rope_table(ctx.positions, self.inv_freq, cos, sin)
        return RotationTables(cos, sin, self.rotary_dim, self.pairing)


@POSITIONS.register("none")
class NoPositionEncoding(Part):
    """Attention that learns order from the causal mask alone."""

    records_cleanly = True

    def __init__(self, params: Dict[str, Any], build: BuildContext):
        pass

    def prepare(self, ctx: StepContext) -> None:
        return None
