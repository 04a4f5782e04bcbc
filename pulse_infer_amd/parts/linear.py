"""y = x W^T for a weight stored [out, in] (reference: src/layer/linear.cpp:213).

In the bfloat16 run the product is the vendor library's (torch.matmul, i.e.
hipBLASLt/rocBLAS, float32 accumulation), as the reference uses cuBLAS
(src/ops/kernels/cuda/matmul_kernel.cu:132-154).  In the float32 run, for a
weight kept in 32-bit, and wherever float32 results are asked of bfloat16
operands, the product is this package's own fused-multiply-add kernel.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..ops import kernels


class Linear:
    def __init__(self, weight: torch.Tensor, mode: str):
        if weight.dim() != 2:
            raise ValueError(f"a linear weight must be a matrix, got shape {tuple(weight.shape)}")
        self.weight = weight
        self.out_features, self.in_features = weight.shape
        self.mode = mode
        self.library = mode == "bfloat16" and weight.dtype == torch.bfloat16

    def forward(self, x: torch.Tensor, out: torch.Tensor, rows: Optional[int] = None) -> torch.Tensor:
        """``out`` [M, out_features] receives the product; its storage type chooses the path."""
        w = self.weight if rows is None else self.weight[:rows]
        if self.library and out.dtype == torch.bfloat16 and x.dtype == torch.bfloat16:
            torch.matmul(x, w.t(), out=out)
        else:
            kernels.gemm_f32(x, w, out)
        return out
