"""Random weights from a configuration and a seed.

Every tensor has a generator of its own, seeded from (seed, tensor name), so a
tensor's values do not depend on which other tensors exist or in which order
they are made.  Linear and embedding weights are normal with standard deviation
1/sqrt(fan_in) (``init="fan_in"``) or a fixed one (``init=0.02``); norm weights
are 1 + U(-0.1, 0.1).  Values are rounded to the storage type once.
``write_model_folder`` writes config.json and model.safetensors; ``RandomSource``
serves the same tensors without a file (for sizes not worth writing to disk).
(The reference has no such mode; its tests seed tensors by hand,
tests/layer/test_rmsnorm.cpp:139-155.)
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Any, Dict, List, Mapping, Tuple, Union

import torch

from .safetensors_io import write_safetensors
from .store import TensorSpec

Init = Union[str, float]


def _seed_for(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & 0x7FFFFFFFFFFFFFFF


def make_tensor(name: str, spec: TensorSpec, seed: int, init: Init = "fan_in",
                dtype: torch.dtype = torch.bfloat16, device: Any = "cpu") -> torch.Tensor:
    gen = torch.Generator(device=device)
    gen.manual_seed(_seed_for(seed, name))
    shape = tuple(spec.shape)
    if spec.kind == "norm":
        t = 1.0 + (torch.rand(shape, generator=gen, device=device, dtype=torch.float32) * 0.2 - 0.1)
    elif spec.kind == "table":
        return torch.randint(0, 2 ** 15, shape, generator=gen, device=device, dtype=torch.int32)
    else:
        if init == "fan_in":
            fan_in = spec.fan_in if spec.fan_in else shape[-1]
            std = float(fan_in) ** -0.5
        else:
            std = float(init)
        t = torch.randn(shape, generator=gen, device=device, dtype=torch.float32) * std
    return t.to(dtype)


class RandomSource:
    """A weight source that generates each tensor when asked for it."""

    def __init__(self, expected: Mapping[str, TensorSpec], seed: int, init: Init = "fan_in",
                 dtype: torch.dtype = torch.bfloat16, device: Any = "cpu", include_optional: bool = False):
        self.expected = {n: s for n, s in expected.items() if include_optional or not s.optional}
        self.seed, self.init, self.dtype, self.device = seed, init, dtype, device
        self.origin = f"<random seed={seed}>"

    def names(self) -> List[str]:
        return list(self.expected)

    def info(self, name: str) -> Tuple[torch.dtype, Tuple[int, ...]]:
        return self.dtype, tuple(self.expected[name].shape)

    def get(self, name: str) -> torch.Tensor:
        return make_tensor(name, self.expected[name], self.seed, self.init, self.dtype, self.device)


def write_model_folder(config: Any, out_dir: str, seed: int, init: Init = "fan_in",
                       dtype: torch.dtype = torch.bfloat16) -> str:
    """Write ``config.json`` and ``model.safetensors`` for ``config`` (any registered configuration class)."""
    from ..models.causal_lm import expected_tensors

    os.makedirs(out_dir, exist_ok=True)
    expected = expected_tensors(config.model_spec())
    source = RandomSource(expected, seed, init, dtype)
    tensors = {name: source.get(name) for name in source.names()}
    write_safetensors(os.path.join(out_dir, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": str(seed), "init": str(init)})
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as fh:
        json.dump(config.to_dict(), fh, indent=2)
    return out_dir
