"""Weights by tensor name.

A *source* answers ``names()``, ``info(name)`` and ``get(name)``; sources are a
folder of safetensors files, an in-memory dictionary, or a seeded generator.
A model states which tensors it expects (``TensorSpec`` by name); ``check`` compares
that with what the source holds and raises ONE ``WeightError`` listing every
missing tensor, every unexpected tensor, every wrong shape and every tensor whose
stored type the run would have to round.  Tensors that no part asked for do not
fail a load by themselves unless ``strict`` is set (the reference loads whatever a
file holds and looks up what it needs, src/core/var.cpp:90-116); they are counted
in a warning, and named in the error when the load fails for another reason,
where they usually are the missing tensors under other names.  ``WeightLoader``
then hands tensors to the parts in the storage type the run mode asks for:

* mode ``bfloat16``: bfloat16 stays, a tensor stored in 32-bit stays 32-bit,
  integer tables become int32; float16 is refused, because bfloat16 would drop
  three bits of its mantissa without a word (the reference refuses any type
  other than the run's, src/core/var.cpp:69-74);
* mode ``float32``: every float tensor is widened to float32, which is exact
  for bfloat16 and float16.

(The reference looks tensors up by their checkpoint names through
``VarBuilder::get`` and reports one problem at a time,
src/core/var.cpp:284-305; names: src/model/qwen3/model.cpp:160-314, :970-1021.)
"""
from __future__ import annotations

import warnings
from dataclasses import dataclass
from typing import Dict, Iterable, List, Mapping, Optional, Sequence, Tuple

import torch

from .safetensors_io import SafetensorsFile, find_weight_files


@dataclass(frozen=True)
class TensorSpec:
    """What a part expects of one tensor.

    ``kind`` drives random initialisation: ``linear`` and ``embedding`` are
    normal with a scale from ``fan_in``; ``norm`` is 1 + U(-0.1, 0.1);
    ``table`` is an integer table.
    """

    shape: Tuple[int, ...]
    kind: str = "linear"
    fan_in: Optional[int] = None
    optional: bool = False


class WeightError(ValueError):
    """Raised once per load, with everything that is wrong."""

    def __init__(self, missing: Sequence[str], unexpected: Sequence[str],
                 wrong_shape: Sequence[Tuple[str, Tuple[int, ...], Tuple[int, ...]]], origin: str = "",
                 narrowed: Sequence[Tuple[str, str]] = ()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.narrowed = list(narrowed)
        lines = [f"weights{' in ' + origin if origin else ''} do not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(
                f"{name}: expected {list(want)}, found {list(got)}" for name, want, got in self.wrong_shape))
        if self.narrowed:
            lines.append(f"  stored types that a bfloat16 run would round ({len(self.narrowed)}; run with dtype float32, "
                         "which widens them exactly, or convert the checkpoint): "
                         + ", ".join(f"{name} ({kind})" for name, kind in self.narrowed))
        super().__init__("\n".join(lines))


class DictSource:
    """Tensors held in memory."""

    def __init__(self, tensors: Mapping[str, torch.Tensor], origin: str = "<memory>"):
        self.tensors = dict(tensors)
        self.origin = origin

    def names(self) -> List[str]:
        return list(self.tensors)

    def info(self, name: str) -> Tuple[torch.dtype, Tuple[int, ...]]:
        t = self.tensors[name]
        return t.dtype, tuple(t.shape)

    def get(self, name: str) -> torch.Tensor:
        return self.tensors[name]


class SafetensorsSource:
    """All safetensors files of a folder, merged; a tensor name held twice is an error
    (reference: src/core/var.cpp:197-207)."""

    def __init__(self, model_dir: str):
        self.origin = model_dir
        files = find_weight_files(model_dir)
        if not files:
            raise FileNotFoundError(f"no *.safetensors file in '{model_dir}'")
        self.files = [SafetensorsFile(f) for f in files]
        self.where: Dict[str, SafetensorsFile] = {}
        for f in self.files:
            for name in f.names():
                if name in self.where:
                    raise ValueError(f"tensor '{name}' is held by both '{self.where[name].path}' and '{f.path}'")
                self.where[name] = f

    def names(self) -> List[str]:
        return list(self.where)

    def info(self, name: str) -> Tuple[torch.dtype, Tuple[int, ...]]:
        i = self.where[name].info(name)
        return i.dtype, i.shape

    def get(self, name: str) -> torch.Tensor:
        return self.where[name].get(name)


def check(source, expected: Mapping[str, TensorSpec], strict: bool = False, mode: Optional[str] = None) -> List[str]:
    """Compare what ``source`` holds with what the model expects; one ``WeightError`` for everything that is wrong.
    Returns the names of tensors that no part asked for (an error by themselves only when ``strict``)."""
    held = set(source.names())
    missing = [n for n, s in expected.items() if n not in held and not s.optional]
    unexpected = sorted(held - set(expected))
    wrong, narrowed = [], []
    for name, spec in expected.items():
        if name in held:
            stored, shape = source.info(name)
            if tuple(shape) != tuple(spec.shape):
                wrong.append((name, tuple(spec.shape), tuple(shape)))
            if mode == "bfloat16" and stored == torch.float16:
                narrowed.append((name, "float16"))
    if missing or wrong or narrowed or (strict and unexpected):
        raise WeightError(missing, unexpected, wrong, getattr(source, "origin", ""), narrowed)
    return unexpected


_MODES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def storage_dtype(stored: torch.dtype, mode: str) -> torch.dtype:
    """The type a tensor stored as ``stored`` is kept in under run mode ``mode``."""
    if mode not in _MODES:
        raise ValueError(f"unknown run dtype '{mode}', choose from {sorted(_MODES)}")
    if not stored.is_floating_point:
        return torch.int32
    if mode == "float32":
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32
    if stored == torch.float16:
        raise ValueError("a float16 tensor cannot be kept in a bfloat16 run without rounding it")
    return torch.bfloat16


class WeightLoader:
    """Checked access to a source for one model build."""

    def __init__(self, source, expected: Mapping[str, TensorSpec], mode: str, device: torch.device,
                 strict: bool = False):
        self.ignored = check(source, expected, strict=strict, mode=mode)
        if self.ignored:
            shown = ", ".join(self.ignored[:4]) + (", ..." if len(self.ignored) > 4 else "")
            warnings.warn(f"{len(self.ignored)} tensors of '{getattr(source, 'origin', '<source>')}' belong to no part "
                          f"of the model and are not loaded ({shown}); strict=True makes this an error", stacklevel=2)
        self.source = source
        self.expected = dict(expected)
        self.mode = mode
        self.device = torch.device(device)

    def has(self, name: str) -> bool:
        return name in set(self.source.names())

    def get(self, name: str) -> torch.Tensor:
        if name not in self.expected:
            raise KeyError(f"tensor '{name}' was not declared by any part")
        t = self.source.get(name)
        dtype = storage_dtype(t.dtype, self.mode)
        # one copy to the device; conversion happens there (exact for widening)
        return t.to(self.device, non_blocking=False).to(dtype).contiguous()

    def get_concat(self, names: Iterable[str]) -> torch.Tensor:
        """Several [out, in] matrices stacked along ``out`` (a layout choice, not new maths)."""
        parts = [self.get(n) for n in names]
        dtypes = {p.dtype for p in parts}
        if len(dtypes) != 1:
            parts = [p.to(torch.float32) for p in parts]
        return torch.cat(parts, dim=0).contiguous()
