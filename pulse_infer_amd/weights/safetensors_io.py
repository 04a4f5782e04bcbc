"""Reading and writing the safetensors container.

Layout: an unsigned 64-bit little-endian header length, a JSON header
``{name: {dtype, shape, data_offsets}}`` (plus an optional ``__metadata__``
object of strings) and the payload.  The checks on the header follow the
reference's reader (reference: src/core/safetensor.cpp:283-378, :447-551):
sizes, offsets inside the payload, byte size equal to shape times item size,
no overlapping ranges.  Tensors are memory-mapped and handed out as torch
tensors without interpreting the file in any other way.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, Iterable, List, Mapping, Optional, Tuple

import numpy as np
import torch


class SafetensorsError(ValueError):
    pass


# dtype tag -> (torch dtype, numpy carrier dtype, item size)
_DTYPES = {
    "F32": (torch.float32, np.float32, 4),
    "F16": (torch.float16, np.float16, 2),
    "BF16": (torch.bfloat16, np.uint16, 2),
    "F64": (torch.float64, np.float64, 8),
    "I64": (torch.int64, np.int64, 8),
    "I32": (torch.int32, np.int32, 4),
    "I16": (torch.int16, np.int16, 2),
    "I8": (torch.int8, np.int8, 1),
    "U8": (torch.uint8, np.uint8, 1),
    "BOOL": (torch.bool, np.bool_, 1),
}
_TAG_OF = {v[0]: k for k, v in _DTYPES.items()}
_MAX_HEADER = 100 * 1024 * 1024


@dataclass(frozen=True)
class TensorInfo:
    name: str
    dtype: torch.dtype
    shape: Tuple[int, ...]
    begin: int
    end: int


class SafetensorsFile:
    """One memory-mapped safetensors file."""

    def __init__(self, path: str):
        self.path = os.fspath(path)
        size = os.path.getsize(self.path)
        if size < 8:
            raise SafetensorsError(f"'{self.path}' is too small to be a safetensors file ({size} bytes)")
        self._fh = open(self.path, "rb")
        (header_len,) = struct.unpack("<Q", self._fh.read(8))
        if header_len <= 0 or header_len > _MAX_HEADER or 8 + header_len > size:
            raise SafetensorsError(f"'{self.path}' has an invalid header size {header_len}")
        try:
            header = json.loads(self._fh.read(header_len).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as exc:
            raise SafetensorsError(f"'{self.path}' has a header that is not valid JSON: {exc}") from exc
        if not isinstance(header, dict):
            raise SafetensorsError(f"'{self.path}' header must be a JSON object")
        self.payload_offset = 8 + header_len
        payload_size = size - self.payload_offset
        self.metadata: Dict[str, str] = {}
        meta = header.pop("__metadata__", None)
        if meta is not None:
            if not isinstance(meta, dict) or not all(isinstance(v, str) for v in meta.values()):
                raise SafetensorsError(f"'{self.path}': __metadata__ must be an object of strings")
            self.metadata = dict(meta)
        self.tensors: Dict[str, TensorInfo] = {}
        for name, entry in header.items():
            self.tensors[name] = self._check_entry(name, entry, payload_size)
        ranges = sorted((t.begin, t.end, t.name) for t in self.tensors.values())
        for (b0, e0, n0), (b1, e1, n1) in zip(ranges, ranges[1:]):
            if b1 < e0:
                raise SafetensorsError(f"'{self.path}': tensors '{n0}' and '{n1}' overlap")
        self._map: Optional[mmap.mmap] = None

    def _check_entry(self, name: str, entry, payload_size: int) -> TensorInfo:
        where = f"'{self.path}': tensor '{name}'"
        if not isinstance(entry, dict):
            raise SafetensorsError(f"{where} must be an object")
        tag, shape, offsets = entry.get("dtype"), entry.get("shape"), entry.get("data_offsets")
        if tag not in _DTYPES:
            raise SafetensorsError(f"{where} has unsupported dtype {tag!r}")
        if not isinstance(shape, list) or not all(isinstance(d, int) and not isinstance(d, bool) for d in shape):
            raise SafetensorsError(f"{where} has an invalid shape {shape!r}")
        if any(d < 0 for d in shape):
            raise SafetensorsError(f"{where} has a negative dimension in {shape}")
        if (not isinstance(offsets, list) or len(offsets) != 2
                or not all(isinstance(o, int) and not isinstance(o, bool) for o in offsets)):
            raise SafetensorsError(f"{where} has invalid data_offsets {offsets!r}")
        begin, end = offsets
        if begin < 0 or begin > end:
            raise SafetensorsError(f"{where} has data_offsets with begin > end: {offsets}")
        if end > payload_size:
            raise SafetensorsError(f"{where} ends at {end}, beyond the payload of {payload_size} bytes")
        numel = 1
        for d in shape:
            numel *= d
        if numel == 0:
            raise SafetensorsError(f"{where} has zero elements")
        if numel * _DTYPES[tag][2] != end - begin:
            raise SafetensorsError(
                f"{where}: {end - begin} bytes do not match shape {shape} of {tag} ({numel * _DTYPES[tag][2]} bytes)")
        return TensorInfo(name, _DTYPES[tag][0], tuple(shape), begin, end)

    def names(self) -> List[str]:
        return list(self.tensors)

    def info(self, name: str) -> TensorInfo:
        return self.tensors[name]

    def get(self, name: str) -> torch.Tensor:
        """The tensor as a CPU tensor that views the mapped file (copy before changing it)."""
        info = self.tensors[name]
        if self._map is None:
            self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ)
        tag = _TAG_OF[info.dtype]
        carrier = _DTYPES[tag][1]
        count = (info.end - info.begin) // _DTYPES[tag][2]
        array = np.frombuffer(self._map, dtype=carrier, count=count, offset=self.payload_offset + info.begin)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # the map is read-only; callers copy before writing
            tensor = torch.from_numpy(array)
        if info.dtype == torch.bfloat16:
            tensor = tensor.view(torch.bfloat16)
        return tensor.reshape(info.shape)

    def close(self) -> None:
        # numpy views may still reference the map; let the garbage collector take it
        self._map = None
        self._fh.close()


def write_safetensors(path: str, tensors: Mapping[str, torch.Tensor],
                      metadata: Optional[Mapping[str, str]] = None) -> None:
    """Write tensors (CPU, any supported dtype) in name order, 8-byte aligned header."""
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _TAG_OF:
            raise SafetensorsError(f"tensor '{name}' has dtype {t.dtype}, which safetensors cannot hold")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _TAG_OF[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = f"{path}.tmp{os.getpid()}"
    with open(tmp, "wb") as fh:
        fh.write(struct.pack("<Q", len(blob)))
        fh.write(blob)
        for name in order:
            t = tensors[name].detach().contiguous().cpu()
            if t.dtype == torch.bfloat16:
                t = t.view(torch.int16)
            elif t.dtype == torch.bool:
                t = t.view(torch.uint8)
            fh.write(t.numpy().tobytes())
    os.replace(tmp, path)


def find_weight_files(model_dir: str) -> List[str]:
    """Every *.safetensors / *.safetensor file of a folder, sorted by path
    (reference: demo/qwen3_infer.cpp:62-83)."""
    files = [os.path.join(model_dir, f) for f in os.listdir(model_dir)
             if f.endswith(".safetensors") or f.endswith(".safetensor")]
    return sorted(files)
