"""Loading the compiled HIP kernels.

There is no fallback: when the library cannot be loaded or built, every op
raises ``KernelLibraryError``.  A library that matches the current sources is
loaded as it is; otherwise it is compiled first (seconds, with progress lines).
"""
from __future__ import annotations

import ctypes
import threading
from typing import Optional

from ..csrc import build as _build
from . import timing


class KernelLibraryError(RuntimeError):
    pass


class KernelError(RuntimeError):
    """An entry point refused its arguments or a launch failed."""


_lock = threading.Lock()
_lib: Optional[ctypes.CDLL] = None
_lib_path: Optional[str] = None


def library_path() -> Optional[str]:
    return _lib_path


def load() -> ctypes.CDLL:
    global _lib, _lib_path
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        try:
            path = _build.existing_library() or _build.build()
            lib = ctypes.CDLL(path)
        except Exception as exc:  # noqa: BLE001 - one loud error, whatever went wrong
            raise KernelLibraryError(
                f"the HIP kernel library of pulse_infer_amd is not available: {exc}. "
                "Build it with `python -m pulse_infer_amd.csrc.build` (needs hipcc).") from exc
        lib.pulse_last_error.restype = ctypes.c_char_p
        _lib, _lib_path = lib, path
        return lib


_variants: dict = {}


def load_variant(source: str, defines: dict) -> ctypes.CDLL:
    """A library compiled from csrc/variants/<source>.hip with the given -D definitions (built on first use)."""
    key = (source, tuple(sorted(defines.items())))
    lib = _variants.get(key)
    if lib is not None:
        return lib
    with _lock:
        lib = _variants.get(key)
        if lib is not None:
            return lib
        try:
            path = _build.existing_variant(source, defines) or _build.build_variant(source, defines)
            lib = ctypes.CDLL(path)
        except Exception as exc:  # noqa: BLE001
            raise KernelLibraryError(f"the HIP kernel variant {source} {defines} is not available: {exc}") from exc
        lib.pulse_last_error.restype = ctypes.c_char_p
        _variants[key] = lib
        return lib


def _invoke(lib: ctypes.CDLL, name: str, args) -> None:
    fn = getattr(lib, name)
    fn.restype = ctypes.c_int
    code = fn(*args)
    if code != 0:
        raise KernelError(f"{name}: {lib.pulse_last_error().decode(errors='replace')}")


def call_in(lib: ctypes.CDLL, name: str, *args, label: str = "") -> None:
    """Call an entry point of ``lib``; a non-zero return becomes a ``KernelError`` with the library's message.
    ``label`` (a shape, say) is added to the name under which a timing table lists the call."""
    if timing._active is not None:
        with timing.region(f"{name} {label}" if label else name):
            _invoke(lib, name, args)
        return
    _invoke(lib, name, args)


def call(name: str, *args, label: str = "") -> None:
    """The same for the core library."""
    call_in(load(), name, *args, label=label)
