"""Compile the HIP sources of this folder into one shared library for gfx950.

The library is built in-tree (``csrc/_build``) when that folder can be written,
else under the temporary directory, keyed by a hash of the sources and flags.
A stamp file beside the library records that hash; a library whose stamp does
not match the sources is rebuilt.  Compilation prints a progress line every few
seconds.  ``python -m pulse_infer_amd.csrc.build`` builds from the command line.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from typing import Dict, List, Optional, Sequence

HERE = os.path.dirname(os.path.abspath(__file__))
ARCH = "gfx950"
LIB_NAME = "libpulse_kernels.so"

# packed float32 instructions are switched off for every kernel
COMMON_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


VARIANT_DIR = os.path.join(HERE, "variants")


def sources() -> List[str]:
    return sorted(f for f in os.listdir(HERE) if f.endswith(".hip"))


def headers() -> List[str]:
    return sorted(f for f in os.listdir(HERE) if f.endswith(".h"))


def source_hash() -> str:
    h = hashlib.sha256()
    h.update(" ".join(COMMON_FLAGS).encode())
    for name in sources() + headers():
        h.update(name.encode())
        with open(os.path.join(HERE, name), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc); "
                       "the HIP kernels cannot be built")


def _writable(path: str) -> bool:
    try:
        os.makedirs(path, exist_ok=True)
        probe = os.path.join(path, f".probe{os.getpid()}.{threading.get_ident()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def build_dirs() -> List[str]:
    """Where a library may live, in order of preference."""
    uid = os.getuid() if hasattr(os, "getuid") else 0
    return [os.path.join(HERE, "_build"),
            os.path.join(tempfile.gettempdir(), f"pulse_infer_amd-{uid}", "build")]


def existing_library() -> Optional[str]:
    """A built library whose stamp matches the current sources, if any."""
    want = source_hash()
    for d in build_dirs():
        lib, stamp = os.path.join(d, LIB_NAME), os.path.join(d, "stamp")
        try:
            if os.path.exists(lib) and open(stamp).read().strip() == want:
                return lib
        except OSError:
            continue
    return None


def _log(msg: str) -> None:
    from .. import log
    log.info(msg)


def build(force: bool = False, verbose: bool = True) -> str:
    """Compile everything and return the path of the library."""
    if not force:
        lib = existing_library()
        if lib:
            return lib
    hipcc = find_hipcc()
    out_dir = next((d for d in build_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError(f"no writable build folder among {build_dirs()}")
    srcs = sources()
    stamp = os.path.join(out_dir, "stamp")
    if os.path.exists(stamp):
        os.remove(stamp)
    t0 = time.time()
    if verbose:
        _log(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir}")

    done = threading.Event()

    def ticker() -> None:
        while not done.wait(10.0):
            _log(f"still compiling ... {time.time() - t0:.0f} s")

    tick = threading.Thread(target=ticker, daemon=True)
    if verbose:
        tick.start()

    def compile_one(name: str) -> str:
        obj = os.path.join(out_dir, name[:-4] + ".o")
        cmd = [hipcc, *COMMON_FLAGS, "-c", os.path.join(HERE, name), "-o", obj]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {name}:\n{proc.stderr[-4000:]}")
        if verbose:
            _log(f"compiled {name} ({time.time() - t0:.0f} s)")
        return obj

    try:
        workers = max(1, min(len(srcs), os.cpu_count() or 4, 8))
        with ThreadPoolExecutor(workers) as pool:
            objs = list(pool.map(compile_one, srcs))
        lib = os.path.join(out_dir, LIB_NAME)
        tmp = lib + f".tmp{os.getpid()}"
        cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"linking {LIB_NAME} failed:\n{proc.stderr[-4000:]}")
        os.replace(tmp, lib)
        with open(stamp, "w") as fh:
            fh.write(source_hash())
    finally:
        done.set()
    if verbose:
        _log(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


# ------------------------------------------------------------------ variants
# A variant is one source of csrc/variants compiled with its own -D definitions into a library of
# its own, e.g. the matrix-core attention for one head size.  Only what a model needs is compiled.
def variant_name(source: str, defines: Dict[str, int]) -> str:
    tail = "_".join(f"{k.lower()}{v}" for k, v in sorted(defines.items()))
    return f"libpulse_{source}_{tail}.so" if tail else f"libpulse_{source}.so"


def variant_hash(source: str, defines: Dict[str, int]) -> str:
    h = hashlib.sha256()
    h.update(" ".join(COMMON_FLAGS).encode())
    h.update(repr(sorted(defines.items())).encode())
    for path in [os.path.join(VARIANT_DIR, source + ".hip")] + [os.path.join(HERE, f) for f in headers()]:
        with open(path, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def existing_variant(source: str, defines: Dict[str, int]) -> Optional[str]:
    want, name = variant_hash(source, defines), variant_name(source, defines)
    for d in build_dirs():
        lib, stamp = os.path.join(d, name), os.path.join(d, name + ".stamp")
        try:
            if os.path.exists(lib) and open(stamp).read().strip() == want:
                return lib
        except OSError:
            continue
    return None


def build_variant(source: str, defines: Dict[str, int], force: bool = False, verbose: bool = True) -> str:
    if not force:
        lib = existing_variant(source, defines)
        if lib:
            return lib
    hipcc = find_hipcc()
    out_dir = next((d for d in build_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError(f"no writable build folder among {build_dirs()}")
    name = variant_name(source, defines)
    lib, stamp = os.path.join(out_dir, name), os.path.join(out_dir, name + ".stamp")
    if os.path.exists(stamp):
        os.remove(stamp)
    t0 = time.time()
    if verbose:
        _log(f"compiling {source}.hip {defines} for {ARCH}")
    done = threading.Event()

    def ticker() -> None:
        while not done.wait(10.0):
            _log(f"still compiling {name} ... {time.time() - t0:.0f} s")

    if verbose:
        threading.Thread(target=ticker, daemon=True).start()
    try:
        tmp = lib + f".tmp{os.getpid()}.{threading.get_ident()}"
        cmd = [hipcc, *COMMON_FLAGS, "-shared", *[f"-D{k}={v}" for k, v in sorted(defines.items())],
               os.path.join(VARIANT_DIR, source + ".hip"), os.path.join(HERE, "error_text.hip"), "-o", tmp]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {source}.hip {defines}:\n{proc.stderr[-4000:]}")
        os.replace(tmp, lib)
        with open(stamp, "w") as fh:
            fh.write(variant_hash(source, defines))
    finally:
        done.set()
    if verbose:
        _log(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
