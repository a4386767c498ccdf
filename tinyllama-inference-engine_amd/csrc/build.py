"""Builds the HIP kernels into one shared library beside the sources and loads it with ctypes.

The library is compiled with hipcc for gfx950 only.  It links against the HIP runtime by its
soname; in a process that has imported torch the runtime torch ships is already loaded and is
the one used, so the streams torch hands out are valid in these kernels.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import subprocess
import sys
import tempfile
import time

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ["elementwise.hip", "rope_cache.hip", "attention_generic.hip", "attention_mfma.hip", "gemm_generic.hip",
           "gemm_skinny.hip", "gemm_rows.hip", "gemm_tiles.hip", "sampling.hip", "library_gemm.hip", "probes.hip"]
HEADERS = ["common.h", "no_alloc.h"]
LIBRARY = "libtlie_hip.so"
FLAGS = ["-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-shared",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument"]

_lib = None


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if candidate and (os.path.isabs(candidate) and os.path.exists(candidate) or not os.path.isabs(candidate)):
            return candidate
    return "hipcc"


def source_digest() -> str:
    digest = hashlib.sha256()
    for name in SOURCES + HEADERS:
        with open(os.path.join(HERE, name), "rb") as handle:
            digest.update(name.encode())
            digest.update(handle.read())
    digest.update(" ".join(FLAGS).encode())
    return digest.hexdigest()[:16]


def library_path() -> str:
    """Beside the sources when that folder can be written, else under the temporary folder."""
    if os.access(HERE, os.W_OK):
        return os.path.join(HERE, LIBRARY)
    folder = os.path.join(tempfile.gettempdir(), f"tlie_hip_{os.getuid()}")
    os.makedirs(folder, exist_ok=True)
    return os.path.join(folder, LIBRARY)


def is_current(path: str | None = None) -> bool:
    path = path or library_path()
    stamp = path + ".digest"
    if not (os.path.isfile(path) and os.path.isfile(stamp)):
        return False
    with open(stamp, "r", encoding="utf-8") as handle:
        return handle.read().strip() == source_digest()


def build(verbose: bool = True) -> str:
    """Compiles every source into the library, always; returns the library's path."""
    path = library_path()
    objects = []
    started = time.time()
    build_dir = os.path.join(os.path.dirname(path), "_build")
    os.makedirs(build_dir, exist_ok=True)
    compile_flags = [flag for flag in FLAGS if flag != "-shared"]
    procs = []
    for name in SOURCES:
        obj = os.path.join(build_dir, name.replace(".hip", ".o"))
        objects.append(obj)
        command = [_hipcc(), *compile_flags, "-c", os.path.join(HERE, name), "-I", HERE, "-o", obj]
        if verbose:
            print(f"[tlie build] compiling {name} for gfx950 ...", file=sys.stderr, flush=True)
        procs.append((name, subprocess.Popen(command, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    for name, proc in procs:
        while True:
            try:
                output, _ = proc.communicate(timeout=20)
                break
            except subprocess.TimeoutExpired:
                if verbose:
                    print(f"[tlie build] still compiling {name} ({time.time() - started:.0f} s) ...", file=sys.stderr, flush=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {name}:\n{output}")
    temporary = path + f".tmp{os.getpid()}"
    link = subprocess.run([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objects, "-ldl", "-o", temporary],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if link.returncode != 0:
        raise RuntimeError(f"hipcc failed to link {LIBRARY}:\n{link.stdout}")
    os.replace(temporary, path)
    with open(path + ".digest", "w", encoding="utf-8") as handle:
        handle.write(source_digest())
    if verbose:
        print(f"[tlie build] built {path} in {time.time() - started:.1f} s", file=sys.stderr, flush=True)
    return path


def load() -> ctypes.CDLL:
    """Loads the library, compiling it first when it is absent or older than its sources.
    There is no fallback: without the library the engine does not run."""
    global _lib
    if _lib is not None:
        return _lib
    import torch  # noqa: F401  (loads the HIP runtime the library binds to)
    path = library_path()
    if not is_current(path):
        build()
    try:
        _lib = ctypes.CDLL(path)
    except OSError as error:
        raise RuntimeError(f"the HIP kernel library {path} cannot be loaded: {error}") from None
    return _lib


if __name__ == "__main__":
    build()
