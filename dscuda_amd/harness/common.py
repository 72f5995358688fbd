"""Library loading, ctypes binding and status checking for the C-ABI.

Mirrors the helpers of the reference harness (``benchmarks/common.py:16-41``):
``library`` / ``bind`` / ``checked`` / ``pointers`` / ``stream`` keep their
names and meaning.  The libraries are looked up at
``<repo>/build/libdscuda_<name>_bench.so`` exactly as there; a missing library
is an error, there is no fallback implementation.
"""

from __future__ import annotations

import ctypes
import os
import sys
from pathlib import Path

import torch

ROOT = Path(__file__).resolve().parents[2]
P, I, F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float

_LIBRARIES: dict[str, ctypes.CDLL] = {}


def library_path(name: str) -> Path:
    """``build/`` under the repository root, or the directory named by the
    environment variable DSCUDA_AMD_LIBRARY_DIR."""
    directory = os.environ.get("DSCUDA_AMD_LIBRARY_DIR")
    base = Path(directory) if directory else ROOT / "build"
    return base / f"libdscuda_{name}_bench.so"


def library(name: str) -> ctypes.CDLL:
    """Load ``build/libdscuda_<name>_bench.so`` (benchmarks/common.py:19-20)."""
    if name not in _LIBRARIES:
        path = library_path(name)
        if not path.exists():
            raise RuntimeError(
                f"{path} is missing: build it with `python -m dscuda_amd.build` "
                "(there is no CPU or PyTorch fallback for the attention kernels)")
        _LIBRARIES[name] = ctypes.CDLL(str(path))
    return _LIBRARIES[name]


def bind(lib, name, signature, result=I):
    """benchmarks/common.py:23-26."""
    function = getattr(lib, name)
    function.argtypes, function.restype = signature, result
    return function


def checked(lib, prefix, status):
    """Raise RuntimeError with the library's message on a non-zero status
    (benchmarks/common.py:29-32)."""
    if status:
        error = bind(lib, f"dscuda_{prefix}_last_error", [], ctypes.c_char_p)
        raise RuntimeError(error().decode())


def leave(status: int = 0):
    """End a finished process that holds a GPU context: wait for the device, flush what was printed, and exit
    without the exit-time teardown of the interpreter and the GPU libraries.  That teardown has ended such a
    process in std::terminate ("terminate called without an active exception", status -6) after all of its
    results were out.  Not for a run under a profiler: its tool writes the trace at exit."""
    if torch.cuda.is_available() and torch.cuda.is_initialized():
        torch.cuda.synchronize()
    sys.stdout.flush()
    sys.stderr.flush()
    os._exit(status)


def pointers(tensors):
    return [x.data_ptr() for x in tensors]


def stream():
    """Raw handle of torch's current stream (benchmarks/common.py:39-40)."""
    return torch.cuda.current_stream().cuda_stream


def c_float(value: float) -> float:
    """The value a C float argument will carry (benchmarks/mla.py:55)."""
    return ctypes.c_float(value).value
