"""Load libtokenmill_hip.so; compile it first if no built library matches the sources.

There is no other implementation behind these kernels: if the library cannot be loaded or built,
importing the ops fails with an error that says why.
"""
from __future__ import annotations

import ctypes
import threading

from tokenmill_amd.csrc import build as _build

_lock = threading.Lock()
_lib: ctypes.CDLL | None = None


class KernelLibraryError(RuntimeError):
    pass


def library() -> ctypes.CDLL:
    global _lib
    with _lock:
        if _lib is None:
            path = _build.find_library()
            if path is None:
                print("[tokenmill_amd] no built kernel library for these sources; compiling "
                      "(a few seconds per file) ...", flush=True)
                try:
                    path = _build.build(verbose=True)
                except Exception as e:      # noqa: BLE001 - reported with its cause
                    raise KernelLibraryError(f"the HIP kernel library could not be built: {e}") from e
            try:
                _lib = ctypes.CDLL(str(path))
            except OSError as e:
                raise KernelLibraryError(f"the HIP kernel library {path} could not be loaded: {e}") from e
            _lib._tm_path = str(path)
    return _lib
