"""Named ranges for profilers (roctx), switched on by RUSTINFER_PROFILE_GPU as in the reference
(crates/infer-core/src/env_flags.rs:18-52).  With the switch off, or without the marker library,
``profile_range`` costs one comparison.  `rocprofv3 --marker-trace --kernel-trace` shows the
ranges beside the kernels they enclose."""
from __future__ import annotations

import contextlib
import ctypes
import os

_lib = None
_on = os.environ.get("RUSTINFER_PROFILE_GPU", "").strip().lower() not in ("", "0", "false", "no", "off")


def _load():
    global _lib, _on
    for name in ("librocprofiler-sdk-roctx.so", "libroctx64.so"):
        try:
            lib = ctypes.CDLL(name)
            lib.roctxRangePushA.argtypes = [ctypes.c_char_p]
            lib.roctxRangePushA.restype = ctypes.c_int
            lib.roctxRangePop.restype = ctypes.c_int
            _lib = lib
            return
        except (OSError, AttributeError):
            continue
    _on = False


@contextlib.contextmanager
def _range(name: str):
    _lib.roctxRangePushA(name.encode())
    try:
        yield
    finally:
        _lib.roctxRangePop()


_NULL = contextlib.nullcontext()


def profile_range(name: str):
    """A context manager that names what runs inside it for the profiler."""
    if not _on:
        return _NULL
    if _lib is None:
        _load()
        if not _on:
            return _NULL
    return _range(name)


def set_enabled(on: bool) -> None:
    global _on
    _on = bool(on)
