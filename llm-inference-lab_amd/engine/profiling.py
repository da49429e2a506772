"""Named ranges for a profiler's timeline (rocTX), off unless asked for.

The reference pushes NVTX ranges around the phases of a step behind a feature flag
(rust/engine/src/profiling.rs:1-18, rust/engine/src/runner/model/qwen2/engine.rs:923-935).
Here ``Ranges.load()`` finds ROCm's rocTX library at run time; ``rocprofv3
--marker-trace`` then shows the ranges.  Without the library, or when not enabled,
``range()`` costs one attribute test.
"""
from __future__ import annotations

import contextlib
import ctypes
import os
from typing import Optional


class Ranges:
    def __init__(self, lib):
        self._push = lib.roctxRangePushA
        self._push.argtypes = [ctypes.c_char_p]
        self._pop = lib.roctxRangePop

    @classmethod
    def load(cls) -> Optional["Ranges"]:
        for name in ("libroctx64.so", "libroctx64.so.4", "/opt/rocm/lib/libroctx64.so",
                     "librocprofiler-sdk-roctx.so", "/opt/rocm/lib/librocprofiler-sdk-roctx.so"):
            try:
                return cls(ctypes.CDLL(name))
            except (OSError, AttributeError):
                continue
        return None

    @contextlib.contextmanager
    def range(self, name: str):
        self._push(name.encode())
        try:
            yield
        finally:
            self._pop()


def ranges_from_environment() -> Optional[Ranges]:
    """``LLMLAB_ROCTX=1`` turns the ranges on."""
    if os.environ.get("LLMLAB_ROCTX", "") not in ("", "0"):
        return Ranges.load()
    return None
