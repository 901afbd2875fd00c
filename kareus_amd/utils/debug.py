"""Named ranges for the ROCm profilers (``rocprofv3 --marker-trace``).

The reference wraps regions in NVTX ranges (kareus/utils/debug.py:7-18, ``nvtx_range(msg)``);
here the same context manager pushes and pops a roctx range through ``librocprofiler-sdk-roctx.so``
(or the older ``libroctx64.so``).  Ranges are off unless ``KAREUS_ROCTX=1`` is set when the package
is imported: a push/pop pair per partition is cheap, but not free, and nothing reads them outside a
profiler run.  With the switch on and no library found the ranges are no-ops.
"""

from __future__ import annotations

import contextlib
import ctypes
import os

_LIBS = ("librocprofiler-sdk-roctx.so", "libroctx64.so")
_push = _pop = None
if os.environ.get("KAREUS_ROCTX", "0") not in ("", "0"):
    for _name in _LIBS:
        try:
            _lib = ctypes.CDLL(_name)
            _push, _pop = _lib.roctxRangePushA, _lib.roctxRangePop
            _push.argtypes, _push.restype = [ctypes.c_char_p], ctypes.c_int
            _pop.argtypes, _pop.restype = [], ctypes.c_int
            break
        except (OSError, AttributeError):
            _push = _pop = None


def roctx_enabled() -> bool:
    return _push is not None


class _Range:
    __slots__ = ("msg",)

    def __init__(self, msg: str) -> None:
        self.msg = msg

    def __enter__(self):
        _push(self.msg.encode())
        return self

    def __exit__(self, *exc):
        _pop()
        return False


_NULL = contextlib.nullcontext()


def roctx_range(msg: str):
    """``with roctx_range("fwd_attn nb0"):`` — a named range in the profiler's marker trace."""
    return _Range(msg) if _push is not None else _NULL


nvtx_range = roctx_range  # the reference's name for the same thing
