"""Small helpers around the engine (profiler ranges)."""

from .debug import roctx_range, roctx_enabled

__all__ = ["roctx_range", "roctx_enabled"]
