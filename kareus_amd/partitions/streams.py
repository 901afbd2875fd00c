"""Indirection between the engine and the device's stream/event objects.

The engine needs four things from the device runtime: the stream work is currently
enqueued on, a way to make another stream current, events, and stream-waits-on-
stream.  ``TorchStreams`` maps them onto ``torch.cuda`` (HIP streams on ROCm).  A
test can install a recording implementation with ``use_stream_api`` and replay a
whole forward/backward on the host to check the ordering rules without a GPU.
"""

from __future__ import annotations

import contextlib
import threading

import torch


class _StreamScope:
    """``with`` block that makes a stream current.  Unlike ``torch.cuda.stream`` it also tells the
    owning ``TorchStreams`` which stream that is, so that the engine's many questions about the
    current stream inside the block cost a thread-local lookup instead of a new stream object."""

    __slots__ = ("api", "stream", "prev_known", "prev")

    def __init__(self, api, stream) -> None:
        self.api, self.stream = api, stream

    def __enter__(self):
        tls = self.api._tls
        self.prev_known = getattr(tls, "current", None)
        self.prev = self.prev_known if self.prev_known is not None else torch.cuda.current_stream()
        torch.cuda.set_stream(self.stream)
        tls.current = self.stream
        return self.stream

    def __exit__(self, *exc):
        torch.cuda.set_stream(self.prev)
        self.api._tls.current = self.prev_known
        return False


class TorchStreams:
    def __init__(self) -> None:
        self._available = None
        self._tls = threading.local()  # .current: the stream set by the innermost stream() block

    def available(self) -> bool:
        if self._available is None:
            self._available = torch.cuda.is_available()
        return self._available

    def current_stream(self):
        known = getattr(self._tls, "current", None)
        if known is not None:
            return known
        return torch.cuda.current_stream() if self.available() else None

    def stream(self, s):
        return contextlib.nullcontext() if s is None else _StreamScope(self, s)

    def new_stream(self):
        return torch.cuda.Stream()

    def new_streams(self, n: int):
        """``n`` streams that the device really runs side by side.

        The HIP runtime multiplexes streams onto a few hardware queues, and two streams that
        share a queue execute strictly one after the other — for nanobatch streams that
        silently removes the overlap the engine is built around.  Which streams share is not
        exposed, so it is measured: a candidate is accepted only if a tiny kernel on it finishes
        while a spinning kernel is still running on every stream accepted so far.  Falls back
        to plain streams when no set of ``n`` concurrent ones is found among the candidates."""
        if n <= 1 or not torch.cuda.is_available():
            return [torch.cuda.Stream() for _ in range(n)]
        candidates = [torch.cuda.Stream() for _ in range(max(16, 4 * n))]
        # first try to stay clear of the caller's stream as well (it runs the nanobatch split and
        # the concatenation); with few hardware queues that may be impossible
        for also_avoid in ([torch.cuda.current_stream()], []):
            chosen = []
            for cand in candidates:
                if all(_run_concurrently(held, cand) for held in also_avoid + chosen):
                    chosen.append(cand)
                    if len(chosen) == n:
                        return chosen
        return candidates[:n]

    def new_event(self):
        return torch.cuda.Event()


def _run_concurrently(a, b, spin_cycles: int = 400_000) -> bool:
    """True if a kernel launched on ``b`` completes while an earlier-launched spinning kernel on
    ``a`` is still running (i.e. the two streams do not share a hardware queue)."""
    flag = torch.zeros(1, device="cuda")
    done_a, done_b = torch.cuda.Event(), torch.cuda.Event()
    torch.cuda.synchronize()
    with torch.cuda.stream(a):
        torch.cuda._sleep(spin_cycles)
        done_a.record(a)
    with torch.cuda.stream(b):
        flag.add_(1.0)
        done_b.record(b)
    done_b.synchronize()
    overlapped = not done_a.query()
    done_a.synchronize()
    return overlapped


_api = TorchStreams()


def stream_api():
    return _api


@contextlib.contextmanager
def use_stream_api(api):
    global _api
    old, _api = _api, api
    try:
        yield api
    finally:
        _api = old
