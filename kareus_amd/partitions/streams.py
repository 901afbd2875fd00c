"""Indirection between the engine and the device's stream/event objects.

The engine needs four things from the device runtime: the stream work is currently
enqueued on, a way to make another stream current, events, and stream-waits-on-
stream.  ``TorchStreams`` maps them onto ``torch.cuda`` (HIP streams on ROCm).  A
test can install a recording implementation with ``use_stream_api`` and replay a
whole forward/backward on the host to check the ordering rules without a GPU.
"""

from __future__ import annotations

import contextlib

import torch


class TorchStreams:
    def available(self) -> bool:
        return torch.cuda.is_available()

    def current_stream(self):
        return torch.cuda.current_stream() if torch.cuda.is_available() else None

    def stream(self, s):
        return contextlib.nullcontext() if s is None else torch.cuda.stream(s)

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
