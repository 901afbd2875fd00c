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

    def new_event(self):
        return torch.cuda.Event()


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
