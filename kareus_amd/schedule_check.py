"""Host-side replay of the engine's stream/event protocol.

``RecordingStreams`` stands in for the device runtime: streams are timelines of
ticks, an event remembers the tick at which it was recorded, a wait adds a
cross-stream edge.  Running a forward/backward of a ``LayerStack`` under it (with the
eager backend, on the CPU) yields the exact order relations the real run would
impose on the device, so tests can ask

* was any event waited on before it was recorded (a schedule that would hang or be
  ignored on the device),
* does partition A happen before partition B, or may they overlap,

for any schedule file, without a GPU.  The reference has no such check; its stream
ordering rests on the event protocol of partition_base.py:145-258 being followed.
"""

from __future__ import annotations

import contextlib
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

Point = Tuple[int, int]  # (stream id, tick)


class FakeEvent:
    def __init__(self, api: "RecordingStreams") -> None:
        self.api = api
        self.point: Optional[Point] = None

    def record(self, stream=None) -> None:
        stream = stream if stream is not None else self.api.current_stream()
        self.point = stream.tick()


class FakeStream:
    def __init__(self, api: "RecordingStreams", sid: int) -> None:
        self.api, self.sid, self.now = api, sid, 0

    def tick(self) -> Point:
        self.now += 1
        return (self.sid, self.now)

    def wait_event(self, event: FakeEvent) -> None:
        if event.point is None:
            self.api.violations.append(f"stream {self.sid} waits on an event that was never recorded")
            return
        self.api.edges.append((event.point, self.tick()))

    def wait_stream(self, other: "FakeStream") -> None:
        self.api.edges.append((other.tick(), self.tick()))

    def __eq__(self, other) -> bool:
        return isinstance(other, FakeStream) and other.sid == self.sid

    def __hash__(self) -> int:
        return hash(self.sid)


@dataclass
class Span:
    name: str
    nano_batch_idx: int
    partition_id: int
    kind: str
    begin: Point
    end: Point = (0, 0)
    op_done: Dict[int, Point] = field(default_factory=dict)  # tick right after op idx was enqueued

    @property
    def compute_end(self) -> Point:
        return self.op_done[max(self.op_done)] if self.op_done else self.begin


class RecordingStreams:
    """Install with ``use_stream_api(RecordingStreams())`` *before* building the LayerStack;
    also use the instance as ``PartitionBase.timer`` to get one span per partition."""

    def __init__(self) -> None:
        self._streams: List[FakeStream] = [FakeStream(self, 0)]
        self._current: List[FakeStream] = [self._streams[0]]
        self.edges: List[Tuple[Point, Point]] = []
        self.violations: List[str] = []
        self.spans: List[Span] = []
        self._open: Dict[int, Span] = {}

    # -- stream API -----------------------------------------------------------------
    def available(self) -> bool:
        return True

    def current_stream(self) -> FakeStream:
        return self._current[-1]

    @contextlib.contextmanager
    def stream(self, s):
        if s is None:
            yield
            return
        self._current.append(s)
        try:
            yield
        finally:
            self._current.pop()

    def new_stream(self) -> FakeStream:
        s = FakeStream(self, len(self._streams))
        self._streams.append(s)
        return s

    def new_event(self) -> FakeEvent:
        return FakeEvent(self)

    # -- partition timer hooks --------------------------------------------------------
    def begin(self, part) -> None:
        self._open[id(part)] = Span(part.partition_key or "-", part.nano_batch_idx, part.partition_id,
                                    type(part).__name__, self.current_stream().tick())

    def op_done(self, part, idx: int) -> None:
        self._open[id(part)].op_done[idx] = self.current_stream().tick()

    def end(self, part) -> None:
        span = self._open.pop(id(part))
        span.end = self.current_stream().tick()
        self.spans.append(span)

    # -- queries ----------------------------------------------------------------------
    def happens_before(self, a: Point, b: Point) -> bool:
        """True iff the device must have passed point ``a`` before it can reach point ``b``."""
        succ: Dict[Point, List[Point]] = {}
        for src, dst in self.edges:
            succ.setdefault(src, []).append(dst)
        # reach[stream] = earliest tick on that stream known to be after ``a``
        reach: Dict[int, int] = {a[0]: a[1]}
        changed = True
        while changed:
            changed = False
            for src, dsts in succ.items():
                if src[0] in reach and src[1] >= reach[src[0]]:
                    for d in dsts:
                        if d[0] not in reach or d[1] < reach[d[0]]:
                            reach[d[0]] = d[1]
                            changed = True
        return b[0] in reach and b[1] >= reach[b[0]]

    def ordered(self, first: Span, second: Span) -> bool:
        """All compute ops of ``first`` are done before ``second`` starts."""
        return self.happens_before(first.compute_end, second.begin)

    def may_overlap(self, x: Span, y: Span) -> bool:
        return not self.ordered(x, y) and not self.ordered(y, x)

    def find(self, kind: str, key: str, nano_batch_idx: int, occurrence: int = 0) -> Span:
        hits = [s for s in self.spans if s.kind == kind and s.name == key and s.nano_batch_idx == nano_batch_idx]
        return hits[occurrence]
