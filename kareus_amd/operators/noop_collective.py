"""The tensor-parallel all-reduce slot on a single GPU: an explicit schedule point.

The reference's ``AllReduce`` operator owns a side stream and an event; a partition
records the event on its compute stream where the schedule says the collective may
start, the side stream waits on it, the collective runs there, and the partition's
stream waits for it at its end
(kareus/transformer_engine/pytorch/ops/basic/all_reduce.py:119-133 stream and event
helpers, :135-178 the collective with the world-size-1 identity at :148-149,
:180-202 ``sync``).

With one GPU there is nothing to reduce, but the slot keeps its place in every
partition and keeps the same four calls.  Each nanobatch runs on its own HIP
stream; the tensor this slot hands over belongs to another nanobatch, and *that
nanobatch's stream* plays the part of the reference's communication stream:

* ``event_record(stream)`` marks the release point on the issuing stream,
* ``event_wait()`` makes the owner's stream wait for that point — the owner may
  not start the next segment before the issuing nanobatch got that far,
* ``fuser_forward`` returns its input (world size 1),
* ``sync(stream)`` makes the issuing stream wait until the owner's stream has passed
  the slot, as it would wait for a real collective to finish.

So the schedule file still decides how far the nanobatch streams may run ahead of
one another: slot ``"none"`` (release after the last op) yields strict alternation,
an early slot lets compute of different nanobatches overlap on the device.
``sm_num``/``block_size`` are accepted and recorded; there is no collective kernel
whose grid they could size.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..partitions.streams import stream_api


class NoOpAllReduce(torch.nn.Module):
    def __init__(self, batch_idx: int = 0, world_size: int = 1, comm_stream=None) -> None:
        super().__init__()
        if world_size != 1:
            raise NotImplementedError(
                "this build runs one GPU's shard; a real all-reduce is outside its scope"
            )
        self.batch_idx = batch_idx
        self.world_size = 1
        self.comm_stream = comm_stream
        self.wait_event = None
        self.done_event = None
        self.last_resource_shape = (None, None)
        self.calls = 0
        if comm_stream is not None:
            self.wait_event = stream_api().new_event()
            self.done_event = stream_api().new_event()

    def set_stream(self, stream) -> None:
        self.comm_stream = stream
        if stream is not None and self.wait_event is None:
            self.wait_event = stream_api().new_event()
            self.done_event = stream_api().new_event()

    def event_record(self, stream) -> None:
        if self.comm_stream is not None and stream is not None:
            self.wait_event.record(stream)

    def event_wait(self) -> None:
        if self.comm_stream is not None:
            self.comm_stream.wait_event(self.wait_event)

    def fuser_forward(self, basic_op_ctxs, input_, *, basic_op_extra_inputs, basic_op_prev_ops,
                      basic_op_next_ops, basic_op_kwargs):
        kw = basic_op_kwargs[0] if basic_op_kwargs else {}
        self.last_resource_shape = (kw.get("sm_num"), kw.get("block_size"))
        self.calls += 1
        return input_, [()]

    def sync(self, current_stream: Optional[object] = None) -> None:
        if self.comm_stream is not None and current_stream is not None:
            if current_stream != self.comm_stream:
                self.done_event.record(self.comm_stream)
                current_stream.wait_event(self.done_event)
