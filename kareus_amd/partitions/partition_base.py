"""State and schedule-point protocol shared by forward and backward partitions.

A partition = the compute ops of one segment for one nanobatch, plus at most one
schedule point (the collective slot of the reference) that hands over a tensor of
the *previous* nanobatch in issue order.  Where inside the op list that hand-over is
released comes from the schedule: ``overlap_window = (start, end)`` given as op
indices or slot names, ``resource_shape = (sm_num, block_size)`` passed through to
the collective.

Follows kareus/megatron/core/partitions/partition_base.py: operator-class ->
group table ``:22-34``, slot naming with merging of adjacent memory-bound ops
``:37-69``, ``"none"`` sentinel and unknown-slot error ``:72-80``, schedule lookup
by ``partition_key`` ``:117-128``, default window ``(0, -1)`` without a schedule
``:136-137``, ``comm_end`` must be -1 ``:158-162``, launch / no-overlap launch /
sync sequences ``:185-258``.
"""

from __future__ import annotations

import contextlib
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple, Union

from ..backend import reserve_compute_units
from ..utils.debug import roctx_enabled, roctx_range
from .context_manager import NanoBatchContext
from .streams import stream_api
from .tensor_graph import CommunicationOp, ComputeOp

OverlapWindow = Tuple[Union[int, str], Union[int, str]]
ResourceShape = Tuple[Optional[int], Optional[int]]

# Operator class name -> slot group.  Names are the reference's class names; the
# schedule files address slots as "<group>_<n>", so these strings are an interface.
_GROUP_BY_CLASS: Dict[str, str] = {
    "ResidualForkOp": "norm",
    "BiasDropoutAddOp": "norm",
    "PartitionableRMSNorm": "norm",
    "QKVPostProcessOp": "rope",
    "RotaryEmbeddingOp": "rope",
    "BiasSwigluOp": "activation",
    "PartitionableLinear": "linear",
    "TEColumnParallelLinearOp": "linear",
    "TERowParallelLinearOp": "linear",
    "TEDotProductAttentionOp": "attn",
}
_MEMORY_BOUND_GROUPS = frozenset({"norm", "rope", "activation"})


def _build_overlap_slots(comp_ops: List[ComputeOp]) -> Dict[str, int]:
    """Name the places a hand-over may be released: ``{"norm_0": 0, "linear_0": 2, ...}``.

    A run of adjacent HBM-bound ops of one group is a single slot at its first op;
    every MFMA-bound op (linear, attention) is a slot of its own.
    """
    slots: Dict[str, int] = {}
    seen: Dict[str, int] = {}
    open_group: Optional[str] = None
    for idx, op in enumerate(comp_ops):
        cls = type(op.operator).__name__
        if cls not in _GROUP_BY_CLASS:
            raise ValueError(f"Unknown operator class {cls!r} — add it to _GROUP_BY_CLASS")
        group = _GROUP_BY_CLASS[cls]
        if group in _MEMORY_BOUND_GROUPS:
            if group == open_group:
                continue
            open_group = group
        else:
            open_group = None
        n = seen.get(group, 0)
        seen[group] = n + 1
        slots[f"{group}_{n}"] = idx
    return slots


def _resolve_slot(slots: Dict[str, int], name: str) -> int:
    if name == "none":
        return -1
    if name not in slots:
        raise KeyError(f"Unknown overlap slot {name!r}. Available: {sorted(slots)}")
    return slots[name]


def _current_stream():
    """The HIP stream kernels are being enqueued on (None on a host-only run)."""
    return stream_api().current_stream()


class _TimerScope:
    def __init__(self, timer, partition) -> None:
        self.timer, self.partition = timer, partition

    def __enter__(self):
        self.timer.begin(self.partition)

    def __exit__(self, *exc):
        self.timer.end(self.partition)
        return False


@dataclass
class PartitionBase:
    partition_id: int
    partition_key: str = ""
    nano_batch_idx: int = 0
    comp_ops: List[ComputeOp] = field(default_factory=list)
    comm_op: Optional[CommunicationOp] = None
    _schedule_config: Optional[Tuple[OverlapWindow, ResourceShape]] = None
    profiling_mode: bool = False
    # Grad mode is off inside autograd.Function.forward, so the caller's value is
    # captured outside and pushed in here (reference: forward_partition.py:66-71).
    is_grad_enabled: bool = True
    # With a single nanobatch there is no other nanobatch to overlap with: the
    # hand-over runs after this partition's own compute whatever the schedule says.
    force_no_overlap: bool = False
    # the schedule's resource shape sets a compute-unit budget for this partition's GEMM launches
    apply_resource_shape: bool = True

    def __post_init__(self) -> None:
        self._overlap_slots: Dict[str, int] = _build_overlap_slots(self.comp_ops)

    # -- schedule ---------------------------------------------------------------
    def load_schedule(self, schedule) -> None:
        config = getattr(schedule, self.partition_key, None) if self.partition_key else None
        if config is not None:
            self._schedule_config = (config.overlap_window, config.resource_shape)

    def _get_comm_config(self) -> Tuple[Tuple[int, int], ResourceShape]:
        if not self._schedule_config:
            return ((0, -1), (None, None))
        (start, end), shape = self._schedule_config
        if isinstance(start, str):
            start = _resolve_slot(self._overlap_slots, start)
        if isinstance(end, str):
            end = _resolve_slot(self._overlap_slots, end)
        return ((start, end), shape)

    def _setup_comm(self) -> Tuple[int, int, Optional[int], Optional[int]]:
        if self.comm_op is None:
            return -1, -1, None, None
        (start, end), (sm_num, block_size) = self._get_comm_config()
        if end != -1:
            raise ValueError(
                f"comm_end must be -1 (sentinel 'none'); got {end}. "
                "Partition execution does not use comm_end — set overlap_end to 'none'."
            )
        if start >= len(self.comp_ops) or start < -1:
            raise ValueError(
                f"comm_start {start} is outside this partition's {len(self.comp_ops)} ops"
            )
        if self.force_no_overlap:
            start = -1
        if start == 0:
            self.comm_op.event_record(_current_stream())
        return start, end, sm_num, block_size

    # -- the hand-over itself ---------------------------------------------------
    def _read_comm_inputs(self, pre_ctx: NanoBatchContext):
        ports = self.comm_op.input_ports
        head = pre_ctx.tensor_store.get(ports[0].tensor_id)
        extras: list = []
        if len(ports) > 1:
            extras = [tuple(pre_ctx.tensor_store.get(p.tensor_id) for p in ports[1:])]
        return head, extras

    def _run_comm(self, pre_ctx, sm_num, block_size, backward: bool):
        head, extras = self._read_comm_inputs(pre_ctx)
        kwargs: Dict[str, Any] = {"sm_num": sm_num, "block_size": block_size}
        if backward:
            kwargs["backward"] = True
        return self.comm_op.fuser_forward(
            [None],
            head,
            basic_op_extra_inputs=extras,
            basic_op_prev_ops=[None],
            basic_op_next_ops=[None],
            basic_op_kwargs=[kwargs],
        )

    def _launch_comm(self, pre_ctx, sm_num, block_size, *, backward: bool = False):
        """Release point reached earlier (event already recorded): wait on it, run."""
        self.comm_op.event_wait()
        return self._run_comm(pre_ctx, sm_num, block_size, backward)

    def _launch_comm_no_overlap(self, pre_ctx, sm_num, block_size, *, backward: bool = False):
        """No slot given: release only after all of this partition's compute."""
        self.comm_op.event_record(_current_stream())
        self.comm_op.event_wait()
        return self._run_comm(pre_ctx, sm_num, block_size, backward)

    def _sync_comm(self, pre_ctx: NanoBatchContext, comm_output, comm_extra_outputs) -> None:
        self.comm_op.sync(_current_stream())
        ports = self.comm_op.output_ports
        src = self.comm_op.input_ports
        store = pre_ctx.tensor_store
        store.set(ports[0].tensor_id, comm_output, store.needs_grad(src[0].tensor_id))
        if comm_extra_outputs:
            for k, port in enumerate(ports[1:]):
                extra = comm_extra_outputs[0][k]
                if extra is not None:
                    store.set(port.tensor_id, extra, store.needs_grad(src[k + 1].tensor_id))

    # -- optional per-partition timing ---------------------------------------------
    # Set ``PartitionBase.timer`` to an object with ``begin(partition)`` / ``end(partition)``
    # (e.g. recording HIP events) to time partitions; None costs nothing.
    timer = None

    def _timed(self):
        t = PartitionBase.timer
        if t is None:
            return contextlib.nullcontext()
        return _TimerScope(t, self)

    def _op_done(self, idx: int) -> None:
        t = PartitionBase.timer
        if t is not None and hasattr(t, "op_done"):
            t.op_done(self, idx)

    # -- stream scoping -----------------------------------------------------------
    def _on_stream(self, ctx: NanoBatchContext):
        """Context manager making the nanobatch's own stream current (if it has one); with a
        schedule it also reserves the compute units the partition's resource shape names for
        the kernels of the other nanobatch streams, and the whole is a named profiler range."""
        on_stream = stream_api().stream(ctx.stream)
        sm_num = 0
        if ctx.stream is not None and self.apply_resource_shape and self._schedule_config and self.comm_op is not None:
            sm_num = self._schedule_config[1][0] or 0
        if not sm_num and not roctx_enabled():
            return on_stream
        scope = contextlib.ExitStack()
        scope.enter_context(on_stream)
        if sm_num:
            scope.enter_context(reserve_compute_units(sm_num))
        if roctx_enabled():
            scope.enter_context(roctx_range(f"{self.partition_key or 'trail'} nb{self.nano_batch_idx}"))
        return scope

    def execute(self, ctx: NanoBatchContext, pre_ctx: NanoBatchContext):
        raise NotImplementedError
