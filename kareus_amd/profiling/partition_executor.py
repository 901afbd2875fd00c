"""One partition in isolation, built straight from a list of operators, for timing sweeps.

Same job and call surface as the reference's profiling bridge
(tests/bayesian/common/partition_executor.py:75-318): ``PartitionExecutor(operators,
comm_operator, direction, partition_key, comm_type, initial_channel_names, comm_channels,
fwd_initial_channel_names)``, then ``run_forward_setup`` (backward only), ``setup_contexts`` and
any number of ``execute(overlap_window, sm_configs)`` calls.  A backward executor owns a
compute-only forward partition over the same operators so one forward pass can fill the
operator contexts that every timed backward run re-uses (the backward partition is created in
``profiling_mode``, which keeps saved activations alive).

Tensor ids of the seeded channels are ``ext_<channel>``; the hand-over operator reads
``comm_in_<channel>`` from the *other* nanobatch's store and writes ``comm_out_<channel>``.
"""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

from ..backend import reserve_compute_units
from ..partitions.backward_partition import BackwardPartition
from ..partitions.context_manager import NanoBatchContext
from ..partitions.forward_partition import ForwardPartition
from ..partitions.tensor_graph import (
    Channel,
    CommunicationOp,
    CommunicationType,
    ComputeOp,
    ComputeOpSpec,
    TensorGraphBuilder,
    TensorPort,
)

# (direction, collective) -> channels the collective reads and rewrites
# (tests/bayesian/common/partition_executor.py:65-71; only the all-reduce exists on one GPU)
DEFAULT_COMM_CHANNELS: Dict[Tuple[str, CommunicationType], List[Channel]] = {
    ("forward", CommunicationType.ALL_REDUCE): [Channel(0, "main")],
    ("backward", CommunicationType.ALL_REDUCE): [Channel(0, "grad_main")],
}


def _ext_ids(names: Sequence[str]) -> Dict[str, str]:
    return {name: f"ext_{name}" for name in names}


class PartitionExecutor:
    def __init__(
        self,
        operators: List,
        comm_operator,
        direction: str,
        partition_key: str,
        comm_type: CommunicationType = CommunicationType.ALL_REDUCE,
        initial_channel_names: Optional[List[str]] = None,
        comm_channels: Optional[List[Channel]] = None,
        fwd_initial_channel_names: Optional[List[str]] = None,
    ) -> None:
        if direction not in ("forward", "backward"):
            raise ValueError(f"Invalid direction: {direction}")
        if comm_channels is None:
            comm_channels = DEFAULT_COMM_CHANNELS.get((direction, comm_type))
            if comm_channels is None:
                raise ValueError(
                    f"No default comm channels for ({direction}, {comm_type}). Pass comm_channels explicitly."
                )
        self.operators = list(operators)
        self.direction = direction
        self.partition_key = partition_key
        names = initial_channel_names or (["main"] if direction == "forward" else ["grad_main"])
        self._initial_channels = _ext_ids(names)

        comp_ops, self._channel_registry = self._compute_ops(direction, self._initial_channels)
        comm_op = CommunicationOp(
            comm_type=comm_type,
            input_ports=[TensorPort(ch.port_idx, f"comm_in_{ch.name}") for ch in comm_channels],
            output_ports=[TensorPort(ch.port_idx, f"comm_out_{ch.name}") for ch in comm_channels],
            operator=comm_operator,
        )
        if direction == "forward":
            self.partition = ForwardPartition(partition_id=0, partition_key=partition_key,
                                              comp_ops=comp_ops, comm_op=comm_op)
            return
        if fwd_initial_channel_names is None:
            raise ValueError("fwd_initial_channel_names is required for backward direction.")
        self.partition = BackwardPartition(partition_id=0, partition_key=partition_key,
                                           comp_ops=comp_ops, comm_op=comm_op, profiling_mode=True)
        self._fwd_initial_channels = _ext_ids(fwd_initial_channel_names)
        self._fwd_setup_partition = ForwardPartition(
            partition_id=0, partition_key=partition_key,
            comp_ops=self._compute_ops("forward", self._fwd_initial_channels)[0], comm_op=None,
        )

    def _compute_ops(self, direction: str, initial: Dict[str, str]) -> Tuple[List[ComputeOp], Dict[str, str]]:
        """Wire the operators, in execution order of ``direction``; op_id = position in the
        forward-order list, so a backward op finds the context its forward twin filled."""
        builder = TensorGraphBuilder()
        builder.add_initial_channels(initial)
        order = range(len(self.operators))
        for i in (order if direction == "forward" else reversed(order)):
            spec = ComputeOpSpec(operator=self.operators[i], is_backward=(direction == "backward"))
            spec.op_id = i
            builder.add_op(spec)
        return builder.build().get_compute_ops(), dict(builder.get_channel_registry())

    # -- contexts -----------------------------------------------------------------
    def run_forward_setup(self, fwd_compute_tensors: Dict[str, object]) -> None:
        """One forward pass over the operators (backward executors only), keeping the
        operator contexts for the timed backward runs."""
        ctx, pre_ctx = NanoBatchContext(batch_idx=0), NanoBatchContext(batch_idx=1)
        for name, tensor in fwd_compute_tensors.items():
            ctx.tensor_store.set(self._fwd_initial_channels[name], tensor)
        self._fwd_setup_partition.is_grad_enabled = True
        self._fwd_setup_partition.execute(ctx=ctx, pre_ctx=pre_ctx)
        ctx.finalize_recomputed_contexts()
        self._fwd_ctx = ctx

    def setup_contexts(self, compute_tensors: Dict[str, object], comm_tensors: List[object]) -> None:
        """``compute_tensors``: channel name -> tensor of the nanobatch that computes;
        ``comm_tensors``: the other nanobatch's tensors handed over, in port order."""
        self.ctx, self.pre_ctx = NanoBatchContext(batch_idx=0), NanoBatchContext(batch_idx=1)
        for name, tensor in compute_tensors.items():
            tid = self._initial_channels.get(name)
            if tid is None:
                raise ValueError(f"Unknown channel name: {name}")
            self.ctx.tensor_store.set(tid, tensor)
        for port, tensor in zip(self.partition.comm_op.input_ports, comm_tensors):
            self.pre_ctx.tensor_store.set(port.tensor_id, tensor)
        if hasattr(self, "_fwd_ctx"):
            self.ctx.op_contexts = self._fwd_ctx.op_contexts

    # -- one timed unit -------------------------------------------------------------
    def execute(self, overlap_window, sm_configs):
        """One run of the partition under ``overlap_window`` and ``sm_configs = (sm, block)``.  The
        ``sm`` compute units are the ones handed to the overlapped work: the partition's own
        device-filling kernels launch on the rest, as they do inside a step, so the measured time
        and energy are those of the partition under that budget."""
        self.partition._schedule_config = (overlap_window, sm_configs)
        sm = (sm_configs[0] if sm_configs else 0) or 0
        with reserve_compute_units(sm):
            return self.partition.execute(ctx=self.ctx, pre_ctx=self.pre_ctx)

    def output(self, channel: str):
        """Tensor the channel holds after the last ``execute``."""
        return self.ctx.tensor_store.get(self._channel_registry[channel])
