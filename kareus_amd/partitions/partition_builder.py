"""Cuts a flat graph into per-nanobatch partitions.

The op list is cut after every collective node: ``[A, AR, B, C, AR, D]`` becomes
segments ``([A], AR), ([B, C], AR), ([D], None)``.  Each segment is issued once per
nanobatch, in nanobatch order.  The partition of nanobatch *i* carries the
hand-over of the nanobatch issued just before it: nanobatch *i-1*'s collective of
the same segment, or — for nanobatch 0 — the last nanobatch's collective of the
previous segment.  With two nanobatches this is exactly the reference rule
(kareus/megatron/core/partitions/partition_builder.py:81-148: NB0 gets the previous
segment's comm, NB1 this segment's; first partition has none ``:95``; one key per
partition, count checked ``:104-111``; comm nodes cloned per partition so each can
be bound to its own physical operator ``:26-37``; segmentation ``:150-183``).

The reference fixes two nanobatches; here the count is a parameter.  One nanobatch
degenerates to serial execution: every partition runs its own segment's hand-over
after its compute.
"""

from __future__ import annotations

from typing import List, Optional, Sequence, Tuple, Type, Union

from .backward_partition import BackwardPartition
from .forward_partition import ForwardPartition
from .partition_base import PartitionBase
from .tensor_graph import CommunicationOp, ComputeOp, TensorGraph

Segment = Tuple[List[ComputeOp], Optional[CommunicationOp]]


def _clone_comm(comm: CommunicationOp) -> CommunicationOp:
    """Same ports, independent ``operator`` slot."""
    return CommunicationOp(
        comm_type=comm.comm_type,
        input_ports=comm.input_ports,
        output_ports=comm.output_ports,
        operator=comm.operator,
    )


class PartitionBuilder:
    def __init__(
        self,
        forward_graph: TensorGraph,
        backward_graph: TensorGraph,
        num_nanobatches: int = 2,
    ) -> None:
        if num_nanobatches < 1:
            raise ValueError(f"num_nanobatches must be >= 1, got {num_nanobatches}")
        self.forward_graph = forward_graph
        self.backward_graph = backward_graph
        self.num_nanobatches = num_nanobatches

    def build_forward_partitions(self, partition_keys: Sequence[str]) -> List[ForwardPartition]:
        return self._form_partitions(self.forward_graph.ops, ForwardPartition, partition_keys)

    def build_backward_partitions(self, partition_keys: Sequence[str]) -> List[BackwardPartition]:
        return self._form_partitions(self.backward_graph.ops, BackwardPartition, partition_keys)

    def _form_partitions(
        self,
        ops: Sequence[Union[ComputeOp, CommunicationOp]],
        partition_class: Type[PartitionBase],
        partition_keys: Sequence[str],
    ) -> list:
        nnb = self.num_nanobatches
        segments = self._split_by_communications(ops)
        expected = nnb * len(segments)
        if len(partition_keys) != expected:
            raise RuntimeError(
                f"Partition key count mismatch: expected {expected} keys "
                f"({nnb} x {len(segments)} segments), got {len(partition_keys)}."
            )

        partitions: list = []
        prev_comm: Optional[CommunicationOp] = None
        for seg_idx, (comp_ops, comm_after) in enumerate(segments):
            for nb in range(nnb):
                if nnb == 1:
                    carried = comm_after
                else:
                    carried = prev_comm if nb == 0 else comm_after
                partitions.append(
                    partition_class(
                        partition_id=len(partitions),
                        partition_key=partition_keys[seg_idx * nnb + nb] or "",
                        nano_batch_idx=nb,
                        comp_ops=comp_ops,
                        comm_op=_clone_comm(carried) if carried is not None else None,
                        force_no_overlap=(nnb == 1),
                    )
                )
            prev_comm = comm_after
        return partitions

    @staticmethod
    def _split_by_communications(
        ops: Sequence[Union[ComputeOp, CommunicationOp]],
    ) -> List[Segment]:
        segments: List[Segment] = []
        pending: List[ComputeOp] = []
        for node in ops:
            if isinstance(node, ComputeOp):
                pending.append(node)
            elif isinstance(node, CommunicationOp):
                if pending:
                    segments.append((pending, node))
                    pending = []
                elif segments:
                    # A collective directly after another one replaces it on the
                    # segment that is already closed.
                    segments[-1] = (segments[-1][0], node)
        if pending:
            segments.append((pending, None))
        return segments
