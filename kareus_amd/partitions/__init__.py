"""Partition-overlap execution engine (public names mirror
kareus/megatron/core/partitions/__init__.py:1-41)."""

from .autograd_function import SeedConfig, TransformerBlockAutogradFunction
from .backward_partition import BackwardPartition
from .context_manager import NanoBatchContext, TensorStore
from .forward_partition import ForwardPartition
from .op_context import (
    BasicOperation,
    OperationContext,
    clear_tensor_data,
    merge_sub_contexts,
    restore_sub_contexts,
)
from .partition_base import OverlapWindow, PartitionBase, ResourceShape
from .partition_builder import PartitionBuilder
from .tensor_graph import (
    Channel,
    CommunicationOp,
    CommunicationOpSpec,
    CommunicationType,
    ComputeOp,
    ComputeOpSpec,
    PartitionableOperator,
    TensorGraph,
    TensorGraphBuilder,
    TensorPort,
)

__all__ = [
    "BackwardPartition",
    "BasicOperation",
    "Channel",
    "CommunicationOp",
    "CommunicationOpSpec",
    "CommunicationType",
    "ComputeOp",
    "ComputeOpSpec",
    "ForwardPartition",
    "NanoBatchContext",
    "OperationContext",
    "OverlapWindow",
    "PartitionableOperator",
    "PartitionBase",
    "PartitionBuilder",
    "ResourceShape",
    "SeedConfig",
    "TensorGraph",
    "TensorGraphBuilder",
    "TensorPort",
    "TensorStore",
    "TransformerBlockAutogradFunction",
    "clear_tensor_data",
    "merge_sub_contexts",
    "restore_sub_contexts",
]
