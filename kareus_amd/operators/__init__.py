"""Partitionable operators of a Llama-style decoder layer (class names are the
reference's: the slot table keys on them)."""

from .attention import TEDotProductAttentionOp
from .bias_dropout_add import BiasDropoutAddOp
from .bias_swiglu import BiasSwigluOp
from .linear import PartitionableLinear, TEColumnParallelLinearOp, TERowParallelLinearOp
from .noop_collective import NoOpAllReduce
from .qkv_postprocess import QKVPostProcessOp
from .residual_fork import ResidualForkOp
from .rmsnorm import PartitionableRMSNorm, RMSNorm
from .rotary_embedding import RotaryEmbeddingOp, rotary_frequencies

__all__ = [
    "BiasDropoutAddOp",
    "BiasSwigluOp",
    "NoOpAllReduce",
    "PartitionableLinear",
    "PartitionableRMSNorm",
    "QKVPostProcessOp",
    "RMSNorm",
    "ResidualForkOp",
    "RotaryEmbeddingOp",
    "TEColumnParallelLinearOp",
    "TEDotProductAttentionOp",
    "TERowParallelLinearOp",
    "rotary_frequencies",
]
