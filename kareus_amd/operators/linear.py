"""Tensor-parallel linear layers as partitionable operators.

``y = x . W^T`` with ``W`` stored ``[out, in]``; backward returns ``dx = dy . W`` and
``dW = dy^T . x`` in the weight's dtype; the input is saved
(kareus/transformer_engine/pytorch/ops/basic/basic_linear_bias.py:140-216, 218-275;
GEMM layouts basic_linear.py:571-582, 847-859, 898-909; a strided nanobatch slice
is made contiguous first :565-569).

The tensor-parallel collective is *declared*, not performed, by the layer: a
row-parallel linear appends an all-reduce on ``main`` after its forward, a
column-parallel linear appends one on ``grad_main`` after its backward
(kareus/megatron/core/extensions/ops/te_linear.py, ``get_forward_ops`` /
``get_backward_ops`` of ``TERowParallelLinearOp`` and ``TEColumnParallelLinearOp``).
Those nodes are where the partition builder cuts the layer into segments.
"""

from __future__ import annotations

from typing import Callable, List, Optional, Union

import torch

from ..backend import get_backend
from ..partitions.op_context import BasicOperation
from ..partitions.tensor_graph import (
    Channel,
    CommunicationOpSpec,
    CommunicationType,
    ComputeOpSpec,
    PartitionableOperator,
)


class PartitionableLinear(BasicOperation, PartitionableOperator):
    """Bias-free linear layer; ``weight`` is ``[output_size, input_size]``."""

    def __init__(
        self,
        input_size: int,
        output_size: int,
        *,
        config=None,
        init_method: Optional[Callable[[torch.Tensor], None]] = None,
        bias: bool = False,
        skip_bias_add: bool = False,
        device=None,
        dtype=None,
        backend="hip",
    ) -> None:
        super().__init__()
        if bias:
            raise NotImplementedError("bias is not part of the Llama-style layer this engine runs")
        self.config = config
        self.has_bias = False
        self.te_return_bias = skip_bias_add
        weight = torch.empty(output_size, input_size, device=device, dtype=dtype)
        if init_method is not None:
            init_method(weight)
        else:
            torch.nn.init.normal_(weight, mean=0.0, std=0.02)
        self.weight = torch.nn.Parameter(weight)
        self._backend_name = backend

    def op_forward(self, ctx, input_, *, prev_op=None, next_op=None):
        n, k = self.weight.shape
        if input_.shape[-1] != k:
            raise ValueError(f"linear with in_features={k} got input of shape {tuple(input_.shape)}")
        x2d = input_.reshape(-1, k)
        if not x2d.is_contiguous():
            x2d = x2d.contiguous()
        y = get_backend(self._backend_name).linear_fwd(x2d, self.weight.detach())
        if ctx.requires_grad:
            ctx.save_for_backward(x2d)
            ctx.input_requires_grad = True
        return y.view(*input_.shape[:-1], n)

    def op_backward(self, ctx, grad_output):
        (x2d,) = ctx.saved_tensors
        n, k = self.weight.shape
        dy = grad_output.reshape(-1, n)
        if not dy.is_contiguous():
            dy = dy.contiguous()
        be = get_backend(self._backend_name)
        dx = be.linear_dgrad(dy, self.weight.detach())
        dw = be.linear_wgrad(dy, x2d) if self.weight.requires_grad else None
        return dx.view(*grad_output.shape[:-1], k), (dw,)

    def __repr__(self) -> str:
        return (f"{type(self).__name__}(in_features={self.weight.shape[1]}, "
                f"out_features={self.weight.shape[0]}, bias=False)")


class TEColumnParallelLinearOp(PartitionableLinear):
    """Output features are sharded; its backward input-gradient needs the all-reduce."""

    def get_backward_ops(self) -> List[Union[ComputeOpSpec, CommunicationOpSpec]]:
        return [
            ComputeOpSpec(operator=self, is_backward=True),
            CommunicationOpSpec(CommunicationType.ALL_REDUCE, [Channel(0, "grad_main")]),
        ]


class TERowParallelLinearOp(PartitionableLinear):
    """Input features are sharded; its forward output needs the all-reduce."""

    def get_forward_ops(self) -> List[Union[ComputeOpSpec, CommunicationOpSpec]]:
        return [
            ComputeOpSpec(operator=self),
            CommunicationOpSpec(CommunicationType.ALL_REDUCE, [Channel(0, "main")]),
        ]
