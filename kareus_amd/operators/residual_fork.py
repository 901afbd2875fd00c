"""Residual fork: forward hands the same tensor to ``main`` and ``residual``;
backward adds the two incoming gradients
(kareus/megatron/core/extensions/ops/residual_fork.py:60-107)."""

from __future__ import annotations

from typing import List

from ..backend import get_backend
from ..partitions.op_context import BasicOperation
from ..partitions.tensor_graph import Channel, PartitionableOperator


class ResidualForkOp(BasicOperation, PartitionableOperator):
    num_extra_outputs = 1
    backward_accepts_out_sink = True
    backward_is_residual_add = True   # backward = grad_main + grad_residual, nothing else

    def __init__(self, backend="hip") -> None:
        super().__init__()
        self._backend_name = backend

    def get_output_channels(self) -> List[Channel]:
        return [Channel(0, "main"), Channel(1, "residual")]

    def fuser_forward(self, basic_op_ctxs, input_, *, basic_op_extra_inputs, basic_op_prev_ops,
                      basic_op_next_ops, basic_op_kwargs):
        return input_, [(input_,)]

    def fuser_backward(self, basic_op_ctxs, grad_output, *, basic_op_grad_extra_outputs):
        (grad_residual,) = basic_op_grad_extra_outputs[0]
        # the engine may name the tensor the sum belongs in (a slice of the block's input gradient)
        sink = basic_op_ctxs[0].__dict__.pop("out_sink", None)
        grad_input = get_backend(self._backend_name).add(grad_output, grad_residual, out=sink)
        return grad_input, [()], [()]
