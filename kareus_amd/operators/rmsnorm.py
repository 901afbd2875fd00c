"""RMSNorm operator (kareus/transformer_engine/pytorch/ops/basic/rmsnorm.py:165-273;
weight initialised to ones :150-153; saves the input and the fp32 reciprocal RMS
:223; wrapper class name from kareus/megatron/core/extensions/ops/te_norm.py:23-25)."""

from __future__ import annotations

import torch

from ..backend import get_backend
from ..partitions.op_context import BasicOperation
from ..partitions.tensor_graph import PartitionableOperator


class RMSNorm(BasicOperation):
    def __init__(self, hidden_size: int, eps: float = 1e-5, device=None, dtype=None,
                 zero_centered_gamma: bool = False, backend="hip") -> None:
        super().__init__()
        if zero_centered_gamma:
            raise NotImplementedError("zero_centered_gamma is not used by the Llama-style layer")
        self.eps = float(eps)
        self.weight = torch.nn.Parameter(torch.ones(hidden_size, device=device, dtype=dtype))
        self._backend_name = backend

    def op_forward(self, ctx, input_, *, prev_op=None, next_op=None):
        h = self.weight.shape[0]
        if input_.shape[-1] != h:
            raise ValueError(f"RMSNorm over {h} features got input of shape {tuple(input_.shape)}")
        x2d = input_.reshape(-1, h)   # a view when the rows have one stride, else a dense copy
        y, rstd = get_backend(self._backend_name).rmsnorm_fwd(x2d, self.weight.detach(), self.eps)
        if ctx.requires_grad:
            ctx.save_for_backward(x2d, rstd)
        return y.view(input_.shape)

    def op_backward(self, ctx, grad_output):
        x2d, rstd = ctx.saved_tensors
        dy = grad_output.reshape(x2d.shape)
        dx, dgamma = get_backend(self._backend_name).rmsnorm_bwd(dy, x2d, rstd, self.weight.detach())
        return dx.view(grad_output.shape), (dgamma,)


class PartitionableRMSNorm(RMSNorm, PartitionableOperator):
    """RMSNorm that can be placed in a partition graph."""
