"""SwiGLU activation ``y = silu(x1) * x2`` with ``x1, x2 = chunk(x, 2, -1)`` (the first
half gates); backward ``dx1 = dy * sig(x1) * (1 + x1 (1 - sig(x1))) * x2``,
``dx2 = dy * silu(x1)``; saves the input
(kareus/megatron/core/extensions/ops/bias_swiglu.py:14-20, 34-44, 94-192)."""

from __future__ import annotations

from typing import List

from ..backend import get_backend
from ..partitions.op_context import BasicOperation
from ..partitions.tensor_graph import Channel, PartitionableOperator


class BiasSwigluOp(BasicOperation, PartitionableOperator):
    forward_is_swiglu = True   # a projection in front may compute this activation in its epilogue
    backward_is_swiglu = True  # ... and the projection behind it its backward, in the input-gradient GEMM

    def __init__(self, has_bias: bool = False, fp8_input_store: bool = False, backend="hip") -> None:
        super().__init__()
        if has_bias:
            raise NotImplementedError("bias is not part of the Llama-style layer this engine runs")
        if fp8_input_store:
            raise NotImplementedError("fp8 activation storage is not supported")
        self.has_bias = False
        self._backend_name = backend

    def get_input_channels(self) -> List[Channel]:
        return [Channel(0, "main")]

    def op_forward(self, ctx, input_, *, prev_op=None, next_op=None):
        shape = input_.shape
        if len(shape) not in (2, 3):
            raise AssertionError(f"Input must be 2D or 3D, got {len(shape)}D")
        if shape[-1] % 2:
            raise ValueError("SwiGLU input width must be even")
        x2d = input_.reshape(-1, shape[-1])
        if not x2d.is_contiguous():
            x2d = x2d.contiguous()
        y = get_backend(self._backend_name).swiglu_fwd(x2d)
        if ctx.requires_grad:
            ctx.save_for_backward(x2d)
            ctx.ori_shape = shape
        return y.view(*shape[:-1], shape[-1] // 2)

    def op_backward(self, ctx, grad_output):
        (x2d,) = ctx.saved_tensors
        dy = grad_output.reshape(x2d.shape[0], x2d.shape[1] // 2)
        if not dy.is_contiguous():
            dy = dy.contiguous()
        dx = get_backend(self._backend_name).swiglu_bwd(dy, x2d)
        return dx.view(ctx.ori_shape), ()
