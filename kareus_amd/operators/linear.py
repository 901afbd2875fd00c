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
from ..partitions.streams import stream_api
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
        # False when kernels of other nanobatch streams fill the GPU next to this layer's GEMMs:
        # then the contraction is not split, which costs the least CU-time (set by the block driver)
        self.split_k = True

    def op_forward(self, ctx, input_, *, prev_op=None, next_op=None):
        n, k = self.weight.shape
        if input_.shape[-1] != k:
            raise ValueError(f"linear with in_features={k} got input of shape {tuple(input_.shape)}")
        x2d = self._rows(input_.reshape(-1, k))
        y = get_backend(self._backend_name).linear_fwd(x2d, self.weight.detach(), split_k=self.split_k)
        if ctx.requires_grad:
            ctx.save_for_backward(x2d)
            ctx.input_requires_grad = True
        return y.view(*input_.shape[:-1], n)

    def op_backward(self, ctx, grad_output):
        (x2d,) = ctx.saved_tensors
        n, k = self.weight.shape
        dy = self._rows(grad_output.reshape(-1, n))
        be = get_backend(self._backend_name)
        dx = be.linear_dgrad(dy, self.weight.detach(), split_k=self.split_k)
        dw = self._weight_grad(be, ctx, dy, x2d, self.split_k) if self.weight.requires_grad else None
        return dx.view(*grad_output.shape[:-1], k), (dw,)

    @staticmethod
    def _rows(t2d):
        """GEMM operands may be row-strided (a one-sequence nanobatch slice of a
        [seq, batch, hidden] tensor is); the reference copies such slices
        (basic_linear.py:565-569), here only layouts a leading dimension cannot express are."""
        if t2d.stride(1) == 1 and t2d.stride(0) % 8 == 0 and t2d.stride(0) >= t2d.shape[1]:
            return t2d
        return t2d.contiguous()

    @staticmethod
    def _weight_grad(be, ctx, dy, x2d, split_k=True):
        """``dW = dy^T . x``.  When the engine attached a ``wgrad_sink`` — one dict shared by
        this layer's contexts of all nanobatches of one backward pass — the first nanobatch to
        get here allocates the gradient and every later one adds its product into the same
        buffer inside the GEMM (the role of ``accumulate_into_main_grad``,
        kareus/transformer_engine/pytorch/ops/basic/basic_linear.py:898-909), after waiting for
        the previous writer's event; later nanobatches then report ``None`` so that autograd
        does not sum a second time."""
        sink = getattr(ctx, "wgrad_sink", None)
        if sink is None:
            return be.linear_wgrad(dy, x2d, split_k=split_k)
        api = stream_api()
        here = api.current_stream()
        buf = sink.get("buf")
        if buf is None:
            buf = sink["buf"] = be.linear_wgrad(dy, x2d, split_k=split_k)
            ret = buf
        else:
            if here is not None and sink.get("event") is not None:
                here.wait_event(sink["event"])
            be.linear_wgrad(dy, x2d, out=buf, accumulate=True, split_k=split_k)
            ret = None
        if here is not None:
            ev = api.new_event()
            ev.record(here)
            sink["event"] = ev
        return ret

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
