"""RMSNorm operator (kareus/transformer_engine/pytorch/ops/basic/rmsnorm.py:165-273;
weight initialised to ones :150-153; saves the input and the fp32 reciprocal RMS
:223; wrapper class name from kareus/megatron/core/extensions/ops/te_norm.py:23-25)."""

from __future__ import annotations

import torch

from ..backend import get_backend
from ..partitions.op_context import BasicOperation
from ..partitions.streams import stream_api
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
        # a view when the rows have one stride; a nanobatch of several sequences cut out of a [s, b, h]
        # tensor stays as it is where the kernels read row runs in place; else a dense copy
        be = get_backend(self._backend_name)
        x2d = be.rows_in_place(input_)
        y, rstd = be.rmsnorm_fwd(x2d, self.weight.detach(), self.eps)
        if ctx.requires_grad:
            ctx.save_for_backward(x2d, rstd)
        return y.view(input_.shape)

    def op_backward(self, ctx, grad_output):
        x2d, rstd = ctx.saved_tensors
        dy = grad_output.reshape(-1, x2d.shape[-1])
        dx, dgamma = self._backward(ctx, dy, x2d, rstd, None, None)
        return dx.view(grad_output.shape), (dgamma,)

    def _backward(self, ctx, dy, x2d, rstd, residual_grad, out2d):
        """Input gradient and weight gradient.  When the engine attached a ``wgrad_sink`` — one
        dict shared by this norm's contexts of all ``n`` nanobatches of one backward pass — every
        nanobatch leaves its fp32 partial rows of the weight gradient in one shared buffer and
        reports ``None``; the last one to get here waits for the others' events, sums all rows
        in fp32 and reports the gradient, rounded once (the reference lets autograd add the
        per-nanobatch bf16 gradients, kareus/megatron/core/partitions/autograd_function.py:346-372)."""
        be = get_backend(self._backend_name)
        sink = getattr(ctx, "wgrad_sink", None)
        n = sink.get("n", 0) if sink is not None else 0
        if n < 2 or not self.weight.requires_grad:
            return be.rmsnorm_bwd(dy, x2d, rstd, self.weight.detach(), residual_grad=residual_grad, out=out2d)
        cols = x2d.shape[-1]
        rows = x2d.numel() // cols
        per = be.rmsnorm_partial_rows(rows, cols)
        api = stream_api()
        here = api.current_stream()
        buf = sink.get("buf")
        if buf is None or buf.shape[0] != n * per:
            buf = sink["buf"] = torch.empty((n * per, cols), dtype=torch.float32, device=x2d.device)
            sink["done"], sink["events"] = 0, []
            # The block comes from the allocator's pool of THIS stream: whatever used it last is ordered
            # before work queued here, not before the other nanobatch streams.  They wait for this event
            # before they write their rows.
            sink["allocated"] = None
            if here is not None:
                sink["allocated"] = (here, api.new_event())
                sink["allocated"][1].record(here)
        elif here is not None and sink.get("allocated") is not None and sink["allocated"][0] != here:
            here.wait_event(sink["allocated"][1])
        k = sink["done"]
        dx, _ = be.rmsnorm_bwd(dy, x2d, rstd, self.weight.detach(), residual_grad=residual_grad, out=out2d,
                               partials_out=buf[k * per:(k + 1) * per])
        sink["done"] = k + 1
        if here is not None and hasattr(buf, "record_stream") and buf.is_cuda:
            buf.record_stream(here)   # the buffer is shared by the nanobatch streams
        if sink["done"] < n:
            if here is not None:
                ev = api.new_event()
                ev.record(here)
                sink["events"].append(ev)
            return dx, None
        if here is not None:
            for ev in sink["events"]:
                here.wait_event(ev)
        return dx, be.rmsnorm_dgamma(buf, self.weight.detach())

    # -- fused backward with the residual fork that precedes the norm in the layer ------------
    def can_fuse_backward_with(self, next_operator) -> bool:
        return bool(getattr(next_operator, "backward_is_residual_add", False))

    def fuser_backward(self, basic_op_ctxs, grad_output, *, basic_op_grad_extra_outputs):
        if len(basic_op_ctxs) == 1:
            return super().fuser_backward(basic_op_ctxs, grad_output,
                                          basic_op_grad_extra_outputs=basic_op_grad_extra_outputs)
        # [norm, fork]: dx = norm_backward(dy) + grad_residual in one pass over the tensor
        # (kareus/megatron/core/extensions/ops/residual_fork.py:104-106 after rmsnorm.py:256-263)
        norm_ctx, fork_ctx = basic_op_ctxs
        (grad_residual,) = basic_op_grad_extra_outputs[1]
        sink = fork_ctx.__dict__.pop("out_sink", None)
        x2d, rstd = norm_ctx.saved_tensors
        be = get_backend(self._backend_name)
        dy = grad_output.reshape(-1, x2d.shape[-1])
        # a one-sequence slice is a row-strided matrix, a wider one has its rows in runs: written in place
        # where the kernels can, else through a dense result and one copy
        out2d = be.rows_view(sink) if sink is not None else None
        dx, dgamma = self._backward(norm_ctx, dy, x2d, rstd, be.rows_in_place(grad_residual), out2d)
        if sink is not None:
            if out2d is None:
                sink.copy_(dx.view(sink.shape))
            dx = sink
        else:
            dx = dx.view(grad_output.shape)
        return dx, [(dgamma,), ()], [(), ()]


class PartitionableRMSNorm(RMSNorm, PartitionableOperator):
    """RMSNorm that can be placed in a partition graph."""
