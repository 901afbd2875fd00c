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

    # -- what the forward may take along in its epilogue ------------------------------------------
    # fuse_residual (set by the block driver on row-parallel layers of a one-GPU shard): the layer
    # also reads the ``residual`` channel and, when the kernels can address the operands, adds it
    # in the GEMM's epilogue; the result is tagged so that the BiasDropoutAddOp behind the
    # all-reduce slot passes it on instead of adding again.  With more than one rank the sum over
    # ranks has to come first, so the flag is only ever set for a world size of one.
    fuse_residual = False
    forward_accepts_out_sink = False
    # how the one weight-gradient GEMM over all nanobatches is planned (see HipBackend.gemm's split_k)
    wgrad_over_all_split_k = True

    def get_input_channels(self) -> List[Channel]:
        if self.fuse_residual:
            return [Channel(0, "main"), Channel(1, "residual")]
        return [Channel(0, "main")]

    @property
    def num_extra_inputs(self) -> int:  # type: ignore[override]
        return 1 if self.fuse_residual else 0

    def can_fuse_forward_with(self, next_operator) -> bool:
        """The SwiGLU activation behind fc1 can be produced by the projection's epilogue."""
        if not getattr(next_operator, "forward_is_swiglu", False) or not self.fuse_activation:
            return False
        check = getattr(get_backend(self._backend_name), "can_fuse_swiglu", None)
        return check is not None and check(self.weight.shape[0])

    fuse_activation = True

    def fuser_forward(self, basic_op_ctxs, input_, *, basic_op_extra_inputs, basic_op_prev_ops,
                      basic_op_next_ops, basic_op_kwargs):
        ctx = basic_op_ctxs[0]
        n, k = self.weight.shape
        if input_.shape[-1] != k:
            raise ValueError(f"linear with in_features={k} got input of shape {tuple(input_.shape)}")
        be = get_backend(self._backend_name)
        x2d = be.rows_in_place(input_)
        if ctx.requires_grad:
            ctx.save_for_backward(x2d)
            ctx.input_requires_grad = True
        w = self.weight.detach()
        if len(basic_op_ctxs) == 2:
            # [fc1, SwiGLU]: x = input . W^T and y = silu(x[:, :F]) * x[:, F:] from one launch
            # (kareus/megatron/core/extensions/ops/bias_swiglu.py:14-20 behind basic_linear.py:571-582)
            act_ctx = basic_op_ctxs[1]
            y = x2d.new_empty((x2d.numel() // k, n // 2))
            x = be.linear_fwd(x2d, w, split_k=self.split_k, swiglu_out=y)
            if act_ctx.requires_grad:
                act_ctx.save_for_backward(x)
                act_ctx.ori_shape = (*input_.shape[:-1], n)
            return y.view(*input_.shape[:-1], n // 2), [(), ()]
        residual = basic_op_extra_inputs[0][0] if (self.fuse_residual and basic_op_extra_inputs) else None
        sink = ctx.__dict__.pop("out_sink", None)
        out_shape = (*input_.shape[:-1], n)
        if residual is not None:
            # in place where the kernels can address them: row-strided one-sequence slices, row runs of wider ones
            res2d = be.rows_view(residual) if residual.shape[-1] == n else None
            out2d = be.rows_view(sink) if (sink is not None and sink.shape[-1] == n) else None
            if (res2d is not None and res2d.numel() // n == x2d.numel() // k
                    and (sink is None or (out2d is not None and out2d.numel() == res2d.numel()))):
                y = be.linear_fwd(x2d, w, split_k=self.split_k, residual=res2d, out=out2d)
                y = sink if sink is not None else y.view(out_shape)
                y._kr_residual_added = True
                return y, [()]
        y = be.linear_fwd(x2d, w, split_k=self.split_k)
        return y.view(out_shape), [()]

    def op_forward(self, ctx, input_, *, prev_op=None, next_op=None):
        out, _ = self.fuser_forward([ctx], input_, basic_op_extra_inputs=[()], basic_op_prev_ops=[prev_op],
                                    basic_op_next_ops=[next_op], basic_op_kwargs=[{}])
        return out

    def can_fuse_backward_with(self, next_operator) -> bool:
        """The backward of the SwiGLU activation that feeds this layer can run in the epilogue of
        the input-gradient GEMM (the product itself is then never written)."""
        if not getattr(next_operator, "backward_is_swiglu", False) or not self.fuse_activation:
            return False
        return bool(getattr(get_backend(self._backend_name), "can_fuse_swiglu_bwd", False))

    def fuser_backward(self, basic_op_ctxs, grad_output, *, basic_op_grad_extra_outputs):
        extra = (grad_output,) if self.fuse_residual else ()
        if len(basic_op_ctxs) == 1:
            dx, param_grads = self.op_backward(basic_op_ctxs[0], grad_output)
            # the residual input passes the incoming gradient through (out = residual + x . W^T)
            return dx, [param_grads], [extra]
        # [this layer, SwiGLU]: d(activation input) = swiglu_backward(dy . W, x) in one launch
        # (kareus/megatron/core/extensions/ops/bias_swiglu.py:34-44 behind basic_linear.py:847-859)
        ctx, act_ctx = basic_op_ctxs
        (x2d,) = ctx.saved_tensors
        (act_in,) = act_ctx.saved_tensors
        n, _k = self.weight.shape
        be = get_backend(self._backend_name)
        dy = be.rows_in_place(grad_output)
        dx = be.linear_dgrad(dy, self.weight.detach(), split_k=self.split_k, swiglu_bwd_x=act_in)
        dw = self._weight_grad(be, ctx, dy, x2d, self.split_k) if self.weight.requires_grad else None
        return dx.view(act_ctx.ori_shape), [(dw,), ()], [extra, ()]

    def op_backward(self, ctx, grad_output):
        (x2d,) = ctx.saved_tensors
        n, k = self.weight.shape
        be = get_backend(self._backend_name)
        dy = be.rows_in_place(grad_output)
        dx = be.linear_dgrad(dy, self.weight.detach(), split_k=self.split_k)
        dw = self._weight_grad(be, ctx, dy, x2d, self.split_k) if self.weight.requires_grad else None
        return dx.view(*grad_output.shape[:-1], k), (dw,)

    @staticmethod
    def _weight_grad(be, ctx, dy, x2d, split_k=True):
        """``dW = dy^T . x``.  The engine attaches a ``wgrad_sink`` — one dict shared by this layer's
        contexts of all nanobatches of one backward pass — so that the layer's gradient is summed over
        the nanobatches here and autograd sees one tensor (the role of ``accumulate_into_main_grad``,
        kareus/transformer_engine/pytorch/ops/basic/basic_linear.py:898-909); the nanobatches that do
        not deliver it report ``None``.

        Where the backend can contract operand pieces (``linear_wgrad_segments``), the sum over the
        nanobatches is one GEMM over all their tokens: every nanobatch leaves its ``(dy, x)`` pair and an
        event in the sink, and the last one to get here launches the product of all pairs, in nanobatch
        order, on the stream of the nanobatch whose turn it is (the launches of a backward pass take the
        streams in rotation, so no nanobatch's chain of input gradients waits behind all of them) — or,
        when the sink carries a ``pending`` list, leaves the launch there for the engine to issue at the end of
        the backward pass, behind every nanobatch's input gradients.
        Otherwise the first nanobatch allocates the gradient and every later one adds its product into
        it inside its own GEMM, after waiting for the previous writer's event."""
        sink = getattr(ctx, "wgrad_sink", None)
        if sink is None:
            return be.linear_wgrad(dy, x2d, split_k=split_k)
        api = stream_api()
        here = api.current_stream()
        n = sink.get("n", 0)
        if n > 1 and sink.get("defer", True) and hasattr(be, "linear_wgrad_segments"):
            ev = None
            if here is not None:
                ev = api.new_event()
                ev.record(here)
            pairs = sink.setdefault("pairs", [])
            # (aliases: the engine drops the storage behind the saved tensor objects after each backward op)
            pairs.append((getattr(ctx, "nanobatch_index", len(pairs)), dy.detach(), x2d.detach(), ev, here))
            if len(pairs) < n:
                return None
            pairs.sort(key=lambda p: p[0])
            sink["pairs"] = None
            pending = sink.get("pending")
            turn = sink.get("turn")
            if turn is None:
                turn = [0]
            # launched at once, the launches of a backward pass take the nanobatch streams in rotation; put off
            # to the end of the pass they all go to the first nanobatch's stream, one after the other
            target = pairs[0 if pending is not None else turn[0] % n][4]
            turn[0] += 1
            dys, xs = [p[1] for p in pairs], [p[2] for p in pairs]
            with api.stream(target):
                dw = dys[0].new_empty((dys[0].shape[-1], xs[0].shape[-1]))

            def launch():
                with api.stream(target):
                    if target is not None:
                        for _, _, _, ready, st in pairs:
                            if ready is not None and st != target:
                                target.wait_event(ready)
                    if be.wgrad_segments_ok(dys, xs):
                        # planned as a GEMM that has the device to itself (cuts of the contraction where the
                        # output has few tiles): the products of the other nanobatches, which used to fill the
                        # device beside each other, are inside it
                        be.linear_wgrad_segments(dys, xs, out=dw, split_k=PartitionableLinear.wgrad_over_all_split_k)
                    else:
                        be.linear_wgrad(dys[0], xs[0], out=dw, split_k=split_k)
                        for d, x in zip(dys[1:], xs[1:]):
                            be.linear_wgrad(d, x, out=dw, accumulate=True, split_k=split_k)
                    if target is not None:
                        # the operands were allocated on their own nanobatch's stream
                        for t in dys + xs:
                            if t.is_cuda:
                                t.record_stream(target)

            if pending is not None:
                pending.append(launch)
            else:
                launch()
            return dw
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
