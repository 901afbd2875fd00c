"""``out = residual + dropout(x [+ bias])`` and its backward
(kareus/megatron/core/extensions/ops/bias_dropout_add.py:15-45, 82-135, channel
declaration :64-67, fuser wrappers :137-185).

The Llama-style layer has no bias, so the bias channel is refused.  With dropout
probability zero (the benchmark workloads) the op is a residual add forward — usually
already done in the epilogue of the projection in front of it — and passes the incoming
gradient to both branches backward.  With hidden dropout it draws the mask, saves it for the
backward as the reference does (``:106-114``), and scales the incoming gradient by
``mask / (1 - p)`` (``:126-131``).  The mask is this library's (Philox keyed by a seed from
PyTorch's CPU generator), not the one ``native_dropout`` would draw."""

from __future__ import annotations

from typing import List

from ..backend import get_backend
from ..partitions.op_context import BasicOperation
from ..partitions.tensor_graph import Channel, PartitionableOperator


class BiasDropoutAddOp(BasicOperation, PartitionableOperator):
    forward_accepts_out_sink = True

    def __init__(self, has_bias: bool = False, dropout_prob: float = 0.0, training: bool = True,
                 backend="hip") -> None:
        super().__init__()
        if has_bias:
            raise NotImplementedError("bias is not part of the Llama-style layer this engine runs")
        if not 0.0 <= dropout_prob < 1.0:
            raise ValueError(f"dropout probability {dropout_prob} is outside [0, 1)")
        self.has_bias = has_bias
        self.num_extra_inputs = 1
        self.dropout_prob = dropout_prob
        self.training = training
        self._backend_name = backend

    def get_input_channels(self) -> List[Channel]:
        return [Channel(0, "main"), Channel(1, "residual")]

    def fuser_forward(self, basic_op_ctxs, input_, *, basic_op_extra_inputs, basic_op_prev_ops,
                      basic_op_next_ops, basic_op_kwargs):
        (residual,) = basic_op_extra_inputs[0]
        ctx = basic_op_ctxs[0]
        p = self.dropout_prob if self.training else 0.0
        ctx.scale = 1.0 / (1.0 - p)
        ctx.has_bias = False
        # the engine may name the tensor the sum belongs in (a slice of the block's output)
        sink = ctx.__dict__.pop("out_sink", None)
        if getattr(input_, "_kr_residual_added", False):
            # the projection in front added the residual in its epilogue (and wrote into the
            # sink if one was named): nothing is left to do here
            if p != 0.0:
                raise RuntimeError("BiasDropoutAddOp: the residual was added in front of the dropout")
            if sink is not None and sink.data_ptr() != input_.data_ptr():
                raise RuntimeError("BiasDropoutAddOp: fused residual result is not in the output sink")
            return input_, [()]
        be = get_backend(self._backend_name)
        if p == 0.0:
            return be.add(residual, input_, out=sink), [()]
        out, mask = be.dropout_add(input_, residual, p, out=sink)
        if ctx.requires_grad:
            ctx.save_for_backward(mask)
        self.last_mask = mask.detach()   # (an alias the engine does not clear) for tests that hand the mask to the oracle
        return out, [()]

    def fuser_backward(self, basic_op_ctxs, grad_output, *, basic_op_grad_extra_outputs):
        ctx = basic_op_ctxs[0]
        if ctx.scale == 1.0:
            # p = 0: dropout backward is the identity, so both branches get grad_output.
            return grad_output, [()], [(grad_output,)]
        (mask,) = ctx.saved_tensors
        dx = get_backend(self._backend_name).dropout_bwd(grad_output, mask, ctx.scale)
        return dx, [()], [(grad_output,)]
