"""``out = residual + dropout(x [+ bias])`` and its backward
(kareus/megatron/core/extensions/ops/bias_dropout_add.py:15-45, 82-135, channel
declaration :64-67, fuser wrappers :137-185).

The decoder layer here runs without bias and with dropout probability zero, so the
op is a residual add forward and passes the incoming gradient to both branches
backward.  Any other setting is refused rather than approximated."""

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
        if dropout_prob != 0.0 and training:
            raise NotImplementedError("hidden dropout > 0 is not supported (mask RNG is not reproduced)")
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
        ctx.scale = 1.0
        ctx.has_bias = False
        # the engine may name the tensor the sum belongs in (a slice of the block's output)
        sink = ctx.__dict__.pop("out_sink", None)
        if getattr(input_, "_kr_residual_added", False):
            # the projection in front added the residual in its epilogue (and wrote into the
            # sink if one was named): nothing is left to do here
            if sink is not None and sink.data_ptr() != input_.data_ptr():
                raise RuntimeError("BiasDropoutAddOp: fused residual result is not in the output sink")
            return input_, [()]
        out = get_backend(self._backend_name).add(residual, input_, out=sink)
        return out, [()]

    def fuser_backward(self, basic_op_ctxs, grad_output, *, basic_op_grad_extra_outputs):
        # p = 0: dropout backward is the identity, so both branches get grad_output.
        return grad_output, [()], [(grad_output,)]
