"""Causal grouped-query attention operator.

Inputs ``main`` (query ``[s, b, nq, hd]``, or the grouped view ``[s, b, nkv, nq/nkv, hd]``
the QKV-split operator produces), ``key`` and ``value`` (``[s, b, nkv, hd]``);
output ``[s, b, nq*hd]``.  Softmax scale ``1/sqrt(hd)``; query head ``i`` attends KV head
``i // (nq/nkv)``; causal mask aligned top-left (``sq == sk``); saves q, k, v, the
output and the fp32 log-sum-exp ``[b, nq, s]``
(kareus/megatron/core/extensions/ops/te_attention.py:343-432;
kareus/transformer_engine/pytorch/attention/dot_product_attention/
dot_product_attention_op.py:218-221 scale, :267-593 forward, :595-632 backward;
kareus/flash_attn/flash_attn_interface.py:289-318, 321-351, 473-493).

The reference transposes to batch-major copies around the flash-attention call;
the kernels here read and write the sequence-major tensors through their strides,
so no layout copy is made in either direction.
"""

from __future__ import annotations

import math
from typing import List

from ..backend import get_backend
from ..partitions.op_context import BasicOperation
from ..partitions.tensor_graph import Channel, PartitionableOperator


class TEDotProductAttentionOp(BasicOperation, PartitionableOperator):
    num_extra_inputs = 2

    def __init__(self, config=None, layer_number: int = 1, attn_mask_type: str = "causal",
                 attention_dropout: float = 0.0, softmax_scale=None, backend="hip") -> None:
        super().__init__()
        if attn_mask_type != "causal":
            raise NotImplementedError("only the causal mask is supported")
        if attention_dropout != 0.0:
            raise NotImplementedError("attention dropout is not supported")
        self.config = config
        self.layer_number = layer_number
        self.softmax_scale = softmax_scale
        self._backend_name = backend
        # True: the attention launches take their unsplit forms whatever the batch (KR_ATTN_BESIDE_OTHER_STREAMS),
        # so a sequence gets the same bits in a nanobatch as in the whole microbatch.  The block driver sets it
        # when the nanobatches run on streams of their own.
        self.beside_other_streams = False

    def get_input_channels(self) -> List[Channel]:
        return [Channel(0, "main"), Channel(1, "key"), Channel(2, "value")]

    def fuser_forward(self, basic_op_ctxs, input_, *, basic_op_extra_inputs, basic_op_prev_ops,
                      basic_op_next_ops, basic_op_kwargs):
        key, value = basic_op_extra_inputs[0]
        q = input_
        if q.dim() not in (4, 5) or key.dim() != 4 or value.dim() != 4:
            raise ValueError("attention expects [s, b, heads, head_dim] tensors")
        s, b, hd = q.shape[0], q.shape[1], q.shape[-1]
        nq = q.shape[2] * q.shape[3] if q.dim() == 5 else q.shape[2]
        if key.shape != value.shape or key.shape[0] != s or key.shape[1] != b or key.shape[3] != hd:
            raise ValueError(f"q {tuple(q.shape)}, k {tuple(key.shape)}, v {tuple(value.shape)} do not match")
        if nq % key.shape[2] or (q.dim() == 5 and q.shape[2] != key.shape[2]):
            raise ValueError("query heads must be a multiple of KV heads")
        scale = self.softmax_scale if self.softmax_scale is not None else 1.0 / math.sqrt(hd)
        ctx = basic_op_ctxs[0]
        out, lse = get_backend(self._backend_name).attn_fwd(q, key, value, scale, True,
                                                            beside_other_streams=self.beside_other_streams)
        if ctx.requires_grad:
            ctx.save_for_backward(q, key, value, out, lse)
            ctx.scale = scale
        return out.view(s, b, nq * hd), [()]

    def fuser_backward(self, basic_op_ctxs, grad_output, *, basic_op_grad_extra_outputs):
        ctx = basic_op_ctxs[0]
        q, key, value, out, lse = ctx.saved_tensors
        dq, dk, dv = get_backend(self._backend_name).attn_bwd(
            grad_output, q, key, value, out, lse, ctx.scale, True, beside_other_streams=self.beside_other_streams
        )
        return dq, [()], [(dk, dv)]
