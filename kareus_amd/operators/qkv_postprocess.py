"""Splits the fused QKV projection into query, key and value.

The projection's output features are grouped per KV group ``g`` as
``[q heads of g ..., k_g, v_g]``: ``[s, b, ng * (nq/ng + 2) * hd]`` is viewed as
``[s, b, ng, (nq/ng + 2) * hd]`` and cut along the last axis.  Forward only makes
views; backward reassembles the three gradients into one tensor
(kareus/megatron/core/extensions/ops/qkv_postprocess.py:84-127, 164-184).

The reference reshapes the query part to ``[s, b, nq, hd]``, which copies whenever
there is more than one group with more than one query head.  Here the query is
handed on as the grouped view ``[s, b, ng, nq/ng, hd]`` (never a copy); the rotary
and attention operators address it through its group/head strides.  All three
outputs remember the fused buffer they are views of (``_kr_fused5``), which lets
the rotary operator rotate q and k in place with one launch, and lets ``merge``
return the attention backward's fused gradient buffer as is.  Pass
``grouped_query_view=False`` to get the reference's dense 4-D query instead.
"""

from __future__ import annotations

from typing import List

import torch

from ..partitions.op_context import BasicOperation
from ..partitions.tensor_graph import Channel, PartitionableOperator


class QKVPostProcessOp(BasicOperation, PartitionableOperator):
    num_extra_outputs = 2

    def __init__(self, num_query_groups_per_partition: int, num_attention_heads_per_partition: int,
                 hidden_size_per_attention_head: int, q_layernorm=None, k_layernorm=None,
                 grouped_query_view: bool = True) -> None:
        super().__init__()
        if q_layernorm is not None or k_layernorm is not None:
            raise NotImplementedError("q/k layernorm is not used by the Llama-style layer")
        if num_attention_heads_per_partition % num_query_groups_per_partition:
            raise ValueError("query heads must be a multiple of KV groups")
        self.ng = num_query_groups_per_partition
        self.nq = num_attention_heads_per_partition
        self.hd = hidden_size_per_attention_head
        self.grouped_query_view = grouped_query_view

    def get_output_channels(self) -> List[Channel]:
        return [Channel(0, "main"), Channel(1, "key"), Channel(2, "value")]

    def split(self, mixed: torch.Tensor):
        ng, hd, per = self.ng, self.hd, self.nq // self.ng
        width = ng * (per + 2) * hd
        if mixed.shape[-1] != width:
            raise ValueError(f"fused QKV width {mixed.shape[-1]} != ng*(nq/ng+2)*hd = {width}")
        fused5 = mixed.view(*mixed.shape[:-1], ng, per + 2, hd)
        q, k, v = fused5[..., :per, :], fused5[..., per, :], fused5[..., per + 1, :]
        if not self.grouped_query_view:
            return q.reshape(*mixed.shape[:-1], self.nq, hd), k, v
        if mixed.is_contiguous():
            for t in (q, k, v):
                t._kr_fused5 = fused5
        return q, k, v

    def merge(self, gq: torch.Tensor, gk: torch.Tensor, gv: torch.Tensor) -> torch.Tensor:
        ng, hd, per = self.ng, self.hd, self.nq // self.ng
        mixed = getattr(gq, "_kr_mixed", None)
        if (mixed is not None and getattr(gk, "_kr_mixed", None) is mixed
                and getattr(gv, "_kr_mixed", None) is mixed):
            return mixed
        gq = gq.reshape(*gk.shape[:-1], per * hd)
        merged = torch.cat([gq, gk, gv], dim=-1)
        return merged.view(*merged.shape[:-2], ng * (per + 2) * hd)

    def fuser_forward(self, basic_op_ctxs, input_, *, basic_op_extra_inputs, basic_op_prev_ops,
                      basic_op_next_ops, basic_op_kwargs):
        q, k, v = self.split(input_)
        return q, [(k, v)]

    def fuser_backward(self, basic_op_ctxs, grad_output, *, basic_op_grad_extra_outputs):
        gk, gv = basic_op_grad_extra_outputs[0]
        return self.merge(grad_output, gk, gv), [()], [()]
