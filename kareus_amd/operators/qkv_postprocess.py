"""Splits the fused QKV projection into query, key and value.

The projection's output features are grouped per KV group ``g`` as
``[q heads of g ..., k_g, v_g]``: ``[s, b, ng * (nq/ng + 2) * hd]`` is viewed as
``[s, b, ng, (nq/ng + 2) * hd]`` and cut along the last axis.  Forward only makes
views; backward reassembles the three gradients into one tensor
(kareus/megatron/core/extensions/ops/qkv_postprocess.py:84-127, 164-184).
"""

from __future__ import annotations

from typing import List

import torch

from ..partitions.op_context import BasicOperation
from ..partitions.tensor_graph import Channel, PartitionableOperator


class QKVPostProcessOp(BasicOperation, PartitionableOperator):
    num_extra_outputs = 2

    def __init__(self, num_query_groups_per_partition: int, num_attention_heads_per_partition: int,
                 hidden_size_per_attention_head: int, q_layernorm=None, k_layernorm=None) -> None:
        super().__init__()
        if q_layernorm is not None or k_layernorm is not None:
            raise NotImplementedError("q/k layernorm is not used by the Llama-style layer")
        if num_attention_heads_per_partition % num_query_groups_per_partition:
            raise ValueError("query heads must be a multiple of KV groups")
        self.ng = num_query_groups_per_partition
        self.nq = num_attention_heads_per_partition
        self.hd = hidden_size_per_attention_head

    def get_output_channels(self) -> List[Channel]:
        return [Channel(0, "main"), Channel(1, "key"), Channel(2, "value")]

    def split(self, mixed: torch.Tensor):
        ng, hd, per = self.ng, self.hd, self.nq // self.ng
        width = ng * (per + 2) * hd
        if mixed.shape[-1] != width:
            raise ValueError(f"fused QKV width {mixed.shape[-1]} != ng*(nq/ng+2)*hd = {width}")
        grouped = mixed.view(*mixed.shape[:-1], ng, (per + 2) * hd)
        q, k, v = torch.split(grouped, [per * hd, hd, hd], dim=-1)
        q = q.unflatten(-1, (per, hd)).flatten(-3, -2)  # [s, b, nq, hd], still a view
        return q, k, v

    def merge(self, gq: torch.Tensor, gk: torch.Tensor, gv: torch.Tensor) -> torch.Tensor:
        ng, hd, per = self.ng, self.hd, self.nq // self.ng
        gq = gq.reshape(*gq.shape[:-2], ng, per * hd)
        merged = torch.cat([gq, gk, gv], dim=-1)
        return merged.view(*merged.shape[:-2], ng * (per + 2) * hd)

    def fuser_forward(self, basic_op_ctxs, input_, *, basic_op_extra_inputs, basic_op_prev_ops,
                      basic_op_next_ops, basic_op_kwargs):
        q, k, v = self.split(input_)
        return q, [(k, v)]

    def fuser_backward(self, basic_op_ctxs, grad_output, *, basic_op_grad_extra_outputs):
        gk, gv = basic_op_grad_extra_outputs[0]
        return self.merge(grad_output, gk, gv), [()], [()]
