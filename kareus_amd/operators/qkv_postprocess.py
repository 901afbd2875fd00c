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

With ``q_layernorm`` and ``k_layernorm`` (Qwen3-style models: an RMSNorm over the head
dimension of every query head and one over every key head, qkv_postprocess.py:115-118,
backward :150-157) one kernel writes a second fused buffer with the query and key heads
normalised and the value heads copied, and the three outputs are views of that buffer, so
everything downstream works as without the norms; the backward rewrites the query and key
heads of the merged gradient in place and returns the two weight gradients, query first.
"""

from __future__ import annotations

from typing import List

import torch

from ..backend import get_backend
from ..partitions.op_context import BasicOperation
from ..partitions.tensor_graph import Channel, PartitionableOperator


class QKVPostProcessOp(BasicOperation, PartitionableOperator):
    num_extra_outputs = 2

    def __init__(self, num_query_groups_per_partition: int, num_attention_heads_per_partition: int,
                 hidden_size_per_attention_head: int, q_layernorm=None, k_layernorm=None,
                 grouped_query_view: bool = True, backend="hip") -> None:
        super().__init__()
        if (q_layernorm is None) != (k_layernorm is None):
            raise NotImplementedError("q_layernorm and k_layernorm come as a pair (qk_layernorm) or not at all")
        for norm in (q_layernorm, k_layernorm):
            if norm is None:
                continue
            if getattr(norm, "bias", None) is not None or isinstance(norm, torch.nn.LayerNorm):
                raise NotImplementedError("q/k layernorm: only an RMSNorm (no mean subtraction, no bias) is supported")
            weight = getattr(norm, "weight", None)
            if weight is None or tuple(weight.shape) != (hidden_size_per_attention_head,) or not hasattr(norm, "eps"):
                raise ValueError("q/k layernorm must be an RMSNorm over the head dimension "
                                 f"({hidden_size_per_attention_head} channels) with a weight and an eps")
        if q_layernorm is not None and float(q_layernorm.eps) != float(k_layernorm.eps):
            raise ValueError("q_layernorm and k_layernorm must share one epsilon")
        self.q_layernorm = q_layernorm   # (registered in this order: the weight gradients come back query first)
        self.k_layernorm = k_layernorm
        self._backend_name = backend
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
        if self.q_layernorm is None:
            q, k, v = self.split(input_)
            return q, [(k, v)]
        ng, hd, per = self.ng, self.hd, self.nq // self.ng
        if input_.shape[-1] != ng * (per + 2) * hd:
            raise ValueError(f"fused QKV width {input_.shape[-1]} != ng*(nq/ng+2)*hd = {ng * (per + 2) * hd}")
        mixed = input_.contiguous()
        be = get_backend(self._backend_name)
        # (the leading dimensions, [s, b] in the layer, are all tokens to the norm)
        normed5, rstd = be.qk_norm_fwd(mixed.view(-1, 1, ng, per + 2, hd), self.q_layernorm.weight.detach(),
                                       self.k_layernorm.weight.detach(), float(self.q_layernorm.eps))
        ctx = basic_op_ctxs[0]
        if ctx.requires_grad:
            ctx.save_for_backward(mixed, rstd)
        q, k, v = self.split(normed5.view(mixed.shape))
        return q, [(k, v)]

    def fuser_backward(self, basic_op_ctxs, grad_output, *, basic_op_grad_extra_outputs):
        gk, gv = basic_op_grad_extra_outputs[0]
        merged = self.merge(grad_output, gk, gv)
        if self.q_layernorm is None:
            return merged, [()], [()]
        mixed, rstd = basic_op_ctxs[0].saved_tensors
        ng, hd, per = self.ng, self.hd, self.nq // self.ng
        merged = merged.contiguous()
        be = get_backend(self._backend_name)
        dmixed5, dgq, dgk = be.qk_norm_bwd(merged.view(-1, 1, ng, per + 2, hd), mixed.view(-1, 1, ng, per + 2, hd), rstd,
                                           self.q_layernorm.weight.detach(), self.k_layernorm.weight.detach())
        return dmixed5.view(mixed.shape), [(dgq, dgk)], [()]
