"""Rotary position embedding on query and key.

``y = t cos f + rotate_half(t) sin f`` on the first ``rot_dim`` channels, halves
layout (not interleaved); backward is the rotation by ``-f``; the frequency table
gets no gradient (kareus/megatron/core/extensions/ops/rotary_embedding.py:50-171;
math kareus/megatron/core/models/common/embedding/rope_utils.py:147-222; the fused
path evaluates the trigonometry in fp32 from the fp32 table,
kareus/apex/transformer/functional/fused_rope.py:27-46).

When query and key arrive as views of one fused QKV buffer (as the QKV-split operator
hands them over) and the backend offers it, both are rotated in place with a single
launch; the fused buffer has no other reader, so nothing observes the overwrite.  The
same holds for the gradient views coming out of the attention backward.
"""

from __future__ import annotations

from typing import List

import torch

from ..backend import get_backend
from ..partitions.op_context import BasicOperation
from ..partitions.tensor_graph import Channel, PartitionableOperator


def rotary_frequencies(seq_len: int, dim: int, base: float = 10000.0, device=None) -> torch.Tensor:
    """``[s, 1, 1, dim]`` fp32 table ``cat(outer(pos, base^(-2i/dim)), same)``
    (3rdparty/Megatron-LM/megatron/core/models/common/embeddings/rotary_pos_embedding.py:
    76-78 inverse frequencies, :129 outer product, :161 concatenation, :167 shape)."""
    inv = 1.0 / (base ** (torch.arange(0, dim, 2, dtype=torch.float32, device=device) / dim))
    ang = torch.outer(torch.arange(seq_len, dtype=torch.float32, device=device), inv)
    return torch.cat((ang, ang), dim=-1)[:, None, None, :]


class RotaryEmbeddingOp(BasicOperation, PartitionableOperator):
    num_extra_inputs = 2
    num_extra_outputs = 1

    def __init__(self, config=None, backend="hip") -> None:
        super().__init__()
        self.config = config
        self._backend_name = backend

    def get_input_channels(self) -> List[Channel]:
        return [Channel(0, "main"), Channel(1, "key"), Channel(2, "rotary_pos_emb")]

    def get_output_channels(self) -> List[Channel]:
        return [Channel(0, "main"), Channel(1, "key")]

    @staticmethod
    def _shared_fused(a, b):
        fa, fb = getattr(a, "_kr_fused5", None), getattr(b, "_kr_fused5", None)
        return fa if (fa is not None and fa is fb) else None

    def fuser_forward(self, basic_op_ctxs, input_, *, basic_op_extra_inputs, basic_op_prev_ops,
                      basic_op_next_ops, basic_op_kwargs):
        key, freqs = basic_op_extra_inputs[0]
        if freqs is None or isinstance(freqs, tuple):
            raise ValueError("rotary_pos_emb cannot be None or a tuple of two tensors")
        if freqs.shape[0] < input_.shape[0]:
            raise ValueError(f"rotary table covers {freqs.shape[0]} positions, sequence has {input_.shape[0]}")
        ctx = basic_op_ctxs[0]
        be = get_backend(self._backend_name)
        fused = self._shared_fused(input_, key)
        if fused is not None and hasattr(be, "rope_fused_inplace"):
            be.rope_fused_inplace(fused, fused.shape[3] - 2, freqs, False)
            q_out, k_out = input_, key
        else:
            q_out = be.rope_fwd(input_, freqs)
            k_out = be.rope_fwd(key, freqs)
        if ctx.requires_grad:
            ctx.save_for_backward(freqs)
        return q_out, [(k_out,)]

    def fuser_backward(self, basic_op_ctxs, grad_output, *, basic_op_grad_extra_outputs):
        (freqs,) = basic_op_ctxs[0].saved_tensors
        (grad_key,) = basic_op_grad_extra_outputs[0]
        be = get_backend(self._backend_name)
        fused = self._shared_fused(grad_output, grad_key)
        if fused is not None and hasattr(be, "rope_fused_inplace"):
            be.rope_fused_inplace(fused, fused.shape[3] - 2, freqs, True)
            dq, dk = grad_output, grad_key
        else:
            dq = be.rope_bwd(grad_output, freqs)
            dk = be.rope_bwd(grad_key, freqs)
        return dq, [()], [(dk, None)]
