"""The two ends around the layer stack, so that a stack computes a loss from token ids:
embedding -> LayerStack -> final RMSNorm -> output layer -> cross entropy.

What the reference runs outside its partitions ("non-partition" work,
tests/bayesian/nonpartition/profile_nonpartition.py:148-486): ``LanguageModelEmbedding``
(3rdparty/Megatron-LM/megatron/core/models/common/embeddings/language_model_embedding.py:95-116,
word embeddings only — rotary positions — and the ``[b s h] -> [s b h]`` layout change), the
block's final layer norm (kareus/megatron/core/transformer/transformer_block.py:521-525), a
column-parallel output layer without bias, and ``compute_language_model_loss``
(3rdparty/Megatron-LM/megatron/core/models/common/language_module/language_module.py:71-101:
labels ``[b, s]``, logits ``[s, b, vocab]``, loss ``[b, s]``).

One GPU holds one vocabulary shard ``[vocab_start, vocab_start + vocab_rows)``.  The embedding
follows the shard semantics (ids of other shards embed to zero, which the missing all-reduce
would fill in); the loss treats the shard's columns as the whole vocabulary, which is exact for a
single shard and is what the per-shard kernels compute before the cross-shard max/sum exchange.
"""

from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor

from .backend import get_backend
from .block import LayerConfig, LayerStack


class _Embedding(torch.autograd.Function):
    @staticmethod
    def forward(ctx, ids, weight, vocab_start, backend):
        ctx.save_for_backward(ids)
        ctx.vocab_start, ctx.backend, ctx.rows = vocab_start, backend, weight.shape[0]
        return get_backend(backend).embedding_fwd(ids, weight.detach(), vocab_start)

    @staticmethod
    def backward(ctx, dout):
        (ids,) = ctx.saved_tensors
        return None, get_backend(ctx.backend).embedding_bwd(ids, dout, ctx.rows, ctx.vocab_start), None, None


class _RMSNorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, gamma, eps, backend):
        x2d = x.reshape(-1, x.shape[-1])
        y, rstd = get_backend(backend).rmsnorm_fwd(x2d, gamma.detach(), eps)
        ctx.save_for_backward(x2d, rstd, gamma)
        ctx.backend = backend
        return y.view(x.shape)

    @staticmethod
    def backward(ctx, dy):
        x2d, rstd, gamma = ctx.saved_tensors
        dx, dgamma = get_backend(ctx.backend).rmsnorm_bwd(dy.reshape(x2d.shape), x2d, rstd, gamma.detach())
        return dx.view(dy.shape), dgamma, None, None


class _Linear(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, backend):
        x2d = x.reshape(-1, x.shape[-1])
        ctx.save_for_backward(x2d, weight)
        ctx.backend = backend
        return get_backend(backend).linear_fwd(x2d, weight.detach()).view(*x.shape[:-1], weight.shape[0])

    @staticmethod
    def backward(ctx, dy):
        x2d, weight = ctx.saved_tensors
        be = get_backend(ctx.backend)
        dy2d = dy.reshape(-1, dy.shape[-1])
        if not dy2d.is_contiguous():
            dy2d = dy2d.contiguous()
        dx = be.linear_dgrad(dy2d, weight.detach())
        return dx.view(*dy.shape[:-1], weight.shape[1]), be.linear_wgrad(dy2d, x2d), None


class _CrossEntropy(torch.autograd.Function):
    """logits [s, b, vocab], labels [b, s] -> loss [b, s] (fp32).  Backward overwrites the logits
    with their gradient (they are dead after the loss), as the fused implementations do."""

    @staticmethod
    def forward(ctx, logits, labels, backend):
        s, b, vocab = logits.shape
        rows = labels.transpose(0, 1).contiguous().view(-1)            # [s, b] order, like the logits
        loss, lse = get_backend(backend).cross_entropy_fwd(logits.reshape(-1, vocab), rows)
        ctx.save_for_backward(logits, rows, lse)
        ctx.backend = backend
        return loss.view(s, b).transpose(0, 1).contiguous()

    @staticmethod
    def backward(ctx, dloss):
        logits, rows, lse = ctx.saved_tensors
        s, b, vocab = logits.shape
        g = dloss.transpose(0, 1).contiguous().view(-1)
        d = get_backend(ctx.backend).cross_entropy_bwd(logits.reshape(-1, vocab), rows, lse, g,
                                                       in_place=logits.is_contiguous())
        return d.view(s, b, vocab), None, None


class LanguageModelEmbedding(torch.nn.Module):
    """Word embeddings of one vocabulary shard; ``forward(input_ids [b, s]) -> [s, b, hidden]``."""

    def __init__(self, config: LayerConfig, vocab_rows: int, vocab_start: int = 0, device=None,
                 generator=None) -> None:
        super().__init__()
        w = torch.empty(vocab_rows, config.hidden_size, dtype=torch.float32)
        w.normal_(0.0, config.init_method_std, generator=generator)
        self.weight = torch.nn.Parameter(w.to(device=device, dtype=config.params_dtype))
        self.vocab_start, self._backend = int(vocab_start), config.backend

    def forward(self, input_ids: Tensor) -> Tensor:
        return _Embedding.apply(input_ids, self.weight, self.vocab_start, self._backend)


class GPTModelShard(torch.nn.Module):
    """``forward(input_ids [b, s], labels [b, s] or None)`` -> loss ``[b, s]`` (fp32) or logits
    ``[s, b, vocab_rows]``."""

    def __init__(self, config: LayerConfig, vocab_rows: int, vocab_start: int = 0, device=None,
                 seed: Optional[int] = None) -> None:
        super().__init__()
        gen = torch.Generator().manual_seed(seed + 1) if seed is not None else None
        self.config = config
        self.embedding = LanguageModelEmbedding(config, vocab_rows, vocab_start, device=device, generator=gen)
        self.decoder = LayerStack(config, device=device, seed=seed)
        self.final_layernorm = torch.nn.Parameter(
            torch.ones(config.hidden_size, device=device, dtype=config.params_dtype))
        w = torch.empty(vocab_rows, config.hidden_size, dtype=torch.float32)
        w.normal_(0.0, config.init_method_std, generator=gen)
        self.output_layer = torch.nn.Parameter(w.to(device=device, dtype=config.params_dtype))

    def forward(self, input_ids: Tensor, labels: Optional[Tensor] = None) -> Tensor:
        be = self.config.backend
        hidden = self.decoder(self.embedding(input_ids))
        hidden = _RMSNorm.apply(hidden, self.final_layernorm, self.config.layernorm_epsilon, be)
        logits = _Linear.apply(hidden, self.output_layer, be)
        if labels is None:
            return logits
        return _CrossEntropy.apply(logits, labels, be)
