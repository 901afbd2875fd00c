"""Block driver: builds the operators of L decoder layers, wires them into the
forward and backward graphs, forms the nanobatch partitions, and runs them through
the single autograd node.

This stands where the reference's ``TransformerBlock`` stands, without Megatron:
graph and partition construction follow
kareus/megatron/core/transformer/transformer_block.py:135-218 (op collection, the
two graphs with forward op ids reused by the backward specs, partition keys, seed
config), binding of the per-nanobatch collective operators :220-267, parameter
order :376-390, and ``forward`` :405-527 (guards, split on the batch axis, one
``apply`` with the parameters repeated per nanobatch, concatenation).  Operator
order inside a layer is kareus/megatron/core/transformer/transformer_layer.py:148-174.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, List, Optional

import torch

from .operators import (
    BiasDropoutAddOp,
    BiasSwigluOp,
    NoOpAllReduce,
    PartitionableRMSNorm,
    QKVPostProcessOp,
    RMSNorm,
    ResidualForkOp,
    RotaryEmbeddingOp,
    TEColumnParallelLinearOp,
    TEDotProductAttentionOp,
    TERowParallelLinearOp,
    rotary_frequencies,
)
from .partitions.op_context import operator_parameters
from .partitions.streams import stream_api
from .partitions import (
    CommunicationType,
    ComputeOp,
    ComputeOpSpec,
    PartitionBuilder,
    SeedConfig,
    TensorGraphBuilder,
    TransformerBlockAutogradFunction,
)


@dataclass
class LayerConfig:
    """Shapes of one GPU's shard of a Llama-style decoder layer.

    ``num_attention_heads`` / ``num_query_groups`` / ``ffn_hidden_size`` are the
    per-shard counts (e.g. 8 of 32 query heads, 2 of 8 KV heads, 3584 of 14336 FFN
    columns for a TP=4 shard); ``hidden_size`` is never sharded.
    """

    hidden_size: int
    num_attention_heads: int
    num_query_groups: int
    kv_channels: int
    ffn_hidden_size: int
    num_layers: int = 1
    layernorm_epsilon: float = 1e-5
    rotary_base: float = 500000.0
    init_method_std: float = 0.02
    num_nanobatches: int = 2
    params_dtype: torch.dtype = torch.bfloat16
    backend: str = "hip"
    use_streams: bool = True
    checkpoint_activations: bool = False
    # weight gradients of all nanobatches are summed inside the wgrad GEMM instead of by autograd
    fuse_wgrad_accumulation: bool = True
    # ... and, where the backend can contract operand pieces, by ONE GEMM per layer over the tokens of all
    # nanobatches, launched when the last nanobatch has delivered its operands (instead of one
    # accumulating GEMM per nanobatch); the nanobatches' operands stay alive until then
    wgrad_over_all_nanobatches: bool = True
    # ... and those launches are issued at the end of the backward pass, behind every nanobatch's input
    # gradients, instead of where the last nanobatch delivers its operands.  A launch in the middle puts one
    # nanobatch's stream out of step with the others; with four nanobatches of one sequence, whose attention
    # and out-projection kernels fill the device only beside each other, keeping them in step is worth 4 % of
    # the step (8B shard), with two wide nanobatches the launches fill gaps where they are (3B shard: 2 % the
    # other way).  None: at the end from four nanobatches on.
    wgrad_launches_at_end: Optional[bool] = None
    # nanobatch outputs (and input gradients) are written into slices of one tensor by the ops
    # that produce them, so joining the nanobatches needs no concatenation
    join_nanobatches_in_place: bool = True
    # HBM passes folded into GEMM epilogues: the SwiGLU activation into fc1, its backward into fc2's
    # input-gradient GEMM, and (one GPU only: no sum over ranks has to come first) the residual adds
    # into the out-projection and fc2
    fuse_forward_epilogues: bool = True
    hidden_dropout: float = 0.0
    attention_dropout: float = 0.0
    add_bias_linear: bool = False
    # an RMSNorm over the head dimension of every query head and of every key head, between the QKV split
    # and the rotary embedding (Qwen3-style models)
    qk_layernorm: bool = False
    # Filled in by the driver / the training loop:
    kareus_scheduler: Optional[Any] = None
    nanobatch_streams: Optional[List[Any]] = field(default=None, repr=False)

    @property
    def qkv_width(self) -> int:
        return (self.num_attention_heads + 2 * self.num_query_groups) * self.kv_channels


def _dense_batch_slices(parts, backend: str = "eager") -> bool:
    """Whether nanobatch slices of this width must be copied.  A nanobatch of one sequence is a matrix
    with row stride ``b*h``; one of 2, 4, 8 or 16 sequences has its rows in runs, which the HIP kernels
    at the two ends of a layer stack address in place (``rows_view``); anything else is copied once."""
    from .backend import get_backend

    view = get_backend(backend).rows_view
    return any(view(p) is None for p in parts)


def _whole_of(parts):
    """The ``[s, b, h]`` tensor of which ``parts`` are the consecutive batch slices, if they are
    exactly that (same storage, strides of the whole, back to back); else None."""
    first = parts[0]
    if first.dim() != 3:
        return None
    s, _, h = first.shape
    b = sum(p.shape[1] for p in parts)
    want = (b * h, h, 1)
    storage, offset = first.untyped_storage().data_ptr(), first.storage_offset()
    for p in parts:
        if (p.dim() != 3 or p.shape[0] != s or p.shape[2] != h or p.dtype != first.dtype
                or p.untyped_storage().data_ptr() != storage or p.storage_offset() != offset):
            return None
        if any(p.shape[d] > 1 and p.stride(d) != want[d] for d in range(3)):
            return None
        offset += p.shape[1] * h
    return first.as_strided((s, b, h), want, first.storage_offset())


class _SplitNanobatches(torch.autograd.Function):
    """``[s, b, h] -> n x [s, b/n, h]`` along the batch dimension (the reference slices with
    ``hidden_states[:, i*nb:(i+1)*nb]``, transformer_block.py:405-527).

    A nanobatch of one sequence is a matrix with row stride ``b*h``; every kernel that touches it
    takes a row stride, so it stays a view.  Wider nanobatches cannot be addressed with a single
    row stride and are copied into dense tensors once.  Backward hands back the tensor the n
    gradients are slices of when the engine wrote them side by side, else concatenates them
    (one copy instead of autograd's zero-fill + copy + add per slice)."""

    @staticmethod
    def forward(ctx, hidden_states, n, backend="eager"):
        nb = hidden_states.shape[1] // n
        parts = [hidden_states[:, i * nb:(i + 1) * nb] for i in range(n)]
        if _dense_batch_slices(parts, backend):
            parts = [p.contiguous() for p in parts]
        return tuple(parts)

    @staticmethod
    def backward(ctx, *grads):
        whole = _whole_of(grads)
        return (whole if whole is not None else torch.cat(grads, dim=1)), None, None


class _JoinNanobatches(torch.autograd.Function):
    """``n x [s, b/n, h] -> [s, b, h]``: the reference concatenates
    (transformer_block.py:405-527); when the engine already wrote the nanobatch outputs side by
    side into one tensor that tensor is the result and nothing is copied.  Backward slices the
    gradient the way ``_SplitNanobatches`` slices the input."""

    @staticmethod
    def forward(ctx, backend, *outs):
        ctx.widths = [o.shape[1] for o in outs]
        ctx.backend = backend
        whole = _whole_of(outs)
        return whole if whole is not None else torch.cat(outs, dim=1)

    @staticmethod
    def backward(ctx, grad):
        if grad.stride(2) != 1 or grad.stride(1) != grad.shape[2] or grad.stride(0) != grad.shape[1] * grad.shape[2]:
            grad = grad.contiguous()
        parts, lo = [], 0
        for w in ctx.widths:
            parts.append(grad[:, lo:lo + w])
            lo += w
        if _dense_batch_slices(parts, ctx.backend):
            parts = [p.contiguous() for p in parts]
        return (None, *parts)


class DecoderLayer(torch.nn.Module):
    """Holds one layer's operators and states their execution order; it has no
    ``forward`` of its own — the partition engine runs the operators."""

    def __init__(self, config: LayerConfig, layer_number: int, device=None, generator=None) -> None:
        super().__init__()
        c, be, dt = config, config.backend, config.params_dtype

        def init(w: torch.Tensor) -> None:
            # Drawn in fp32 on the host and cast, so every backend/device sees the
            # same values for a given generator state.
            vals = torch.empty(w.shape, dtype=torch.float32).normal_(0.0, c.init_method_std, generator=generator)
            w.copy_(vals.to(w.dtype))

        lin = dict(config=c, init_method=init, bias=False, device=device, dtype=dt, backend=be)
        self.attn_residual_fork = ResidualForkOp(backend=be)
        self.input_layernorm = PartitionableRMSNorm(c.hidden_size, c.layernorm_epsilon, device=device, dtype=dt, backend=be)
        self.linear_qkv = TEColumnParallelLinearOp(c.hidden_size, c.qkv_width, skip_bias_add=False, **lin)
        head_norm = (lambda: RMSNorm(c.kv_channels, c.layernorm_epsilon, device=device, dtype=dt, backend=be)
                     ) if c.qk_layernorm else (lambda: None)
        self.qkv_postprocess = QKVPostProcessOp(c.num_query_groups, c.num_attention_heads, c.kv_channels,
                                                q_layernorm=head_norm(), k_layernorm=head_norm(), backend=be)
        self.rotary = RotaryEmbeddingOp(config=c, backend=be)
        self.core_attention = TEDotProductAttentionOp(config=c, layer_number=layer_number, backend=be,
                                                      attention_dropout=c.attention_dropout)
        self.linear_proj = TERowParallelLinearOp(c.num_attention_heads * c.kv_channels, c.hidden_size,
                                                 skip_bias_add=True, **lin)
        self.self_attn_bda = BiasDropoutAddOp(has_bias=c.add_bias_linear, dropout_prob=c.hidden_dropout, backend=be)
        self.mlp_residual_fork = ResidualForkOp(backend=be)
        self.pre_mlp_layernorm = PartitionableRMSNorm(c.hidden_size, c.layernorm_epsilon, device=device, dtype=dt, backend=be)
        self.linear_fc1 = TEColumnParallelLinearOp(c.hidden_size, 2 * c.ffn_hidden_size, skip_bias_add=True, **lin)
        self.activation = BiasSwigluOp(has_bias=c.add_bias_linear, backend=be)
        self.linear_fc2 = TERowParallelLinearOp(c.ffn_hidden_size, c.hidden_size, skip_bias_add=True, **lin)
        self.mlp_bda = BiasDropoutAddOp(has_bias=c.add_bias_linear, dropout_prob=c.hidden_dropout, backend=be)
        fuse = bool(getattr(c, "fuse_forward_epilogues", False))
        self.linear_fc1.fuse_activation = fuse    # SwiGLU forward in fc1's epilogue
        self.linear_fc2.fuse_activation = fuse    # SwiGLU backward in the epilogue of fc2's input gradient
        # (with hidden dropout the residual is added behind the dropout, by the op that follows)
        for row_parallel in (self.linear_proj, self.linear_fc2):
            row_parallel.fuse_residual = fuse and c.hidden_dropout == 0.0
            row_parallel.forward_accepts_out_sink = fuse and c.hidden_dropout == 0.0

    def get_all_operators(self) -> List:
        return [
            self.attn_residual_fork, self.input_layernorm,
            self.linear_qkv, self.qkv_postprocess, self.rotary, self.core_attention, self.linear_proj,
            self.self_attn_bda,
            self.mlp_residual_fork, self.pre_mlp_layernorm,
            self.linear_fc1, self.activation, self.linear_fc2,
            self.mlp_bda,
        ]

    def forward(self, *args, **kwargs):
        raise RuntimeError("DecoderLayer is executed by the partition engine, not called directly")


class LayerStack(torch.nn.Module):
    """``forward(hidden_states [s, b, h], attention_mask=None, rotary_pos_emb [s,1,1,hd])``."""

    def __init__(self, config: LayerConfig, device=None, seed: Optional[int] = None) -> None:
        super().__init__()
        if config.num_nanobatches < 1:
            raise ValueError("num_nanobatches must be >= 1")
        self.config = config
        gen = torch.Generator().manual_seed(seed) if seed is not None else None
        self.layers = torch.nn.ModuleList(
            DecoderLayer(config, i + 1, device=device, generator=gen) for i in range(config.num_layers)
        )
        self._build_partitions()
        self.set_tensor_parallel_group(None)

    @property
    def scheduler(self):
        return getattr(self.config, "kareus_scheduler", None)

    # -- graph / partitions -------------------------------------------------------
    def _build_partitions(self) -> None:
        ops: List = []
        for layer in self.layers:
            ops.extend(layer.get_all_operators())

        fwd = TensorGraphBuilder()
        fwd.add_initial_channels({"main": "ext_main", "rotary_pos_emb": "ext_rotary_pos_emb"})
        op_id_of = {}
        for op in ops:
            for spec in op.get_forward_ops():
                node = fwd.add_op(spec)
                if isinstance(node, ComputeOp):
                    op_id_of[id(spec.operator)] = node.op_id
        self.forward_tensor_graph = fwd.build()

        bwd = TensorGraphBuilder()
        bwd.add_initial_channels({"grad_main": "ext_grad_main"})
        for op in reversed(ops):
            for spec in op.get_backward_ops():
                if isinstance(spec, ComputeOpSpec) and spec.op_id is None:
                    spec.op_id = op_id_of.get(id(spec.operator))
                bwd.add_op(spec)
        self.backward_tensor_graph = bwd.build()

        n, num_layers = self.config.num_nanobatches, len(self.layers)
        trail_rest = [""] * (n - 1)
        fwd_keys = (["fwd_attn"] * n + ["fwd_mlp"] * n) * num_layers + ["fwd_trail"] + trail_rest
        bwd_keys = (["bwd_mlp"] * n + ["bwd_attn"] * n) * num_layers + ["bwd_trail"] + trail_rest
        builder = PartitionBuilder(self.forward_tensor_graph, self.backward_tensor_graph, num_nanobatches=n)
        self.forward_partitions = builder.build_forward_partitions(partition_keys=fwd_keys)
        self.backward_partitions = builder.build_backward_partitions(partition_keys=bwd_keys)
        self.seed_config = SeedConfig()

    def _assign_comm_operators(self, comm_type, comm_ops) -> None:
        for part in self.forward_partitions + self.backward_partitions:
            if part.comm_op is not None and part.comm_op.comm_type == comm_type:
                part.comm_op.operator = comm_ops[part.nano_batch_idx]

    def set_tensor_parallel_group(self, tp_group=None) -> None:
        """Bind one schedule-point operator per nanobatch.  The operator bound to
        nanobatch *i*'s partitions hands over nanobatch *i-1*'s tensor, so its
        'communication stream' is nanobatch *i-1*'s compute stream."""
        if tp_group is not None:
            raise NotImplementedError("one GPU: the tensor-parallel group has a single member")
        n = self.config.num_nanobatches
        streams = self._streams()
        for layer in self.layers:
            for op in (layer.linear_qkv, layer.linear_proj, layer.linear_fc1, layer.linear_fc2):
                op.split_k = streams is None
            # with several nanobatches the attention launches take the forms that cost the least compute-unit
            # time (no split of the keys at small batches), which is what counts beside the other nanobatch
            # streams: 0.4-0.9 % of the nanobatched step on the 3B and 8B layers.  The choice follows the
            # nanobatch count, not the streams, so that a run on one stream gives the bits of a run on several.
            layer.core_attention.beside_other_streams = n > 1
        self.allreduce_comm_ops = [
            NoOpAllReduce(batch_idx=i, world_size=1, comm_stream=streams[(i - 1) % n] if streams else None)
            for i in range(n)
        ]
        self._assign_comm_operators(CommunicationType.ALL_REDUCE, self.allreduce_comm_ops)

    def _streams(self):
        c = self.config
        api = stream_api()
        if not c.use_streams or c.num_nanobatches < 2 or not api.available():
            c.nanobatch_streams = None
            return None
        if c.nanobatch_streams is None:
            many = getattr(api, "new_streams", None)
            c.nanobatch_streams = (many(c.num_nanobatches) if many is not None
                                   else [api.new_stream() for _ in range(c.num_nanobatches)])
        return c.nanobatch_streams

    def _get_all_params(self) -> List[torch.nn.Parameter]:
        params: List[torch.nn.Parameter] = []
        for layer in self.layers:
            for op in layer.get_all_operators():
                params.extend(operator_parameters(op))
        return params

    def rotary_pos_emb(self, seq_len: int, device=None) -> torch.Tensor:
        """The fp32 rotary table [s, 1, 1, hd]; built once per (length, device) and kept."""
        key = (seq_len, str(device))
        cache = self.__dict__.setdefault("_rotary_cache", {})
        if key not in cache:
            cache.clear()  # one table at a time is enough: the sequence length rarely changes
            cache[key] = rotary_frequencies(seq_len, self.config.kv_channels, self.config.rotary_base,
                                            device=device)
        return cache[key]

    # -- execution ----------------------------------------------------------------
    def forward(self, hidden_states: torch.Tensor, attention_mask=None, rotary_pos_emb=None,
                **unsupported) -> torch.Tensor:
        for name, value in unsupported.items():
            if value is not None:
                raise NotImplementedError(f"{name} is not supported by the partition engine")
        if attention_mask is not None:
            raise NotImplementedError("the causal mask is implicit; pass attention_mask=None")
        if isinstance(rotary_pos_emb, tuple):
            raise NotImplementedError("a (q, k) pair of rotary tables is not supported")
        if hidden_states.dim() != 3 or hidden_states.shape[2] != self.config.hidden_size:
            raise ValueError(f"hidden_states must be [s, b, {self.config.hidden_size}]")
        n = self.config.num_nanobatches
        s, b, _ = hidden_states.shape
        if b < n or b % n:
            raise ValueError(f"batch size {b} must be a positive multiple of {n} nanobatches")
        if rotary_pos_emb is None:
            rotary_pos_emb = self.rotary_pos_emb(s, device=hidden_states.device)

        hs = _SplitNanobatches.apply(hidden_states, n, self.config.backend) if n > 1 else (hidden_states,)
        params = self._get_all_params()
        outs = TransformerBlockAutogradFunction.apply(
            *hs, rotary_pos_emb, None,
            self.forward_partitions, self.backward_partitions,
            self.forward_tensor_graph, self.backward_tensor_graph,
            self.scheduler, self.config, self.seed_config,
            torch.is_grad_enabled(), self.config.checkpoint_activations,
            *(params * n),
        )
        return outs[0] if n == 1 else _JoinNanobatches.apply(self.config.backend, *outs)
