"""The four partitions of a decoder layer as stand-alone, repeatable units.

Each ``PartitionTest`` owns the operators of one partition kind, synthetic tensors of one
nanobatch, a hand-over operator and a ``PartitionExecutor``; ``test_config(overlap_window,
sm_configs)`` runs the partition once.  Follows the reference's per-partition drivers
(tests/bayesian/partitions/{fwd_attn,fwd_mlp,bwd_attn,bwd_mlp}/overlap_test.py:
``PartitionTest.__init__`` builds tensors, operators and executor; ``test_config`` calls
``executor.execute``), with the operator lists the engine itself cuts out of a layer:

    fwd_attn  fork, norm, qkv, qkv-post, rope, attention, proj          | all-reduce(main)
    fwd_mlp   bias-dropout-add, fork, norm, fc1, swiglu, fc2            | all-reduce(main)
    bwd_mlp   gradients of  fc1, swiglu, fc2, bias-dropout-add          | all-reduce(grad_main)
    bwd_attn  gradients of  qkv, qkv-post, rope, attention, proj,
              bias-dropout-add, fork, norm                             | all-reduce(grad_main)

Synthetic data as in the reference drivers: N(0,1) activations and gradients of shape
``[seq, batch / nanobatches, hidden]``, rotary table from positions 0..seq-1.
"""

from __future__ import annotations

from typing import Dict, List, Tuple

import torch

from ..block import DecoderLayer, LayerConfig
from ..operators import NoOpAllReduce
from ..operators.rotary_embedding import rotary_frequencies
from ..partitions.partition_base import _build_overlap_slots
from ..partitions.streams import stream_api
from ..partitions.tensor_graph import CommunicationType
from .partition_executor import PartitionExecutor

PARTITION_KEYS = ("fwd_attn", "fwd_mlp", "bwd_mlp", "bwd_attn")


def _operators(layer: DecoderLayer, key: str) -> List:
    attn = [layer.linear_qkv, layer.qkv_postprocess, layer.rotary, layer.core_attention, layer.linear_proj]
    mlp = [layer.linear_fc1, layer.activation, layer.linear_fc2]
    if key == "fwd_attn":
        return [layer.attn_residual_fork, layer.input_layernorm] + attn
    if key == "fwd_mlp":
        return [layer.self_attn_bda, layer.mlp_residual_fork, layer.pre_mlp_layernorm] + mlp
    if key == "bwd_mlp":
        return mlp + [layer.mlp_bda]
    if key == "bwd_attn":
        return attn + [layer.self_attn_bda, layer.mlp_residual_fork, layer.pre_mlp_layernorm]
    raise ValueError(f"unknown partition key {key!r}; expected one of {PARTITION_KEYS}")


class PartitionTest:
    def __init__(self, key: str, config: LayerConfig, batch_size: int, seq_len: int,
                 device=None, seed: int = 1234) -> None:
        if batch_size % config.num_nanobatches:
            raise ValueError("batch_size must be a multiple of config.num_nanobatches")
        self.key, self.config = key, config
        self.device = torch.device(device) if device is not None else torch.device("cpu")
        self.dtype = config.params_dtype
        self.seq_length, self.batch_size = seq_len, batch_size
        self.nano_batch_size = batch_size // config.num_nanobatches
        gen = torch.Generator().manual_seed(seed)
        self.layer = DecoderLayer(config, 1, device=self.device, generator=gen)
        self.comp_ops = _operators(self.layer, key)
        self._gen = gen

        api = stream_api()
        self.comm_stream = api.new_stream() if (self.device.type == "cuda" and api.available()) else None
        self.comm_op = NoOpAllReduce(batch_idx=0, world_size=1, comm_stream=self.comm_stream)

        backward = key.startswith("bwd")
        fwd_names = {"fwd_attn": ["main", "rotary_pos_emb"], "fwd_mlp": ["main", "residual"],
                     "bwd_mlp": ["main", "residual"],
                     "bwd_attn": ["main", "residual", "rotary_pos_emb"]}[key]
        bwd_names = {"bwd_mlp": ["grad_main"], "bwd_attn": ["grad_main", "grad_residual"]}.get(key)
        self.executor = PartitionExecutor(
            operators=self.comp_ops,
            comm_operator=self.comm_op,
            direction="backward" if backward else "forward",
            partition_key=key,
            comm_type=CommunicationType.ALL_REDUCE,
            initial_channel_names=bwd_names if backward else fwd_names,
            fwd_initial_channel_names=fwd_names if backward else None,
        )
        self.forward_tensors = {name: self._tensor(name) for name in fwd_names}
        self.handover = self._randn(self.config.hidden_size)
        if backward:
            self.executor.run_forward_setup(self.forward_tensors)
            self.grad_tensors = {name: self._randn(self.config.hidden_size, grad=False) for name in bwd_names}
            self.executor.setup_contexts(self.grad_tensors, [self.handover])
        else:
            self.executor.setup_contexts(self.forward_tensors, [self.handover])

    # -- synthetic inputs -----------------------------------------------------------
    def _randn(self, width: int, grad: bool = True) -> torch.Tensor:
        t = torch.randn(self.seq_length, self.nano_batch_size, width, generator=self._gen)
        t = t.to(self.device, self.dtype)
        return t.requires_grad_(True) if grad else t

    def _tensor(self, channel: str) -> torch.Tensor:
        c = self.config
        if channel == "rotary_pos_emb":
            return rotary_frequencies(self.seq_length, c.kv_channels, c.rotary_base, device=self.device)
        return self._randn(c.hidden_size)  # "main" (a partition's first op reads hidden-width rows) / "residual"

    # -- what a sweep may ask for -----------------------------------------------------
    @property
    def overlap_slots(self) -> Dict[str, int]:
        return dict(_build_overlap_slots(self.executor.partition.comp_ops))

    @property
    def overlap_windows(self) -> List[Tuple[str, str]]:
        """Every release point this partition has, earliest first, then ``("none", "none")``
        (release after the partition's last op)."""
        slots = sorted(self.overlap_slots.items(), key=lambda kv: kv[1])
        return [(name, "none") for name, _ in slots] + [("none", "none")]

    def test_config(self, overlap_window, sm_configs):
        return self.executor.execute(tuple(overlap_window), tuple(sm_configs))
