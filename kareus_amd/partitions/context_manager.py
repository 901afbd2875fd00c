"""Per-nanobatch run-time state: the tensor table and the per-op contexts.

A partition computing nanobatch *i* reads and writes ``ctx.tensor_store`` of that
nanobatch; the schedule point it carries touches the store of the nanobatch whose
tensor it hands over (``pre_ctx``).  Semantics follow
kareus/megatron/core/partitions/context_manager.py: store get/set with a
descriptive ``KeyError`` ``:43-56``, op-context creation and lookup ``:101-126``,
flatten/restore of saved tensors in ``op_id`` order ``:128-171``, recompute
finalisation ``:173-186`` and selective clearing ``:188-206``.

Two additions serve the one-GPU engine: a context may own a HIP stream (all work of
its nanobatch is enqueued there), and the store remembers which ids need gradients
so the engine never has to flip ``requires_grad`` on tensors produced inside an
autograd ``Function``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Sequence, Tuple

import torch

from .op_context import OperationContext, clear_tensor_data


@dataclass
class TensorStore:
    """Tensor-id -> tensor table of one nanobatch."""

    _tensors: Dict[str, torch.Tensor] = field(default_factory=dict)
    _needs_grad: Dict[str, bool] = field(default_factory=dict)

    def set(self, tensor_id: str, tensor: torch.Tensor, requires_grad: Optional[bool] = None) -> None:
        self._tensors[tensor_id] = tensor
        if requires_grad is None:
            requires_grad = bool(getattr(tensor, "requires_grad", False))
        self._needs_grad[tensor_id] = requires_grad

    def get(self, tensor_id: str) -> torch.Tensor:
        try:
            return self._tensors[tensor_id]
        except KeyError:
            raise KeyError(
                f"TensorStore: tensor_id '{tensor_id}' not found. "
                f"Available ids: {sorted(self._tensors)}"
            ) from None

    def needs_grad(self, tensor_id: str) -> bool:
        return self._needs_grad.get(tensor_id, False)

    def __contains__(self, tensor_id: str) -> bool:
        return tensor_id in self._tensors

    def get_by_ports(self, ports: Sequence[Any]) -> List[torch.Tensor]:
        return [self.get(p.tensor_id) for p in ports]

    def set_from_ports(self, ports: Sequence[Any], tensors: Sequence[Optional[torch.Tensor]]) -> None:
        for port, tensor in zip(ports, tensors):
            if tensor is not None:
                self.set(port.tensor_id, tensor)


@dataclass
class NanoBatchContext:
    """Everything one nanobatch carries across partitions.

    Life cycle: forward ops obtain a fresh ``OperationContext`` each
    (``create_op_context``) -> ``flatten_saved_tensors`` hands their ``to_save``
    lists to autograd -> ``restore_saved_tensors`` slices them back at the start of
    backward -> backward ops look their context up by the same ``op_id``.
    """

    batch_idx: int
    tensor_store: TensorStore = field(default_factory=TensorStore)
    op_contexts: Dict[int, OperationContext] = field(default_factory=dict)
    stream: Optional[Any] = None  # torch.cuda.Stream this nanobatch runs on (None: caller's)
    # op_id -> tensor that op's forward output is to be written into (consumed when the op runs)
    output_sinks: Dict[int, torch.Tensor] = field(default_factory=dict)
    _saved_tensors: List[Optional[torch.Tensor]] = field(default_factory=list)
    _saved_ranges: Dict[int, Tuple[int, int]] = field(default_factory=dict)

    def create_op_context(self, op_id: int) -> OperationContext:
        ctx = OperationContext()
        self.op_contexts[op_id] = ctx
        return ctx

    def get_op_context(self, op_id: int) -> OperationContext:
        return self.op_contexts[op_id]

    def flatten_saved_tensors(self) -> List[Optional[torch.Tensor]]:
        flat: List[Optional[torch.Tensor]] = []
        ranges: Dict[int, Tuple[int, int]] = {}
        for op_id in sorted(self.op_contexts):
            ctx = self.op_contexts[op_id]
            if ctx.to_save:
                ranges[op_id] = (len(flat), len(flat) + len(ctx.to_save))
                flat.extend(ctx.to_save)
                ctx.to_save = None
        self._saved_tensors, self._saved_ranges = flat, ranges
        return flat

    def restore_saved_tensors(self, saved_tensors: Sequence[Optional[torch.Tensor]]) -> None:
        for op_id, (lo, hi) in self._saved_ranges.items():
            self.op_contexts[op_id].saved_tensors = tuple(saved_tensors[lo:hi])

    def finalize_recomputed_contexts(self) -> None:
        """After a recompute pass: what ops registered becomes what backward reads."""
        for op_id in sorted(self.op_contexts):
            ctx = self.op_contexts[op_id]
            if ctx.to_save:
                ctx.saved_tensors = tuple(ctx.to_save)
                ctx.to_save = None

    def clear_saved_tensors_except(self, protected: set) -> None:
        """Free every saved/registered activation whose object id is not protected."""
        for ctx in self.op_contexts.values():
            for attr in ("saved_tensors", "to_save"):
                held = getattr(ctx, attr)
                if held is not None:
                    clear_tensor_data(*[t for t in held if t is not None and id(t) not in protected])
                    setattr(ctx, attr, None)
