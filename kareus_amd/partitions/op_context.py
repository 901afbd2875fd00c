"""Operator-side protocol objects: the per-op context and the operator base class.

The engine talks to every operator through two calls, ``fuser_forward`` and
``fuser_backward``, handing it an externally owned ``OperationContext``.  The
signatures and the context fields follow TransformerEngine's fusible-op protocol
as the reference uses it
(3rdparty/TransformerEngine/transformer_engine/pytorch/ops/op.py:28-57 for the
context, :71-161 and :458-503 for the two calls).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Iterable, List, Optional, Tuple

import torch


@dataclass
class OperationContext:
    """State one operator keeps between its forward and its backward.

    ``save_for_backward`` only *registers* tensors in ``to_save``; the engine moves
    them into ``saved_tensors`` (through autograd's saved-tensor list, or directly
    after a recompute).  Operators may hang any extra attribute on the instance.
    """

    saved_tensors: Optional[Tuple[Optional[torch.Tensor], ...]] = None
    to_save: Optional[Tuple[Optional[torch.Tensor], ...]] = None
    _saved_tensors_range: Optional[Tuple[int, int]] = None
    requires_grad: bool = True

    def save_for_backward(self, *tensors: Optional[torch.Tensor]) -> None:
        self.to_save = tensors


def clear_tensor_data(*tensors: Optional[torch.Tensor]) -> None:
    """Drop the storage behind each tensor object now instead of at refcount zero.

    Same role as TransformerEngine's helper of that name, which the reference calls
    after each backward op (backward_partition.py:107-115): saved activations are
    released op by op so a nanobatch's peak memory is one op's worth, not a layer's.
    Only the Python tensor object is rebound; other views of the storage keep it.
    """
    for t in tensors:
        if t is not None:
            t.data = torch.empty(0, device=t.device, dtype=t.dtype)


def operator_parameters(op: torch.nn.Module):
    """``op.parameters()`` in the same order.  An operator without submodules (most of a layer's) is answered
    from its own parameter table: the generic walk over the module tree costs the host several microseconds
    per operator, every step and nanobatch."""
    if op._modules:
        return list(op.parameters())
    return [p for p in op._parameters.values() if p is not None]


class BasicOperation(torch.nn.Module):
    """Base class of every compute operator.

    Subclasses implement ``op_forward(ctx, x, *, prev_op, next_op, **kw)`` and
    ``op_backward(ctx, dy)`` -> ``(dx, param_grads)``; ops with extra inputs or
    outputs override the ``fuser_*`` pair instead.
    """

    num_extra_inputs: int = 0
    num_extra_outputs: int = 0

    def op_forward(self, ctx: OperationContext, input_: torch.Tensor, **kwargs) -> torch.Tensor:
        raise NotImplementedError

    def op_backward(
        self, ctx: OperationContext, grad_output: torch.Tensor
    ) -> Tuple[torch.Tensor, Iterable[Optional[torch.Tensor]]]:
        raise NotImplementedError

    def fuser_forward(
        self,
        basic_op_ctxs: List[OperationContext],
        input_: torch.Tensor,
        *,
        basic_op_extra_inputs: List[Tuple[torch.Tensor, ...]],
        basic_op_prev_ops: List[Optional["BasicOperation"]],
        basic_op_next_ops: List[Optional["BasicOperation"]],
        basic_op_kwargs: List[Dict[str, Any]],
    ) -> Tuple[torch.Tensor, List[Tuple[torch.Tensor, ...]]]:
        if self.num_extra_inputs or self.num_extra_outputs:
            raise RuntimeError(
                f"{type(self).__name__} has extra inputs/outputs and must override fuser_forward"
            )
        out = self.op_forward(
            basic_op_ctxs[0],
            input_,
            prev_op=basic_op_prev_ops[0],
            next_op=basic_op_next_ops[0],
            **basic_op_kwargs[0],
        )
        return out, [()]

    def fuser_backward(
        self,
        basic_op_ctxs: List[OperationContext],
        grad_output: torch.Tensor,
        *,
        basic_op_grad_extra_outputs: List[Tuple[torch.Tensor, ...]],
    ) -> Tuple[torch.Tensor, List[Iterable[Optional[torch.Tensor]]], List[Tuple]]:
        if self.num_extra_inputs or self.num_extra_outputs:
            raise RuntimeError(
                f"{type(self).__name__} has extra inputs/outputs and must override fuser_backward"
            )
        dx, param_grads = self.op_backward(basic_op_ctxs[0], grad_output)
        return dx, [param_grads], [()]


def merge_sub_contexts(ctx: OperationContext, subs: List[OperationContext]) -> None:
    """Pool what several helper contexts want saved into their parent context and
    remember each helper's slice (reference: extensions/ops/utils.py:6-26)."""
    pooled: List[Optional[torch.Tensor]] = []
    for sub in subs:
        if sub.to_save is None:
            continue
        lo = len(pooled)
        pooled.extend(sub.to_save)
        sub._saved_tensors_range = (lo, len(pooled))
        sub.to_save = None
    if pooled:
        ctx.save_for_backward(*pooled)


def restore_sub_contexts(ctx: OperationContext, subs: List[OperationContext]) -> None:
    """Inverse of ``merge_sub_contexts`` (reference: extensions/ops/utils.py:29-44)."""
    if ctx.saved_tensors is None:
        return
    for sub in subs:
        if sub._saved_tensors_range is not None:
            lo, hi = sub._saved_tensors_range
            sub.saved_tensors = ctx.saved_tensors[lo:hi]
