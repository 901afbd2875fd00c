"""Backward execution of one partition.

Follows kareus/megatron/core/partitions/backward_partition.py:36-145: ops come from
the backward graph (already reversed, channels ``grad_*``); each looks up the
context its forward twin filled (same ``op_id``), stops the partition early when
that context needs no gradient, returns parameter gradients keyed by ``op_id`` and
frees the saved activations of every op as soon as it has run (kept in
``profiling_mode`` so one forward can feed many timed backward runs; tensors whose
object id is in ``protected_tensor_ids`` are shared between nanobatches and kept).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

from .context_manager import NanoBatchContext
from .op_context import clear_tensor_data
from .partition_base import PartitionBase, _current_stream


@dataclass
class BackwardPartition(PartitionBase):
    # adjacent ops that offer a fused backward (RMSNorm + the residual fork in front of it) run
    # as one call; the numbers are those of the separate calls
    fuse_backward_ops: bool = True

    def execute(
        self,
        ctx: NanoBatchContext,
        pre_ctx: NanoBatchContext,
        protected_tensor_ids: Optional[set] = None,
    ) -> Dict[int, List]:
        with self._on_stream(ctx), self._timed():
            return self._execute(ctx, pre_ctx, protected_tensor_ids or set())

    def _fusable_follower(self, idx: int, start: int, ctx: NanoBatchContext):
        """The op after ``idx`` when the two can run as one fused backward: the first op offers it
        (``can_fuse_backward_with``), the second consumes the first's only output and needs a
        gradient, and the scheduled launch point does not fall between them."""
        if not self.fuse_backward_ops or idx + 1 >= len(self.comp_ops) or start == idx + 1:
            return None
        op, nxt = self.comp_ops[idx], self.comp_ops[idx + 1]
        offer = getattr(op.operator, "can_fuse_backward_with", None)
        if offer is None or not offer(nxt.operator):
            return None
        outs, nxt_ins = op.get_output_tensor_ids(), nxt.get_input_tensor_ids()
        if not outs or not nxt_ins or nxt_ins[0] != outs[0]:
            return None
        if not ctx.get_op_context(nxt.op_id).requires_grad:
            return None
        if any(t not in ctx.tensor_store for t in nxt_ins[1:]):
            return None
        return nxt

    def _execute(self, ctx, pre_ctx, protected: set) -> Dict[int, List]:
        start, _end, sm_num, block_size = self._setup_comm()
        store = ctx.tensor_store
        comm_out, comm_extra = None, []
        launched = False
        grad_params: Dict[int, List] = {}

        idx, num_ops = 0, len(self.comp_ops)
        while idx < num_ops:
            op = self.comp_ops[idx]
            op_ctx = ctx.get_op_context(op.op_id)
            if not op_ctx.requires_grad:
                break

            in_ids = op.get_input_tensor_ids()
            dy = store.get(in_ids[0])
            group, group_ctxs = [op], [op_ctx]
            grad_extra_out = [tuple(store.get(t) for t in in_ids[1:])] if len(in_ids) > 1 else []
            follower = self._fusable_follower(idx, start, ctx)
            if follower is not None:
                group.append(follower)
                group_ctxs.append(ctx.get_op_context(follower.op_id))
                grad_extra_out = [tuple(store.get(t) for t in in_ids[1:]),
                                  tuple(store.get(t) for t in follower.get_input_tensor_ids()[1:])]
            last = idx + len(group) - 1

            if start == idx:
                comm_out, comm_extra = self._launch_comm(pre_ctx, sm_num, block_size, backward=True)
                launched = True

            dx, op_param_grads, grad_extra_in = op.operator.fuser_backward(
                group_ctxs, dy, basic_op_grad_extra_outputs=grad_extra_out
            )

            for k, (member, member_ctx) in enumerate(zip(group, group_ctxs)):
                grad_params[member.op_id] = list(op_param_grads[k]) if len(group) > 1 else [
                    g for grads in op_param_grads for g in grads]
                if not self.profiling_mode:
                    if member_ctx.saved_tensors is not None:
                        clear_tensor_data(
                            *[t for t in member_ctx.saved_tensors if t is not None and id(t) not in protected]
                        )
                    member_ctx.saved_tensors = None
                self._op_done(idx + k)
            if last == start - 1:
                self.comm_op.event_record(_current_stream())

            store.set(group[-1].get_output_tensor_ids()[0], dx)
            # gradients of extra inputs: every member of a fused group may have some (a projection
            # that adds the residual in its epilogue hands the residual's gradient on)
            for k, member in enumerate(group):
                extras_k = grad_extra_in[k] if (grad_extra_in and len(grad_extra_in) == len(group)) else (
                    grad_extra_in[-1] if (grad_extra_in and k == len(group) - 1) else ())
                for j, tid in enumerate(member.get_output_tensor_ids()[1:]):
                    g = extras_k[j] if j < len(extras_k) else None
                    if g is not None:
                        store.set(tid, g)
            idx = last + 1

        if self.comm_op is not None:
            if not launched:  # no slot given, or the op loop stopped before reaching it
                comm_out, comm_extra = self._launch_comm_no_overlap(
                    pre_ctx, sm_num, block_size, backward=True
                )
            self._sync_comm(pre_ctx, comm_out, comm_extra)
        return grad_params
