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
    def execute(
        self,
        ctx: NanoBatchContext,
        pre_ctx: NanoBatchContext,
        protected_tensor_ids: Optional[set] = None,
    ) -> Dict[int, List]:
        with self._on_stream(ctx), self._timed():
            return self._execute(ctx, pre_ctx, protected_tensor_ids or set())

    def _execute(self, ctx, pre_ctx, protected: set) -> Dict[int, List]:
        start, _end, sm_num, block_size = self._setup_comm()
        store = ctx.tensor_store
        comm_out, comm_extra = None, []
        launched = False
        grad_params: Dict[int, List] = {}

        for idx, op in enumerate(self.comp_ops):
            op_ctx = ctx.get_op_context(op.op_id)
            if not op_ctx.requires_grad:
                break

            in_ids = op.get_input_tensor_ids()
            dy = store.get(in_ids[0])
            grad_extra_out = [tuple(store.get(t) for t in in_ids[1:])] if len(in_ids) > 1 else []

            if start == idx:
                comm_out, comm_extra = self._launch_comm(pre_ctx, sm_num, block_size, backward=True)
                launched = True

            dx, op_param_grads, grad_extra_in = op.operator.fuser_backward(
                [op_ctx], dy, basic_op_grad_extra_outputs=grad_extra_out
            )

            grad_params[op.op_id] = [g for group in op_param_grads for g in group]
            if not self.profiling_mode:
                if op_ctx.saved_tensors is not None:
                    clear_tensor_data(
                        *[t for t in op_ctx.saved_tensors if t is not None and id(t) not in protected]
                    )
                op_ctx.saved_tensors = None

            self._op_done(idx)
            if idx == start - 1:
                self.comm_op.event_record(_current_stream())

            out_ids = op.get_output_tensor_ids()
            store.set(out_ids[0], dx)
            if grad_extra_in and grad_extra_in[0]:
                for k, tid in enumerate(out_ids[1:]):
                    g = grad_extra_in[0][k]
                    if g is not None:
                        store.set(tid, g)

        if self.comm_op is not None:
            if not launched:  # no slot given, or the op loop stopped before reaching it
                comm_out, comm_extra = self._launch_comm_no_overlap(
                    pre_ctx, sm_num, block_size, backward=True
                )
            self._sync_comm(pre_ctx, comm_out, comm_extra)
        return grad_params
