"""Forward execution of one partition.

Follows kareus/megatron/core/partitions/forward_partition.py:30-127: per op create
the context, gather inputs by port, decide ``requires_grad``, release the
hand-over when the scheduled op index is reached, run the op, record the release
event right after op ``start-1``, store outputs by port; afterwards run a
non-overlapped hand-over if ``start == -1`` and finally sync and publish its
result into the other nanobatch's store.
"""

from __future__ import annotations

from dataclasses import dataclass

from .context_manager import NanoBatchContext
from .partition_base import PartitionBase, _current_stream


@dataclass
class ForwardPartition(PartitionBase):
    def execute(self, ctx: NanoBatchContext, pre_ctx: NanoBatchContext) -> None:
        with self._on_stream(ctx), self._timed():
            self._execute(ctx, pre_ctx)

    def _execute(self, ctx: NanoBatchContext, pre_ctx: NanoBatchContext) -> None:
        start, _end, sm_num, block_size = self._setup_comm()
        store = ctx.tensor_store
        comm_out, comm_extra = None, []

        for idx, op in enumerate(self.comp_ops):
            op_ctx = ctx.create_op_context(op.op_id)
            in_ids = op.get_input_tensor_ids()
            x = store.get(in_ids[0])
            extras = [tuple(store.get(t) for t in in_ids[1:])] if len(in_ids) > 1 else []

            needs_grad = self.is_grad_enabled and (
                any(store.needs_grad(t) for t in in_ids)
                or any(p.requires_grad for p in op.operator.parameters())
            )
            op_ctx.requires_grad = needs_grad
            if ctx.output_sinks and op.op_id in ctx.output_sinks:
                op_ctx.out_sink = ctx.output_sinks.pop(op.op_id)

            if start == idx:
                comm_out, comm_extra = self._launch_comm(pre_ctx, sm_num, block_size)

            x, extra_out = op.operator.fuser_forward(
                [op_ctx],
                x,
                basic_op_extra_inputs=extras,
                basic_op_prev_ops=[None],
                basic_op_next_ops=[None],
                basic_op_kwargs=[{}],
            )

            self._op_done(idx)
            if idx == start - 1:
                self.comm_op.event_record(_current_stream())

            out_ids = op.get_output_tensor_ids()
            store.set(out_ids[0], x, needs_grad)
            for k, tid in enumerate(out_ids[1:]):
                extra = extra_out[0][k] if extra_out and extra_out[0] else None
                if extra is not None:
                    store.set(tid, extra, needs_grad)

        if self.comm_op is not None:
            if start == -1:
                comm_out, comm_extra = self._launch_comm_no_overlap(pre_ctx, sm_num, block_size)
            self._sync_comm(pre_ctx, comm_out, comm_extra)
