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
from .op_context import operator_parameters
from .partition_base import PartitionBase, _current_stream


@dataclass
class ForwardPartition(PartitionBase):
    # adjacent ops that offer a fused forward (fc1 + the SwiGLU activation behind it) run as one
    # call; the numbers are those of the separate calls
    fuse_forward_ops: bool = True

    def execute(self, ctx: NanoBatchContext, pre_ctx: NanoBatchContext) -> None:
        with self._on_stream(ctx), self._timed():
            self._execute(ctx, pre_ctx)

    def _fusable_follower(self, idx: int, start: int):
        """The op after ``idx`` when the two can run as one fused forward: the first op offers it
        (``can_fuse_forward_with``), the second is a plain one-in/one-out op consuming the
        first's only output, and the scheduled launch point does not fall between them."""
        if not self.fuse_forward_ops or idx + 1 >= len(self.comp_ops) or start == idx + 1:
            return None
        op, nxt = self.comp_ops[idx], self.comp_ops[idx + 1]
        offer = getattr(op.operator, "can_fuse_forward_with", None)
        if offer is None or not offer(nxt.operator):
            return None
        outs, nxt_ins = op.get_output_tensor_ids(), nxt.get_input_tensor_ids()
        if len(outs) != 1 or len(nxt_ins) != 1 or nxt_ins[0] != outs[0] or len(nxt.get_output_tensor_ids()) != 1:
            return None
        return nxt

    def _execute(self, ctx: NanoBatchContext, pre_ctx: NanoBatchContext) -> None:
        start, _end, sm_num, block_size = self._setup_comm()
        store = ctx.tensor_store
        comm_out, comm_extra = None, []

        idx, num_ops = 0, len(self.comp_ops)
        while idx < num_ops:
            op = self.comp_ops[idx]
            in_ids = op.get_input_tensor_ids()
            x = store.get(in_ids[0])
            extras = [tuple(store.get(t) for t in in_ids[1:])] if len(in_ids) > 1 else []
            follower = self._fusable_follower(idx, start)
            group = [op] if follower is None else [op, follower]

            needs_grad = self.is_grad_enabled and (
                any(store.needs_grad(t) for t in in_ids)
                or any(p.requires_grad for member in group for p in operator_parameters(member.operator))
            )
            group_ctxs = []
            for member in group:
                op_ctx = ctx.create_op_context(member.op_id)
                op_ctx.requires_grad = needs_grad
                if ctx.output_sinks and member.op_id in ctx.output_sinks:
                    op_ctx.out_sink = ctx.output_sinks.pop(member.op_id)
                group_ctxs.append(op_ctx)
            last = idx + len(group) - 1

            if start == idx:
                comm_out, comm_extra = self._launch_comm(pre_ctx, sm_num, block_size)

            k = len(group)
            x, extra_out = op.operator.fuser_forward(
                group_ctxs,
                x,
                basic_op_extra_inputs=extras if k == 1 else [extras[0] if extras else (), ()],
                basic_op_prev_ops=[None] * k,
                basic_op_next_ops=[None] * k,
                basic_op_kwargs=[{} for _ in range(k)],
            )

            for j in range(k):
                self._op_done(idx + j)
            if last == start - 1:
                self.comm_op.event_record(_current_stream())

            out_ids = group[-1].get_output_tensor_ids()
            store.set(out_ids[0], x, needs_grad)
            for j, tid in enumerate(out_ids[1:]):
                extra = extra_out[-1][j] if extra_out and extra_out[-1] else None
                if extra is not None:
                    store.set(tid, extra, needs_grad)
            idx = last + 1

        if self.comm_op is not None:
            if start == -1:
                comm_out, comm_extra = self._launch_comm_no_overlap(pre_ctx, sm_num, block_size)
            self._sync_comm(pre_ctx, comm_out, comm_extra)
