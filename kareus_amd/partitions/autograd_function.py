"""The single autograd node around all layers, all partitions and all nanobatches.

Follows kareus/megatron/core/partitions/autograd_function.py: ``SeedConfig``
``:27-60``; forward seeds one context per nanobatch, runs the forward partitions
in issue order loading the scheduler's current item into each ``:149-177``, reads
the outputs from the ``main`` channel ``:180-184`` and either keeps only the inputs
(activation checkpointing ``:199-212``) or flattens every op's saved tensors into
autograd's list ``:213-221``; backward recomputes or restores ``:236-288``, seeds
the gradient stores ``:294-298``, runs the backward partitions collecting parameter
gradients per nanobatch ``:312-327`` and returns one gradient list per copy of the
parameters so autograd's accumulation sums the nanobatches ``:346-372``; gradient
count check ``:84-87``.

Differences from the reference, both required by the one-GPU target: the number of
nanobatches is not fixed at two (it is read off the argument list), and each
nanobatch may own a HIP stream, forked from and joined back to the caller's stream
here.  Dropout is not replayed during recompute because the layer runs with p = 0.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import torch
from torch import Tensor

from .context_manager import NanoBatchContext, TensorStore
from .streams import stream_api
from .tensor_graph import TensorGraph

# Non-tensor arguments that follow the nanobatch inputs, rotary table and mask.
_NUM_CONTROL_ARGS = 9


@dataclass(frozen=True)
class SeedConfig:
    """Tensor ids / channel names through which the block enters and leaves a graph."""

    h_tid: str = "ext_main"
    rotary_tid: Optional[str] = "ext_rotary_pos_emb"
    mask_tid: Optional[str] = None
    fwd_output_channel: str = "main"
    bwd_grad_tid: str = "ext_grad_main"
    bwd_output_channel: str = "grad_main"


def _flatten_grad_params(grad_params: Dict[int, List], num_params: int) -> List[Optional[Tensor]]:
    flat: List[Optional[Tensor]] = []
    for op_id in sorted(grad_params):
        flat.extend(grad_params[op_id])
    assert len(flat) == num_params, (
        f"Parameter gradient count mismatch: expected {num_params}, got {len(flat)}"
    )
    return flat


def _nanobatch_streams(config, n: int) -> List[Optional[object]]:
    streams = getattr(config, "nanobatch_streams", None)
    if not streams:
        return [None] * n
    if len(streams) != n:
        raise ValueError(f"config.nanobatch_streams has {len(streams)} streams for {n} nanobatches")
    return list(streams)


def _fork(streams: Sequence[Optional[object]]) -> None:
    """Side streams start after everything already enqueued on the caller's stream."""
    if any(s is not None for s in streams):
        here = stream_api().current_stream()
        for s in streams:
            if s is not None and s != here:
                s.wait_stream(here)


def _join(streams: Sequence[Optional[object]]) -> None:
    """The caller's stream continues after everything enqueued on the side streams."""
    if any(s is not None for s in streams):
        here = stream_api().current_stream()
        for s in streams:
            if s is not None and s != here:
                here.wait_stream(s)


def _batch_slices(like: Sequence[Tensor]) -> Optional[List[Tensor]]:
    """One new ``[s, b, h]`` tensor cut along the batch axis into views shaped like the given
    per-nanobatch tensors, or None when those are not ``[s, b_i, h]`` tensors of one kind."""
    first = like[0]
    if first.dim() != 3 or any(
        t.dim() != 3 or t.shape[0] != first.shape[0] or t.shape[2] != first.shape[2]
        or t.dtype != first.dtype or t.device != first.device for t in like
    ):
        return None
    widths = [t.shape[1] for t in like]
    whole = first.new_empty((first.shape[0], sum(widths), first.shape[2]))
    views, lo = [], 0
    for w in widths:
        views.append(whole[:, lo : lo + w])
        lo += w
    return views


def _last_compute_op(graph: TensorGraph, capability: str) -> Optional[int]:
    """op_id of the graph's final compute op if its operator can write into a given tensor."""
    ops = graph.get_compute_ops()
    if ops and getattr(ops[-1].operator, capability, False):
        return ops[-1].op_id
    return None


def _fused_producer_of_last(graph: TensorGraph) -> Optional[int]:
    """op_id of the projection in front of the graph's final residual add if it may add the
    residual in its own epilogue: it is then the op that writes the block's output."""
    ops = graph.get_compute_ops()
    if len(ops) >= 2 and getattr(ops[-2].operator, "fuse_residual", False):
        return ops[-2].op_id
    return None


def _seed_forward(ctxs, hs, rotary, mask, seed: SeedConfig) -> None:
    for ctx, h in zip(ctxs, hs):
        ctx.tensor_store.set(seed.h_tid, h)
        if rotary is not None and seed.rotary_tid is not None:
            ctx.tensor_store.set(seed.rotary_tid, rotary, False)
        if mask is not None and seed.mask_tid is not None:
            ctx.tensor_store.set(seed.mask_tid, mask, False)


def _run_forward(partitions, ctxs, schedule, is_grad_enabled: bool) -> None:
    n = len(ctxs)
    for part in partitions:
        part.is_grad_enabled = is_grad_enabled
        if schedule is not None:
            part.load_schedule(schedule)
        i = part.nano_batch_idx
        part.execute(ctx=ctxs[i], pre_ctx=ctxs[(i - 1) % n])


class TransformerBlockAutogradFunction(torch.autograd.Function):
    """``apply(h_1, ..., h_N, rotary_pos_emb, attention_mask, forward_partitions,
    backward_partitions, forward_tensor_graph, backward_tensor_graph, scheduler,
    config, seed_config, is_grad_enabled, checkpoint_activations,
    *params (N times over))`` -> ``(out_1, ..., out_N)``.

    N is found from the position of ``forward_partitions`` (the first list).
    """

    @staticmethod
    def forward(func_ctx, *args):
        first_list = next(i for i, a in enumerate(args) if isinstance(a, list))
        n = first_list - 2
        if n < 1:
            raise TypeError("expected at least one nanobatch input before rotary_pos_emb")
        hs = list(args[:n])
        rotary, mask = args[n], args[n + 1]
        (
            fwd_parts,
            bwd_parts,
            fwd_graph,
            bwd_graph,
            scheduler,
            config,
            seed,
            is_grad_enabled,
            checkpoint_activations,
        ) = args[n + 2 : n + 2 + _NUM_CONTROL_ARGS]
        params = args[n + 2 + _NUM_CONTROL_ARGS :]
        assert len(params) % n == 0, (
            f"Expected the parameter list repeated {n} times (one copy per nanobatch), "
            f"got {len(params)} tensors"
        )

        streams = _nanobatch_streams(config, n)
        ctxs = [NanoBatchContext(batch_idx=i, stream=streams[i]) for i in range(n)]
        _seed_forward(ctxs, hs, rotary, mask, seed)

        # The nanobatch outputs are written side by side into one [s, b, h] tensor, so the
        # caller can put them together without a copy; likewise the input gradients in backward.
        in_place = n > 1 and bool(getattr(config, "join_nanobatches_in_place", False))
        if in_place:
            last = _last_compute_op(fwd_graph, "forward_accepts_out_sink")
            sinks = _batch_slices(hs) if last is not None else None
            if sinks is not None:
                producer = _fused_producer_of_last(fwd_graph)
                for c, sink in zip(ctxs, sinks):
                    c.output_sinks[last] = sink
                    if producer is not None:
                        c.output_sinks[producer] = sink

        schedule = scheduler.current_schedule if scheduler is not None else None
        if checkpoint_activations:
            # the recomputation in backward has to draw the same dropout masks
            # (kareus/megatron/core/partitions/autograd_function.py:143-146)
            func_ctx.fwd_cpu_rng_state = torch.get_rng_state()
            func_ctx.fwd_cuda_rng_state = torch.cuda.get_rng_state() if torch.cuda.is_available() else None
        _fork(streams)
        _run_forward(fwd_parts, ctxs, schedule, is_grad_enabled)
        _join(streams)

        out_tid = fwd_graph.get_output_channel(seed.fwd_output_channel)
        outs = [c.tensor_store.get(out_tid) for c in ctxs]

        func_ctx.n = n
        func_ctx.streams = streams
        func_ctx.backward_partitions = bwd_parts
        func_ctx.backward_tensor_graph = bwd_graph
        func_ctx.scheduler = scheduler
        func_ctx.seed_config = seed
        func_ctx.num_params = len(params) // n
        func_ctx.rotary_pos_emb = rotary
        func_ctx.attention_mask = mask
        func_ctx.checkpoint_activations = checkpoint_activations
        func_ctx.fuse_wgrad_accumulation = bool(getattr(config, "fuse_wgrad_accumulation", False))
        func_ctx.wgrad_over_all_nanobatches = bool(getattr(config, "wgrad_over_all_nanobatches", True))
        func_ctx.wgrad_launches_at_end = getattr(config, "wgrad_launches_at_end", None)
        func_ctx.join_in_place = in_place

        if checkpoint_activations:
            func_ctx.forward_partitions = fwd_parts
            func_ctx.is_grad_enabled = is_grad_enabled
            func_ctx.save_for_backward(*hs)
            keep = {id(t) for t in (*hs, *outs, rotary, mask) if t is not None}
            for c in ctxs:
                c.tensor_store = TensorStore()
                c.clear_saved_tensors_except(keep)
        else:
            func_ctx.ctxs = ctxs
            flat: List[Optional[Tensor]] = []
            counts: List[int] = []
            for c in ctxs:
                saved = c.flatten_saved_tensors()
                counts.append(len(saved))
                flat.extend(saved)
                c.tensor_store = TensorStore()
            func_ctx.saved_counts = counts
            func_ctx.save_for_backward(*flat)

        return tuple(outs)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(func_ctx, *grad_outs):
        n: int = func_ctx.n
        seed: SeedConfig = func_ctx.seed_config
        streams = func_ctx.streams
        rotary, mask = func_ctx.rotary_pos_emb, func_ctx.attention_mask
        scheduler = func_ctx.scheduler
        schedule = scheduler.current_schedule if scheduler is not None else None

        _fork(streams)
        if func_ctx.checkpoint_activations:
            hs = func_ctx.saved_tensors
            ctxs = [NanoBatchContext(batch_idx=i, stream=streams[i]) for i in range(n)]
            _seed_forward(ctxs, hs, rotary, mask, seed)
            # with the generators as they were before the forward pass, and put back afterwards
            # (kareus/megatron/core/partitions/autograd_function.py:263-266)
            devices = [torch.cuda.current_device()] if func_ctx.fwd_cuda_rng_state is not None else []
            with torch.random.fork_rng(devices=devices, enabled=True):
                torch.set_rng_state(func_ctx.fwd_cpu_rng_state)
                if func_ctx.fwd_cuda_rng_state is not None:
                    torch.cuda.set_rng_state(func_ctx.fwd_cuda_rng_state)
                _run_forward(func_ctx.forward_partitions, ctxs, schedule, func_ctx.is_grad_enabled)
            for c in ctxs:
                c.finalize_recomputed_contexts()
        else:
            ctxs = func_ctx.ctxs
            saved = func_ctx.saved_tensors
            lo = 0
            for c, cnt in zip(ctxs, func_ctx.saved_counts):
                c.restore_saved_tensors(saved[lo : lo + cnt])
                lo += cnt

        for c, g in zip(ctxs, grad_outs):
            c.tensor_store = TensorStore()
            c.tensor_store.set(seed.bwd_grad_tid, g)

        pending = None
        if func_ctx.fuse_wgrad_accumulation and n > 1:
            # one sink per layer operator, shared by that operator's contexts of all nanobatches
            sinks: Dict[int, dict] = {}
            # ("turn": a counter all sinks share, by which launches that serve all nanobatches take the
            # nanobatch streams in rotation)
            turn = [0]
            at_end = func_ctx.wgrad_launches_at_end
            if at_end is None:
                at_end = n >= 4
            # ("pending": where such launches are left to be issued behind the last partition of the pass)
            pending = [] if (at_end and func_ctx.wgrad_over_all_nanobatches) else None
            for c in ctxs:
                for op_id, op_ctx in c.op_contexts.items():
                    op_ctx.wgrad_sink = sinks.setdefault(
                        op_id, {"n": n, "turn": turn, "defer": func_ctx.wgrad_over_all_nanobatches,
                                "pending": pending})
                    op_ctx.nanobatch_index = c.batch_idx

        if func_ctx.join_in_place:
            last = _last_compute_op(func_ctx.backward_tensor_graph, "backward_accepts_out_sink")
            sinks = _batch_slices(grad_outs) if last is not None else None
            if sinks is not None:
                for c, sink in zip(ctxs, sinks):
                    if last in c.op_contexts:
                        c.op_contexts[last].out_sink = sink

        protected = {id(t) for t in (rotary, mask) if t is not None}
        per_nb: List[Dict[int, List]] = [{} for _ in range(n)]
        for part in func_ctx.backward_partitions:
            if schedule is not None:
                part.load_schedule(schedule)
            i = part.nano_batch_idx
            got = part.execute(ctx=ctxs[i], pre_ctx=ctxs[(i - 1) % n], protected_tensor_ids=protected)
            per_nb[i].update(got)
        for launch in pending or ():
            launch()
        _join(streams)

        grad_tid = func_ctx.backward_tensor_graph.get_output_channel(seed.bwd_output_channel)
        dhs = [c.tensor_store.get(grad_tid) if grad_tid is not None else None for c in ctxs]

        grads: List[Optional[Tensor]] = []
        for i in range(n):
            grads.extend(_flatten_grad_params(per_nb[i], func_ctx.num_params))

        func_ctx.ctxs = None
        return (*dhs, None, None, *([None] * _NUM_CONTROL_ARGS), *grads)
