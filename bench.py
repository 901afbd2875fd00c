#!/usr/bin/env python3
"""Layer fwd+bwd throughput of the partition-overlap engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c4|c2|c3|c5|c1gpu]

A step = one forward+backward of the decoder-layer stack over one synthetic batch, inputs
resident in HBM.  Prints ONE JSON line (metric: layer fwd+bwd tokens/s) that also carries
  roofline      the kernel with the largest share of the step's kernel time (the weight-gradient
                GEMM of fc1 at nanobatch shape, in the accumulating form most of its launches take),
                timed live with HIP events around its launches inside K steps of the nanobatched
                step's own launches issued on one stream (on concurrent streams an event interval
                also holds the wait for compute units; that interval is reported beside it),
                against the 2.5 PFLOP/s dense bf16 MFMA peak; `roofline_others` has the other two
                layouts of fc1
  cpu_baseline  the CPU oracle (plain PyTorch fp32 layer) timed on the host cores on a bounded
                sample of the same layer shape
  serial_1nb    the same layer and data run as one nanobatch on one stream, timed right after the
                headline steps with the same warm-up and step count
plus end-to-end MFMA utilisation, overlap efficiency (sum of serially timed partition times /
overlapped wall time), joules/token and the host's enqueue time per step.

`value` is the workload as configured: its own nanobatch count (four for c4) on concurrent
streams.  `--nanobatches N` runs another count; `--nanobatches auto` reports the faster of the
workload's count and a single nanobatch, picked from interleaved rounds (the reference, too,
falls back to sequential execution where nanobatching costs more than it gives:
tests/artifact/README.md:190-196), and `config.nanobatches` names the count that was run.

The chip is pre-heated for two seconds before anything is timed, and the ways of running the
layer that are compared (nanobatches on their own streams, one nanobatch, the same nanobatches on
one stream) are also timed in interleaved rounds (`overlap`), so that all of them see the same
power and thermal state.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import torch  # noqa: E402

MFMA_PEAK_BF16 = 2.5e15  # dense bf16, FLOP/s
HBM_PEAK = 8.0e12

# name -> (hidden, nq, nkv, hd, ffn, layers, batch, seq, nanobatches)
WORKLOADS = {
    "c1gpu": dict(h=512, nq=8, nkv=8, hd=64, ffn=1376, layers=1, b=2, s=256, nnb=2,
                  label="the CPU plumbing layer (h512, 8 heads of 64, ffn 1376) in bf16 on the device"),
    "c2": dict(h=3072, nq=3, nkv=1, hd=128, ffn=1024, layers=1, b=8, s=4096, nnb=2,
               label="Llama-3.2-3B layer, TP=8 shard, MBS 8 x seq 4096, 2 nanobatches"),
    "c3": dict(h=3072, nq=24, nkv=8, hd=128, ffn=8192, layers=1, b=4, s=4096, nnb=2,
               label="Llama-3.2-3B full-width layer, MBS 4 x seq 4096"),
    "c4": dict(h=4096, nq=8, nkv=2, hd=128, ffn=3584, layers=1, b=4, s=4096, nnb=4,
               label="Llama-3.1-8B layer, TP=4 shard, MBS 4 x seq 4096, 4 nanobatches"),
    "c5": dict(h=4096, nq=32, nkv=8, hd=128, ffn=14336, layers=4, b=2, s=8192, nnb=2,
               label="4-layer full-width Llama-3.1-8B stack, MBS 2 x seq 8192, 2 nanobatches"),
    # not one of the benchmark configurations: the reference's second training configuration as shipped
    # (tests/artifact/conf/megatron_qwen3_1.7b_config.yaml: q / k head norms, hidden dropout 0.1)
    "qwen3": dict(h=2048, nq=2, nkv=1, hd=128, ffn=768, layers=1, b=8, s=4096, nnb=2, qk_layernorm=True,
                  hidden_dropout=0.1,
                  label="Qwen3-1.7B layer, TP=8 shard, MBS 8 x seq 4096, 2 nanobatches, q/k head norms, hidden dropout 0.1"),
}


def total_flops(w) -> float:
    t = w["b"] * w["s"]
    gemm_fwd = 2 * t * (w["h"] * (w["nq"] + 2 * w["nkv"]) * w["hd"] + w["nq"] * w["hd"] * w["h"]
                        + w["h"] * 2 * w["ffn"] + w["ffn"] * w["h"])
    attn_fwd = 2 * w["b"] * w["nq"] * w["s"] ** 2 * w["hd"]
    return w["layers"] * (3 * gemm_fwd + 3.5 * attn_fwd)


def make_model(w, nnb, device, use_streams=True, schedule=None, all_on_one_stream=False):
    """``all_on_one_stream``: the engine is set up as for concurrent nanobatch streams (same launch plans,
    same event edges) but every nanobatch is given the caller's stream, so the very same launches run one
    after the other."""
    from kareus_amd import LayerConfig, LayerStack

    cfg = LayerConfig(hidden_size=w["h"], num_attention_heads=w["nq"], num_query_groups=w["nkv"],
                      kv_channels=w["hd"], ffn_hidden_size=w["ffn"], num_layers=w["layers"],
                      num_nanobatches=nnb, backend="hip", use_streams=use_streams,
                      **{k: w[k] for k in ("qk_layernorm", "hidden_dropout") if k in w})
    cfg.kareus_scheduler = schedule
    if all_on_one_stream and nnb > 1:
        cfg.nanobatch_streams = [torch.cuda.current_stream()] * nnb
    return LayerStack(cfg, device=device, seed=1234)


def make_scheduler(path, nnb):
    """The communication scheduler over a per-microbatch plan file (None without a file or with a
    single nanobatch, which has nothing to schedule)."""
    if not path or nnb < 2:
        return None
    from kareus_amd.scheduler import PipelineCommScheduler
    from kareus_amd.scheduler.parser import parse_schedule_file

    stages = parse_schedule_file(path, False, False)
    return PipelineCommScheduler(path, pp_rank=0, num_microbatches=len(stages[0]))


class Stepper:
    """Runs steps of one model; with a scheduler every step is one microbatch of the plan (forward
    and backward instruction), and the plan starts over when its microbatches are used up."""

    def __init__(self, model, x, go):
        self.model, self.x, self.go = model, x, go
        self.sch = model.config.kareus_scheduler
        self.left = 0

    def step(self):
        sch = self.sch
        if sch is not None:
            if self.left == 0:
                sch.on_step_begin()
                self.left = len(sch._schedule_items)
            sch.on_instruction_begin("forward")
        for p in self.model.parameters():
            p.grad = None
        self.x.grad = None
        y = self.model(self.x)
        if sch is not None:
            sch.on_instruction_end("forward")
            sch.on_instruction_begin("backward")
        y.backward(self.go)
        if sch is not None:
            sch.on_instruction_end("backward")
            self.left -= 1
            if self.left == 0:
                sch.on_step_end()

    def run(self, steps):
        for _ in range(steps):
            self.step()

    def timed(self, steps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        self.run(steps)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps


class EventTimer:
    """Records a HIP event pair around every partition (serial run, one stream)."""

    def __init__(self):
        self.spans = []

    def begin(self, part):
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        self._open = ev

    def end(self, part):
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        self.spans.append((type(part).__name__, part.partition_key or "trail", self._open, ev))

    def totals(self):
        out = {}
        for cls, key, a, b in self.spans:
            name = key if key else cls
            out[name] = out.get(name, 0.0) + a.elapsed_time(b)
        return out


def partition_times(stepper, iters=3):
    from kareus_amd.partitions.partition_base import PartitionBase

    stepper.run(1)
    torch.cuda.synchronize()
    timer = EventTimer()
    PartitionBase.timer = timer
    try:
        stepper.run(iters)
        torch.cuda.synchronize()
    finally:
        PartitionBase.timer = None
    return {k: v / iters for k, v in timer.totals().items()}


def partition_timeline(w, device, steps=24, wgrad_launches_at_end=None):
    """When each partition of each nanobatch starts and ends on the device inside one step in steady state:
    an event pair around every partition on its own stream (no profiler: the host runs at its own speed),
    times in microseconds from the start of the step's first partition.  ``step_us`` is the average over the
    run, ``partitions_end_us`` the end of the last partition: what follows are the weight gradients put off
    to the end of the backward pass."""
    from kareus_amd.partitions.partition_base import PartitionBase

    gen = torch.Generator().manual_seed(42)
    x = torch.randn(w["s"], w["b"], w["h"], generator=gen).to(device, torch.bfloat16).requires_grad_(True)
    go = torch.randn(w["s"], w["b"], w["h"], generator=gen).to(device, torch.bfloat16)
    model = make_model(w, w["nnb"], device)
    model.config.wgrad_launches_at_end = wgrad_launches_at_end
    st = Stepper(model, x, go)
    st.run(5)
    preheat(st, 2.0)

    class Marks:
        def __init__(self):
            self.rows, self.step, self.begun = [], -1, None

        def begin(self, part):
            self.begun = torch.cuda.Event(enable_timing=True)
            self.begun.record()

        def end(self, part):
            done = torch.cuda.Event(enable_timing=True)
            done.record()
            kind = "fwd" if "Forward" in type(part).__name__ else "bwd"
            self.rows.append((self.step, kind, part.partition_key or "trail", part.nano_batch_idx, self.begun, done))

    marks = Marks()
    PartitionBase.timer = marks
    try:
        first = torch.cuda.Event(enable_timing=True)
        first.record()
        for i in range(steps):
            marks.step = i
            st.step()
        last = torch.cuda.Event(enable_timing=True)
        last.record()
        torch.cuda.synchronize()
    finally:
        PartitionBase.timer = None
    shown = steps - 3
    rows = [(first.elapsed_time(b) * 1e3, first.elapsed_time(e) * 1e3, kind, key, nb)
            for (i, kind, key, nb, b, e) in marks.rows if i == shown]
    t0 = min(r[0] for r in rows)
    return {"workload_nanobatches": w["nnb"], "step_us": first.elapsed_time(last) * 1e3 / steps,
            "partitions_end_us": max(r[1] for r in rows) - t0,
            "partitions": [{"nanobatch": nb, "pass": kind, "partition": key, "start_us": round(a - t0, 1),
                            "end_us": round(b - t0, 1)} for a, b, kind, key, nb in sorted(rows)]}


# HBM-side bytes per launch from hardware counters (FETCH_SIZE and WRITE_SIZE of two profiler
# runs of `bench.py --roofline-only`, each scaled by what the same counter reads for
# `bench.py --copy-calibration`).  Keyed by (layout, M, N, K); a shape that was not profiled
# reports null.  A constant read off a profile, not something measured in this run: the entry
# names the profile it came from, and it is only reported while the GEMM source is the one the
# counters were read with (first 16 hex digits of its SHA-256).
TRAFFIC_GEMM_SOURCE = "1a6828d98a39b5eb"
MEASURED_TRAFFIC = {
    # (FETCH_SIZE KiB x 2.000 + WRITE_SIZE KiB x 1.000) x 1024, means over the launches of `bench.py --roofline-only`
    # one nanobatch of four (4096 tokens), what the default run launches; the weight gradient is one launch over
    # the operand pieces of all four nanobatches
    ("TN", 4096, 7168, 4096): {"bytes": (180551.6 * 2.000 + 90074.8) * 1024, "source": "profiles/gemm_fc1_c4.md"},
    ("NN", 4096, 4096, 7168): {"bytes": (172289.5 * 2.000 + 32769.4) * 1024, "source": "profiles/gemm_fc1_c4.md"},
    ("NT", 7168, 4096, 16384, "pieces"): {"bytes": (772842.6 * 2.000 + 57344.8) * 1024, "source": "profiles/gemm_fc1_c4.md"},
    # the whole microbatch as one nanobatch (16384 tokens, --nanobatches 1)
    ("NT", 7168, 4096, 16384): {"bytes": (839136.2 * 2.000 + 57344.9) * 1024, "source": "profiles/gemm_fc1_c4.md"},
    ("TN", 16384, 7168, 4096): {"bytes": (721271.9 * 2.000 + 344090.9) * 1024, "source": "profiles/gemm_fc1_c4.md"},
    ("NN", 16384, 4096, 7168): {"bytes": (688467.1 * 2.000 + 131076.5) * 1024, "source": "profiles/gemm_fc1_c4.md"},
}


def _gemm_source_is_the_profiled_one() -> bool:
    import hashlib

    path = os.path.join(ROOT, "kareus_amd", "csrc", "kr_gemm.hip")
    try:
        with open(path, "rb") as f:
            return hashlib.sha256(f.read()).hexdigest()[:16] == TRAFFIC_GEMM_SOURCE
    except OSError:
        return False


def _gemm_operands(layout, m, n, k, device):
    a = torch.randn((k, m) if layout == "NT" else (m, k), device=device).bfloat16()
    if layout == "TN":
        b = (torch.randn(n, k, device=device) * 0.02).bfloat16()
    elif layout == "NN":
        b = (torch.randn(k, n, device=device) * 0.02).bfloat16()
    else:
        b = torch.randn(k, n, device=device).bfloat16()
    return a, b


def time_gemm(be, layout, m, n, k, device, launches=30, fused_swiglu=False, residual=False, accumulate=False,
              fused_swiglu_backward=False, alone=False, preheat_s=0.0, pieces=1):
    """Average duration of one launch, HIP events on the stream the kernel is launched on.  ``preheat_s``:
    launch the same GEMM back to back for that long first, so that the timed launches see the clocks a
    sustained run settles at instead of a rested chip's.  ``pieces`` > 1 (layout NT): the operands are that
    many separate allocations of k / pieces rows each, contracted in one launch (the weight gradient over
    all nanobatches of a microbatch)."""
    a, b = _gemm_operands(layout, m, n, k, device)
    if pieces > 1:
        a_pieces = [t.clone() for t in a.chunk(pieces)]
        b_pieces = [t.clone() for t in b.chunk(pieces)]
    out = torch.empty(m, n, device=device, dtype=torch.bfloat16)
    y = torch.empty(m, n // 2, device=device, dtype=torch.bfloat16) if fused_swiglu else None
    r = torch.randn(m, n, device=device).bfloat16() if residual else None
    # fc1's saved output (gate | up): the epilogue turns the product into its gradient
    hx = torch.randn(m, 2 * n, device=device).bfloat16() if fused_swiglu_backward else None
    code = {"TN": 0, "NN": 1, "NT": 2}[layout]

    def fn():
        if pieces > 1:
            be.linear_wgrad_segments(a_pieces, b_pieces, out=out, accumulate=accumulate, split_k=True)
        elif hx is not None:
            be.gemm(code, a, b, m, n, k, split_k=None, swiglu_bwd_x=hx)
        else:
            be.gemm(code, a, b, m, n, k, out=out, accumulate=accumulate, split_k=alone, swiglu_out=y, residual=r)

    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    t_end = time.perf_counter() + preheat_s
    while time.perf_counter() < t_end:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(launches):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / launches


def _roofline_entry(kernel, layout, m, n, k, sec):
    flops = 2.0 * m * n * k
    achieved = flops / sec / 1e12
    key = (layout, m, n, k, "pieces") if "one launch over" in kernel else (layout, m, n, k)
    traffic = MEASURED_TRAFFIC.get(key) if _gemm_source_is_the_profiled_one() else None
    return {
        "bound": "mfma", "kernel": kernel, "shape": [m, n, k],
        "flops_per_launch": flops, "avg_launch_us": sec * 1e6,
        "achieved": achieved, "peak": MFMA_PEAK_BF16 / 1e12, "unit": "TFLOP/s",
        "frac": achieved * 1e12 / MFMA_PEAK_BF16,
        "traffic": traffic["bytes"] if traffic else None,
        "traffic_source": traffic["source"] if traffic else None,
    }


class GemmEventTimer:
    """HIP events around the GEMM launches of given (layout, M, N, K) while a step runs: the events
    are recorded on the stream the kernel is launched on (the current one), so on that stream an
    interval is the kernel's own duration.  Two event records per watched launch, nothing else."""

    def __init__(self, be, shapes):
        self.be, self.shapes = be, set(shapes)
        self.pairs = {}     # (shape, accumulating) -> [(start event, end event)]

    def __enter__(self):
        inner = self.be.gemm

        def gemm(layout, a, b, m, n, k, *args, **kw):
            key = (layout, m, n, k)
            if key not in self.shapes:
                return inner(layout, a, b, m, n, k, *args, **kw)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            r = inner(layout, a, b, m, n, k, *args, **kw)
            e1.record()
            self.pairs.setdefault((key, bool(kw.get("accumulate"))), []).append((e0, e1))
            return r

        inner_segments = self.be.linear_wgrad_segments

        def segments(dys, xs, *args, **kw):
            key = (2, dys[0].shape[-1], xs[0].shape[-1], sum(d.shape[0] for d in dys))
            if key not in self.shapes:
                return inner_segments(dys, xs, *args, **kw)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            r = inner_segments(dys, xs, *args, **kw)
            e1.record()
            self.pairs.setdefault((key, bool(kw.get("accumulate"))), []).append((e0, e1))
            return r

        self.be.gemm = gemm
        self.be.linear_wgrad_segments = segments
        return self

    def __exit__(self, *exc):
        del self.be.gemm    # back to the class's methods
        del self.be.linear_wgrad_segments
        return False

    def seconds(self, key, accumulating=None):
        """(average duration of a launch, launches) of the launches of a shape — all of them, or only those
        that do / do not accumulate into their output; call after the device has been synchronised."""
        pairs = [p for (k, acc), v in self.pairs.items() if k == key and accumulating in (None, acc) for p in v]
        if not pairs:
            return None, 0
        return sum(a.elapsed_time(b) for a, b in pairs) * 1e-3 / len(pairs), len(pairs)


def dominant_gemm_shapes(w, nnb):
    """(layout code, M, N, K) of fc1's forward (TN) and input gradient (NN) at the token count of one
    nanobatch and of its weight gradient (NT), which the engine computes once per step over the tokens of
    all nanobatches."""
    t, two_f, h = (w["b"] // nnb) * w["s"], 2 * w["ffn"], w["h"]
    return {"NT": (2, two_f, h, t * nnb), "TN": (0, t, two_f, h), "NN": (1, t, h, two_f)}


def dominant_kernel_roofline(w, nnb, device, launches=30, preheat_s=0.0):
    """The three GEMMs of fc1, which hold the largest share of the step's kernel time, each launched back
    to back on its own: the forward (TN, with the SwiGLU epilogue the engine runs it with), the input
    gradient (NN) and the weight gradient dW[2F, h] = dy[T, 2F]^T . x[T, h] (NT; with several nanobatches one
    launch over the operand pieces of all of them).  Returned with the one that takes the most time per step
    first: with several nanobatches the forward (one launch per nanobatch; the weight gradient is a single
    launch), with one nanobatch the weight gradient."""
    from kareus_amd.backend import get_backend

    be = get_backend("hip")
    t, two_f, h = (w["b"] // nnb) * w["s"], 2 * w["ffn"], w["h"]
    fuse = be.can_fuse_swiglu(two_f)
    first = {"TN": preheat_s, "NT": preheat_s / 2} if nnb > 1 else {"NT": preheat_s, "TN": preheat_s / 2}
    nt = _roofline_entry("gemm_kernel<NT> (fc1 weight gradient%s)" % (f", one launch over {nnb} nanobatches" if nnb > 1 else ""),
                         "NT", two_f, h, t * nnb,
                         time_gemm(be, "NT", two_f, h, t * nnb, device, launches, alone=True, preheat_s=first["NT"], pieces=nnb))
    tn = _roofline_entry("gemm_kernel<TN%s> (fc1 forward)" % (", SwiGLU epilogue" if fuse else ""), "TN", t, two_f, h,
                         time_gemm(be, "TN", t, two_f, h, device, launches, fused_swiglu=fuse, preheat_s=first["TN"]))
    nn = _roofline_entry("gemm_kernel<NN> (fc1 input gradient)", "NN", t, h, two_f,
                         time_gemm(be, "NN", t, h, two_f, device, launches, preheat_s=preheat_s / 2))
    return (tn, [nn, nt]) if nnb > 1 else (nt, [tn, nn])


def time_library_matmul(layout, m, n, k, device, launches=30):
    """The same product through ``torch.matmul`` (the vendor's GEMM library), same operands and
    layout, plain store: a yardstick for the kernel, not part of the step."""
    a, b = _gemm_operands(layout, m, n, k, device)
    out = torch.empty(m, n, device=device, dtype=torch.bfloat16)
    lhs = a.t() if layout == "NT" else a
    rhs = b.t() if layout == "TN" else b

    def fn():
        torch.matmul(lhs, rhs, out=out)

    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(launches):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / launches


def gemm_kernels(w, nnb, device, launches=30, with_library=False):
    """Every GEMM of the layer alone on the GPU at the nanobatch shape, the way the engine launches
    it (forward of fc1 with the SwiGLU epilogue, of the out-projection and fc2 with the residual
    epilogue, fc2's input gradient with the SwiGLU-backward epilogue, weight gradients also
    accumulating into an existing buffer; planned for the launch's own latency with one nanobatch,
    for compute-unit time beside the other streams of several): TFLOP/s against the peak."""
    from kareus_amd.backend import get_backend

    be = get_backend("hip")
    t, h, f = (w["b"] // nnb) * w["s"], w["h"], w["ffn"]
    qkv, proj_in = (w["nq"] + 2 * w["nkv"]) * w["hd"], w["nq"] * w["hd"]
    layers = [("qkv", h, qkv), ("proj", proj_in, h), ("fc1", h, 2 * f), ("fc2", f, h)]
    rows = []
    for name, k_in, n_out in layers:
        variants = [
            ("forward", "TN", t, n_out, k_in, dict(fused_swiglu=name == "fc1" and be.can_fuse_swiglu(n_out),
                                                    residual=name in ("proj", "fc2"))),
            ("input gradient", "NN", t, k_in, n_out, dict(fused_swiglu_backward=True) if name == "fc2" else {}),
            ("weight gradient", "NT", n_out, k_in, t, {}),
            ("weight gradient, accumulating", "NT", n_out, k_in, t, dict(accumulate=True)),
        ]
        if nnb > 1:
            variants.append((f"weight gradient, one launch over {nnb} nanobatches", "NT", n_out, k_in, t * nnb,
                             dict(pieces=nnb)))
        for what, layout, m, n, k, kw in variants:
            sec = time_gemm(be, layout, m, n, k, device, launches, alone=nnb == 1, **kw)
            flops = 2.0 * m * n * k
            rows.append({"gemm": f"{name} {what}", "layout": layout, "shape": [m, n, k], "epilogue": kw,
                         "avg_launch_us": sec * 1e6, "TFLOPs": flops / sec / 1e12,
                         "frac_of_peak": flops / sec / MFMA_PEAK_BF16})
            if with_library and not kw.get("accumulate"):
                rows[-1]["library_matmul_us"] = time_library_matmul(layout, m, n, k, device, launches) * 1e6
    return rows


def power_trace(w, device, seconds=2.0):
    """Board power and shader clock (hwmon, 100 Hz) while the GPU idles, runs one GEMM back to back,
    runs the attention kernels, an HBM-bound kernel, and the layer step with the workload's
    nanobatch count and with one nanobatch: what the step's time and energy are made of."""
    from kareus_amd.backend import get_backend
    from kareus_amd.energy import ClockReader, PowerSampler

    be = get_backend("hip")
    sampler, clock = PowerSampler(0, hz=100.0), ClockReader(0)
    t_nb, two_f, h = (w["b"] // w["nnb"]) * w["s"], 2 * w["ffn"], w["h"]
    a, b = _gemm_operands("TN", t_nb, two_f, h, device)
    out = torch.empty(t_nb, two_f, device=device, dtype=torch.bfloat16)
    q = torch.randn(w["s"], w["b"], w["nq"], w["hd"], device=device, dtype=torch.bfloat16)
    k = torch.randn(w["s"], w["b"], w["nkv"], w["hd"], device=device, dtype=torch.bfloat16)
    v = torch.randn_like(k)
    xa = torch.randn(w["b"] * w["s"], h, device=device, dtype=torch.bfloat16)
    xb = torch.randn_like(xa)
    gen = torch.Generator().manual_seed(42)
    x = torch.randn(w["s"], w["b"], h, generator=gen).to(device, torch.bfloat16).requires_grad_(True)
    go = torch.randn(w["s"], w["b"], h, generator=gen).to(device, torch.bfloat16)
    steppers = {n: Stepper(make_model(w, n, device), x, go) for n in sorted({w["nnb"], 1})}
    phases = [
        ("idle", None, 0.0),
        ("gemm fc1 forward, back to back", lambda: be.gemm(0, a, b, t_nb, two_f, h, out=out, split_k=False),
         2.0 * t_nb * two_f * h),
        ("attention forward, whole microbatch", lambda: be.attn_fwd(q, k, v, w["hd"] ** -0.5),
         2.0 * w["b"] * w["nq"] * w["s"] ** 2 * w["hd"]),
        ("residual add (HBM-bound)", lambda: be.add(xa, xb), 0.0),
    ] + [(f"layer step, {n} nanobatch(es)", steppers[n].step, total_flops(w)) for n in steppers]
    rows = []
    for name, fn, flops in phases:
        calls = 0
        if fn is not None:
            for _ in range(3):
                fn()
        torch.cuda.synchronize()
        sampler.start()
        clock.start()
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            if fn is None:
                time.sleep(0.05)
            else:
                for _ in range(8):
                    fn()
                calls += 8
                torch.cuda.synchronize()
        t1 = time.perf_counter()
        sampler.stop()
        clock.stop()
        joules = sampler.energy_joules(t0, t1) if sampler.available else None
        mhz = clock.values(t0 + 0.5, t1)
        rows.append({
            "phase": name, "seconds": t1 - t0, "calls": calls,
            "ms_per_call": (t1 - t0) / calls * 1e3 if calls else None,
            "mean_watts": joules / (t1 - t0) if joules else None,
            "joules_per_call": joules / calls if joules and calls else None,
            "sclk_mhz_mean": sum(mhz) / len(mhz) if mhz else None,
            "sclk_mhz_min": min(mhz) if mhz else None, "sclk_mhz_max": max(mhz) if mhz else None,
            "TFLOPs": flops * calls / (t1 - t0) / 1e12 if flops and calls else None,
        })
    return {"bus_id": sampler.bus_id, "rows": rows}


def copy_calibration(device, n=1 << 29, launches=10):
    """kr_add over n bf16 elements: reads 2*n*2 bytes, writes n*2 bytes per launch — the known-size
    kernel against which the FETCH_SIZE / WRITE_SIZE counters are scaled."""
    from kareus_amd.backend import get_backend

    be = get_backend("hip")
    a = torch.ones(n, device=device, dtype=torch.bfloat16)
    b = torch.ones(n, device=device, dtype=torch.bfloat16)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(launches):
        be.add(a, b)
    e1.record()
    torch.cuda.synchronize()
    sec = e0.elapsed_time(e1) * 1e-3 / launches
    return {"kernel": "add_kernel", "elements": n, "read_bytes": 4 * n, "write_bytes": 2 * n,
            "avg_launch_us": sec * 1e6, "achieved_GBps": 6 * n / sec / 1e9}


def hbm_kernels(w, nnb, device, launches=50):
    """Every HBM-bound kernel of the layer alone on the GPU, at the nanobatch shape and at the
    whole-microbatch shape: average launch time (HIP events on the launch stream) and
    algorithmic bytes (operands read once, results written once) per second against 8 TB/s."""
    from kareus_amd.backend import get_backend
    from kareus_amd.operators.rotary_embedding import rotary_frequencies

    be = get_backend("hip")
    bf = torch.bfloat16
    rows_out = []

    def timed(fn):
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(launches):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / launches

    def report(name, tokens, nbytes, fn):
        sec = timed(fn)
        rows_out.append({"kernel": name, "tokens": tokens, "bytes": nbytes, "avg_launch_us": sec * 1e6,
                         "achieved_TBps": nbytes / sec / 1e12, "frac_of_8TBps": nbytes / sec / HBM_PEAK})

    h, f, hd = w["h"], w["ffn"], w["hd"]
    heads = w["nq"] + w["nkv"]
    for t in sorted({(w["b"] // nnb) * w["s"], w["b"] * w["s"]}):
        x = torch.randn(t, h, device=device, dtype=bf)
        y = torch.randn(t, h, device=device, dtype=bf)
        gamma = torch.ones(h, device=device, dtype=bf)
        report("add_kernel (residual add)", t, 3 * t * h * 2, lambda: be.add(x, y))
        report("rmsnorm_fwd_kernel", t, 2 * t * h * 2, lambda: be.rmsnorm_fwd(x, gamma, 1e-5))
        normed, rstd = be.rmsnorm_fwd(x, gamma, 1e-5)
        report("rmsnorm_bwd_kernel + rmsnorm_dgamma_kernel", t, 3 * t * h * 2,
               lambda: be.rmsnorm_bwd(y, x, rstd, gamma))
        report("rmsnorm_bwd_kernel<ADD> (+ residual gradient) + dgamma", t, 4 * t * h * 2,
               lambda: be.rmsnorm_bwd(y, x, rstd, gamma, residual_grad=normed))
        u = torch.randn(t, 2 * f, device=device, dtype=bf)
        dy = torch.randn(t, f, device=device, dtype=bf)
        report("swiglu_fwd_kernel", t, 3 * t * f * 2, lambda: be.swiglu_fwd(u))
        report("swiglu_bwd_kernel", t, 5 * t * f * 2, lambda: be.swiglu_bwd(dy, u))
        s_len = w["s"]
        qk = torch.randn(s_len, t // s_len, heads, hd, device=device, dtype=bf)
        freqs = rotary_frequencies(s_len, hd, 500000.0, device=device)
        report("rope_kernel (q and k heads)", t, 2 * t * heads * hd * 2, lambda: be.rope_fwd(qk, freqs))
        # hidden dropout (not part of the benchmark workloads, p = 0 there): two bf16 operands read, the
        # sum and a byte mask written; backward one bf16 operand and the mask read, one result written
        _, mask = be.dropout_add(x, y, 0.1)
        report("dropout_add_kernel (p = 0.1)", t, t * h * (3 * 2 + 1), lambda: be.dropout_add(x, y, 0.1))
        report("dropout_bwd_kernel", t, t * h * (2 * 2 + 1), lambda: be.dropout_bwd(y, mask, 1 / 0.9))
        # q / k layernorm of the QKV split (Qwen3-style layers; not part of the benchmark workloads): the
        # fused buffer read and written once forward; backward the gradient and the saved input of the
        # query and key heads read, their gradient rewritten in place
        per = w["nq"] // w["nkv"]
        if hd in (64, 128, 256):
            fused = torch.randn(s_len, t // s_len, w["nkv"], per + 2, hd, device=device, dtype=bf)
            dfused = torch.randn_like(fused)
            gq, gk = torch.ones(hd, device=device, dtype=bf), torch.ones(hd, device=device, dtype=bf)
            _, rs = be.qk_norm_fwd(fused, gq, gk, 1e-5)
            report("qk_norm_fwd_kernel", t, 2 * fused.numel() * 2 + rs.numel() * 4,
                   lambda: be.qk_norm_fwd(fused, gq, gk, 1e-5))
            report("qk_norm_bwd_kernel + qk_norm_dgamma_kernel", t, 3 * t * heads * hd * 2 + rs.numel() * 4,
                   lambda: be.qk_norm_bwd(dfused, fused, rs, gq, gk))
    return rows_out


def attention_kernels(w, nnb, device, launches=20):
    """Causal attention forward and backward alone on the GPU, at the nanobatch batch and at the
    whole-microbatch batch: average time of one forward / one backward call (HIP events on the
    launch stream) and causal FLOPs (2*b*nq*s^2*hd forward, 2.5x backward) per second."""
    from kareus_amd.backend import get_backend

    be = get_backend("hip")
    bf = torch.bfloat16
    s_len, nq, nkv, hd = w["s"], w["nq"], w["nkv"], w["hd"]
    scale = hd ** -0.5
    out = []

    def timed(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(launches):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / launches

    for b in sorted({w["b"] // nnb, w["b"]}):
        q = torch.randn(s_len, b, nq, hd, device=device, dtype=bf)
        k = torch.randn(s_len, b, nkv, hd, device=device, dtype=bf)
        v = torch.randn(s_len, b, nkv, hd, device=device, dtype=bf)
        o, lse = be.attn_fwd(q, k, v, scale)
        do = torch.randn_like(o)
        flops = 2.0 * b * nq * s_len * s_len * hd
        t_f = timed(lambda: be.attn_fwd(q, k, v, scale))
        t_b = timed(lambda: be.attn_bwd(do, q, k, v, o, lse, scale))
        out.append({"batch": b, "seq": s_len, "q_heads": nq, "kv_heads": nkv, "head_dim": hd,
                    "fwd_us": t_f * 1e6, "fwd_TFLOPs": flops / t_f / 1e12,
                    "fwd_frac_of_peak": flops / t_f / MFMA_PEAK_BF16,
                    "bwd_us": t_b * 1e6, "bwd_TFLOPs": 2.5 * flops / t_b / 1e12,
                    "bwd_frac_of_peak": 2.5 * flops / t_b / MFMA_PEAK_BF16})
    return out


def attention_padded_shapes(device):
    """Attention shapes outside the MFMA kernels (a head dimension below 128, a sequence that is not whole
    128-row tiles), forward and backward alone on the GPU both ways: padded into the MFMA kernels through the
    workspace (what the engine runs) and on the general fp32 kernels.  Causal FLOPs as in attention_kernels."""
    from kareus_amd.backend import get_backend

    be = get_backend("hip")
    out = []

    def timed(fn, launches):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(launches):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / launches

    for s_len, b, nq, nkv, hd in [(1000, 4, 8, 2, 128), (4000, 4, 8, 2, 128), (4096, 2, 32, 8, 64), (2048, 4, 16, 16, 64)]:
        per = nq // nkv
        fused = torch.randn(s_len, b, nkv, per + 2, hd, device=device).bfloat16()   # the fused QKV layout
        q, k, v = fused[:, :, :, :per], fused[:, :, :, per], fused[:, :, :, per + 1]
        do = torch.randn(s_len, b, nq, hd, device=device).bfloat16()
        scale, flops = hd ** -0.5, 2.0 * b * nq * s_len * s_len * hd
        row = {"seq": s_len, "batch": b, "q_heads": nq, "kv_heads": nkv, "head_dim": hd}
        for name, general in (("padded_into_mfma", False), ("general_kernels", True)):
            o, lse = be.attn_fwd(q, k, v, scale, general_kernels=general)
            n = 3 if general else 10
            t_f = timed(lambda: be.attn_fwd(q, k, v, scale, general_kernels=general), n)
            t_b = timed(lambda: be.attn_bwd(do, q, k, v, o, lse, scale, general_kernels=general), n)
            row[name] = {"fwd_us": t_f * 1e6, "bwd_us": t_b * 1e6, "fwd_TFLOPs": flops / t_f / 1e12,
                         "bwd_TFLOPs": 2.5 * flops / t_b / 1e12}
        out.append(row)
    return out


def cpu_baseline(w, budget_s=25.0):
    """The CPU oracle (fp32 PyTorch, autograd backward) on a bounded sample: same layer widths,
    one sequence of at most 1024 tokens, as many iterations as fit the time budget."""
    from oracle import llama_layer_ref as ref

    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    s = min(w["s"], 1024)
    dims = ref.LayerDims(w["h"], w["nq"], w["nkv"], w["hd"], w["ffn"])
    gen = torch.Generator().manual_seed(1234)
    params = [ref.init_layer_params(dims, gen)]
    if w.get("qk_layernorm"):
        params[0].update(q_norm=torch.ones(w["hd"]), k_norm=torch.ones(w["hd"]))
    x = torch.randn(s, 1, w["h"], generator=gen)
    go = torch.randn(s, 1, w["h"], generator=gen)
    freqs = ref.rope_table(s, w["hd"], dims.rope_base)
    ref.stack_forward_backward(x, params, dims, go, freqs)  # warm-up
    times = []
    t_start = time.perf_counter()
    while len(times) < 5 and (time.perf_counter() - t_start) < budget_s:
        t0 = time.perf_counter()
        ref.stack_forward_backward(x, params, dims, go, freqs)
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    return {
        "value": s / med, "unit": "tokens/s", "cores": cores, "kind": "port",
        "sample": f"one layer of the same widths, fp32, b=1 x s={s}, median of {len(times)} fwd+bwd",
    }


class _FixedSchedule:
    """A scheduler stand-in that hands every partition the same window and resource shape."""

    def __init__(self, window, reserved_cus):
        from kareus_amd.scheduler import CommConfig, ScheduleItem

        cc = CommConfig(window, (reserved_cus, 1024))
        self.current_schedule = ScheduleItem(cc, cc, cc, cc)
        self._schedule_items = [self.current_schedule]

    def on_step_begin(self): pass
    def on_step_end(self): pass
    def on_instruction_begin(self, name): pass
    def on_instruction_end(self, name=None): pass


def cu_budget_sweep(w, device, budgets=(0, 8, 16, 32, 64), rounds=4, steps=6):
    """The nanobatched layer step under schedules that reserve 0..64 compute units for the other
    nanobatch streams (every partition's GEMMs launch on the rest), for the earliest release point
    and for release after the partition; interleaved rounds after a pre-heat, median ms per step."""
    gen = torch.Generator().manual_seed(42)
    x = torch.randn(w["s"], w["b"], w["h"], generator=gen).to(device, torch.bfloat16).requires_grad_(True)
    go = torch.randn(w["s"], w["b"], w["h"], generator=gen).to(device, torch.bfloat16)
    ways = {}
    for window in (("norm_0", "none"), ("none", "none")):
        for cus in budgets:
            model = make_model(w, w["nnb"], device, schedule=_FixedSchedule(window, cus))
            ways[f"release {window[0]}, {cus} units reserved"] = Stepper(model, x, go)
    ways["no schedule"] = Stepper(make_model(w, w["nnb"], device), x, go)
    ways["one nanobatch"] = Stepper(make_model(w, 1, device, use_streams=False), x, go)
    for st in ways.values():
        st.run(2)
    preheat(ways["no schedule"], 2.0)
    med, _ = interleaved_rounds(ways, steps, rounds)
    return {name: t * 1e3 for name, t in med.items()}


class _SuppressedLaunches:
    """Timing only: the library entry points named here return success without launching (their outputs
    keep whatever the buffers held), so a step runs as if those kernels cost nothing."""

    def __init__(self, lib, names):
        self.lib, self.names, self.saved = lib, names, {}

    def __enter__(self):
        for n in self.names:
            self.saved[n] = getattr(self.lib, n)
            setattr(self.lib, n, lambda *a, **k: 0)
        return self

    def __exit__(self, *exc):
        for n, fn in self.saved.items():
            setattr(self.lib, n, fn)


def overlap_bound(w, device, rounds=4, steps=8):
    """What overlap between nanobatches could win on one GPU at best, and whether the host limits it.

    (1) The nanobatched step with its HBM-bound launches (RMSNorm forward / backward, rotary embedding,
        the norm weight-gradient reduction) suppressed: the time it would take if every one of them hid
        completely behind the other nanobatches' MFMA-bound kernels.  Timing only — results are wrong.
    (2) The same for the one-nanobatch step (its floor without those kernels).
    (6) Both steps with only the rotary embedding's launches suppressed: the most that folding the rotation
        into the neighbouring kernels (qkv GEMM epilogue, attention backward stores) could win.
    (3) The nanobatched step with a busy wait added to the host's work per step: GPU time against host time.
    (5) The nanobatched step with the weight gradients as one launch per layer where the last nanobatch
        delivers its operands (instead of at the end of the backward pass), and as one accumulating launch per
        nanobatch (the reference's way).
    (4) The nanobatched step with the attention kernels in the forms they take when a launch has the device
        to itself (keys split between the halves of a workgroup at one sequence) instead of the forms the engine
        picks beside other streams (no split: fewer workgroups, less compute-unit time).
    All interleaved after a pre-heat, median ms per step."""
    from kareus_amd.backend import get_backend

    gen = torch.Generator().manual_seed(42)
    x = torch.randn(w["s"], w["b"], w["h"], generator=gen).to(device, torch.bfloat16).requires_grad_(True)
    go = torch.randn(w["s"], w["b"], w["h"], generator=gen).to(device, torch.bfloat16)
    nano = Stepper(make_model(w, w["nnb"], device), x, go)
    serial = Stepper(make_model(w, 1, device, use_streams=False), x, go)
    unsplit = Stepper(make_model(w, w["nnb"], device), x, go)
    for layer in unsplit.model.layers:
        layer.core_attention.beside_other_streams = False
    in_place = Stepper(make_model(w, w["nnb"], device), x, go)     # weight-gradient launches where the last nanobatch delivers
    in_place.model.config.wgrad_launches_at_end = False
    per_nb = Stepper(make_model(w, w["nnb"], device), x, go)       # one accumulating weight gradient per nanobatch
    per_nb.model.config.wgrad_over_all_nanobatches = False
    for st in (nano, serial, unsplit, in_place, per_nb):
        st.run(2)
    preheat(nano, 2.0)
    lib = get_backend("hip").lib
    hbm = ["kr_rmsnorm_fwd", "kr_rmsnorm_bwd", "kr_rmsnorm_bwd_add", "kr_rmsnorm_dgamma", "kr_rope"]
    samples = {k: [] for k in ("nanobatched", "one nanobatch", "nanobatched, HBM-bound launches suppressed",
                               "one nanobatch, HBM-bound launches suppressed",
                               "nanobatched, rotary embedding launches suppressed",
                               "one nanobatch, rotary embedding launches suppressed",
                               "nanobatched, attention kernels in the forms they take alone on the device",
                               "nanobatched, weight gradients launched where the last nanobatch delivers its operands",
                               "nanobatched, one accumulating weight gradient per nanobatch")}
    for _ in range(rounds):
        samples["nanobatched"].append(nano.timed(steps))
        samples["nanobatched, weight gradients launched where the last nanobatch delivers its operands"].append(in_place.timed(steps))
        samples["nanobatched, one accumulating weight gradient per nanobatch"].append(per_nb.timed(steps))
        samples["nanobatched, attention kernels in the forms they take alone on the device"].append(unsplit.timed(steps))
        samples["one nanobatch"].append(serial.timed(steps))
        with _SuppressedLaunches(lib, hbm):
            samples["nanobatched, HBM-bound launches suppressed"].append(nano.timed(steps))
            samples["one nanobatch, HBM-bound launches suppressed"].append(serial.timed(steps))
        with _SuppressedLaunches(lib, ["kr_rope"]):
            samples["nanobatched, rotary embedding launches suppressed"].append(nano.timed(steps))
            samples["one nanobatch, rotary embedding launches suppressed"].append(serial.timed(steps))
    out = {"ms_per_step": {k: sorted(v)[len(v) // 2] * 1e3 for k, v in samples.items()}}

    def spin(us):
        end = time.perf_counter() + us * 1e-6
        while time.perf_counter() < end:
            pass

    plain_step = nano.step
    delays = {}
    for extra_us in (0, 300, 600, 1000, 1500):
        def step():
            spin(extra_us)
            plain_step()
        nano.step = step
        nano.run(4)
        gpu = sorted(nano.timed(24) for _ in range(3))[1]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        nano.run(12)                      # the queues are empty: this is the host's own time per step
        host = (time.perf_counter() - t0) / 12
        torch.cuda.synchronize()
        delays[f"+{extra_us} us of host work per step"] = {"ms_per_step": gpu * 1e3, "host_ms_per_step": host * 1e3}
    nano.step = plain_step
    out["host_delay"] = delays
    return out


def preheat(stepper, seconds=2.0):
    """Run the layer until the chip has been busy for `seconds`: clocks and temperature settle at what a
    training run sees, instead of the first timed window getting a cool chip and the last a hot one."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        stepper.run(4)
        torch.cuda.synchronize()


def interleaved_rounds(steppers, steps_per_turn, rounds):
    """Time the given ways of running the layer in turn, `rounds` times over (A B C A B C ...), so that
    all of them see the same chip state; returns name -> median seconds per step."""
    samples = {name: [] for name in steppers}
    for _ in range(rounds):
        for name, st in steppers.items():
            samples[name].append(st.timed(steps_per_turn))
    return {name: sorted(v)[len(v) // 2] for name, v in samples.items()}, samples


def host_enqueue_ms(stepper, repeats=5):
    """Host time to enqueue one step (forward and backward calls return once everything is queued);
    the GPU is idle at the start of each measurement, so nothing here waits for the device."""
    times = []
    for _ in range(repeats):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        stepper.step()
        times.append(time.perf_counter() - t0)
        torch.cuda.synchronize()
    return sorted(times)[len(times) // 2] * 1e3


def energy_per_iteration(stepper, tokens, sec_per_step, min_seconds=2.0, min_steps=20):
    """Board power sampled at 100 Hz on a thread while the layer runs; every iteration ends with a device
    synchronisation and a timestamp, and the samples are integrated over each iteration's window (the
    pattern of the reference's per-window energy measurement, tests/bayesian/common/hardware.py:121-132).
    Iterations shorter than two sampling periods are grouped so that every window holds samples."""
    from kareus_amd.energy import PowerSampler

    sampler = PowerSampler(0, hz=100.0)
    if not sampler.available:
        return {"joules_per_token": None}
    group = max(1, int(0.03 / sec_per_step) + 1)            # iterations per energy window (>= 30 ms)
    windows = max(min_steps // group + 1, int(min_seconds / (sec_per_step * group)) + 1)
    sampler.start()
    torch.cuda.synchronize()
    marks = [time.perf_counter()]
    for _ in range(windows):
        stepper.run(group)
        torch.cuda.synchronize()
        marks.append(time.perf_counter())
    sampler.stop()
    per_iter = []
    for a, b in zip(marks, marks[1:]):
        e = sampler.energy_joules(a, b)
        if e is not None:
            per_iter.append(e / group)
    total = sampler.energy_joules(marks[0], marks[-1])
    if total is None or not per_iter:
        return {"joules_per_token": None}
    n = windows * group
    return {
        "joules_per_token": total / (n * tokens), "mean_watts": total / (marks[-1] - marks[0]),
        "energy": {"iterations": n, "iterations_per_window": group, "joules_per_iteration_mean": total / n,
                   "joules_per_iteration_min": min(per_iter), "joules_per_iteration_max": max(per_iter),
                   "joules_per_iteration": [round(e, 4) for e in per_iter[:32]],
                   "power_sensor_bus_id": sampler.bus_id},
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c4", choices=sorted(WORKLOADS))
    ap.add_argument("--nanobatches", default="workload",
                    help="'workload' (default): the workload's nanobatch count, which is what `value` reports; "
                         "'auto': the faster of that count and one nanobatch, measured; or a number")
    ap.add_argument("--schedule", default=None,
                    help="per-microbatch plan file for the nanobatched run (default: the shipped plan for c5, none otherwise)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip the partition, energy and host-enqueue legs")
    ap.add_argument("--one-stream", action="store_true",
                    help="run every nanobatch on the caller's stream (no overlap; for profiling)")
    ap.add_argument("--same-launches-one-stream", action="store_true",
                    help="run only: K steps of the nanobatched step's own launches, all on the caller's stream "
                         "(the region the roofline kernel is timed in; for the kernel trace of it)")
    ap.add_argument("--roofline-only", action="store_true",
                    help="run only the dominant-kernel leg (the command profiled under profiles/)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run only a residual-add kernel of known size (calibrates FETCH_SIZE/WRITE_SIZE)")
    ap.add_argument("--attention-kernels", action="store_true",
                    help="run only the attention forward/backward stand-alone (TFLOP/s against the MFMA peak)")
    ap.add_argument("--attention-padded-shapes", action="store_true",
                    help="run only: attention at head dimension 64 and ragged lengths, padded into the MFMA kernels "
                         "and on the general kernels")
    ap.add_argument("--hbm-kernels", action="store_true",
                    help="run only the HBM-bound kernels stand-alone (achieved TB/s against 8 TB/s)")
    ap.add_argument("--with-library-matmul", action="store_true",
                    help="with --gemm-kernels: also time torch.matmul on the plain GEMMs, as a yardstick")
    ap.add_argument("--gemm-kernels", action="store_true",
                    help="run only the layer's twelve GEMMs stand-alone at nanobatch shape, as the engine launches them")
    ap.add_argument("--cu-budget-sweep", action="store_true",
                    help="run only the nanobatched step under schedules reserving 0..64 compute units")
    ap.add_argument("--overlap-bound", action="store_true",
                    help="run only: the nanobatched step with its HBM-bound launches suppressed (the best any "
                         "overlap could do) and with extra host work per step")
    ap.add_argument("--partition-timeline", action="store_true",
                    help="run only: start and end of every partition of every nanobatch inside one step (events, "
                         "no profiler), with the weight-gradient launches where the engine puts them and where the "
                         "last nanobatch delivers its operands")
    ap.add_argument("--power-trace", action="store_true",
                    help="run only the power / shader-clock trace over kernels and layer steps")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs one GPU's shard of the layer; --gpus must be 1 "
                 "(no collective path exists to run on more)")
    if not torch.cuda.is_available():
        sys.exit("bench.py: needs a HIP device")

    w = dict(WORKLOADS[args.workload])
    choice = args.nanobatches
    if choice not in ("auto", "workload"):
        w["nnb"] = int(choice)
        choice = "fixed"
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.roofline_only:
        # stand-alone leg: a 2 s pre-heat in front, so that its launches run at the clocks they run at inside a step
        main_kernel, others = dominant_kernel_roofline(w, w["nnb"], device, preheat_s=2.0)
        print(json.dumps({"roofline": main_kernel, "roofline_others": others}))
        return
    if args.copy_calibration:
        print(json.dumps({"copy_calibration": copy_calibration(device)}))
        return
    if args.attention_kernels:
        print(json.dumps({"attention_kernels": attention_kernels(w, w["nnb"], device)}))
        return
    if args.partition_timeline:
        print(json.dumps({"partition_timeline": {
            "as the engine runs it": partition_timeline(w, device),
            "weight gradients launched where the last nanobatch delivers": partition_timeline(w, device, wgrad_launches_at_end=False)}}))
        return
    if args.attention_padded_shapes:
        print(json.dumps({"attention_padded_shapes": attention_padded_shapes(device)}))
        return
    if args.hbm_kernels:
        print(json.dumps({"hbm_kernels": hbm_kernels(w, w["nnb"], device)}))
        return
    if args.gemm_kernels:
        print(json.dumps({"gemm_kernels": gemm_kernels(w, w["nnb"], device, with_library=args.with_library_matmul)}))
        return
    if args.cu_budget_sweep:
        print(json.dumps({"cu_budget_sweep_ms_per_step": cu_budget_sweep(w, device)}))
        return
    if args.power_trace:
        print(json.dumps({"power_trace": power_trace(w, device)}))
        return
    if args.same_launches_one_stream:
        gen = torch.Generator().manual_seed(42)
        x = torch.randn(w["s"], w["b"], w["h"], generator=gen).to(device, torch.bfloat16).requires_grad_(True)
        go = torch.randn(w["s"], w["b"], w["h"], generator=gen).to(device, torch.bfloat16)
        st = Stepper(make_model(w, w["nnb"], device, all_on_one_stream=True), x, go)
        st.run(2)
        preheat(st, 2.0)
        st.run(args.warmup)
        print(json.dumps({"same_launches_one_stream_ms_per_step": st.timed(args.steps) * 1e3, "steps": args.steps}))
        return
    if args.overlap_bound:
        print(json.dumps({"overlap_bound": overlap_bound(w, device)}))
        return
    gen = torch.Generator().manual_seed(42)
    x = torch.randn(w["s"], w["b"], w["h"], generator=gen).to(device, torch.bfloat16).requires_grad_(True)
    go = torch.randn(w["s"], w["b"], w["h"], generator=gen).to(device, torch.bfloat16)
    tokens = w["b"] * w["s"]
    flops = total_flops(w)

    schedule_path = args.schedule
    if schedule_path is None and args.workload == "c5":
        from kareus_amd.plans import plan_path

        schedule_path = plan_path("llama31_8b_4layers_mbs2_seq8192.py")
    nano = Stepper(make_model(w, w["nnb"], device, use_streams=not args.one_stream,
                              schedule=make_scheduler(schedule_path, w["nnb"])), x, go)
    ways = {"nanobatched": nano}
    if w["nnb"] > 1:
        ways["serial_1nb"] = Stepper(make_model(w, 1, device, use_streams=False), x, go)
        if not args.no_extras:
            ways["same_nb_one_stream"] = Stepper(make_model(w, w["nnb"], device, use_streams=False,
                                                            schedule=make_scheduler(schedule_path, w["nnb"])), x, go)
    # for the roofline kernel only: the launches of the nanobatched step, one after the other
    same_launches = None
    if w["nnb"] > 1 and not args.one_stream:
        same_launches = Stepper(make_model(w, w["nnb"], device, all_on_one_stream=True,
                                           schedule=make_scheduler(schedule_path, w["nnb"])), x, go)
        same_launches.run(2)
    for st in ways.values():
        st.run(2)
    preheat(nano, 2.0)
    med, samples = interleaved_rounds(ways, max(3, args.steps // 4), 5)
    picked = "nanobatched"
    if choice == "auto" and "serial_1nb" in med and med["serial_1nb"] < med["nanobatched"]:
        picked = "serial_1nb"
    runner = ways[picked]
    run_nnb = 1 if picked == "serial_1nb" else w["nnb"]

    # the headline: W warm-up steps, then exactly K timed steps of the chosen configuration
    runner.run(args.warmup)
    from kareus_amd.backend import get_backend

    watched = dominant_gemm_shapes(w, run_nnb)
    if run_nnb > 1:
        # With several nanobatches the host needs nearly as long to enqueue a step as the device to run it, and
        # the roofline kernel is timed in a region of its own below anyway: the headline steps carry no events;
        # the intervals of the watched GEMMs on the concurrent streams come from K further steps right after.
        sec = runner.timed(args.steps)
        with GemmEventTimer(get_backend("hip"), watched.values()) as in_step:
            runner.timed(args.steps)
    else:
        with GemmEventTimer(get_backend("hip"), watched.values()) as in_step:
            sec = runner.timed(args.steps)
    # A kernel's interval on its own stream is its duration only while nothing else runs beside it.  With the
    # nanobatches on concurrent streams it also holds the time its workgroups wait for compute units that the
    # other streams' kernels occupy, so the roofline kernel is timed in a second region of K steps of the SAME
    # nanobatches — the same launches, shapes and epilogues — on one stream.
    alone_in_step = None
    if run_nnb > 1 and same_launches is not None:
        same_launches.run(args.warmup)
        with GemmEventTimer(get_backend("hip"), watched.values()) as alone_in_step:
            one_stream_sec = same_launches.timed(args.steps)
    # beside it, timed the same way: the one-nanobatch (serial) step of the same layer and data
    serial_sec = None
    if "serial_1nb" in ways and picked != "serial_1nb":
        ways["serial_1nb"].run(args.warmup)
        serial_sec = ways["serial_1nb"].timed(args.steps)

    out = {
        "metric": "layer fwd+bwd tokens/sec on 1 MI355X",
        "value": tokens / sec, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": sec * 1e3, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{args.workload}: {w['label']}", "hidden": w["h"], "q_heads": w["nq"],
                   "kv_heads": w["nkv"], "head_dim": w["hd"], "ffn": w["ffn"], "layers": w["layers"],
                   "batch": w["b"], "seq_len": w["s"], "nanobatches": run_nnb,
                   "nanobatches_of_the_workload": w["nnb"],
                   "nanobatch_choice": {"auto": "measured: the faster of the workload's count and one nanobatch",
                                        "workload": "the workload's count", "fixed": "given on the command line"}[choice],
                   "schedule_file": os.path.relpath(schedule_path, ROOT) if (schedule_path and run_nnb > 1) else None},
        "mfma_util_end_to_end": flops / sec / MFMA_PEAK_BF16,
        "tflops_end_to_end": flops / sec / 1e12,
    }
    if serial_sec is not None:
        out["serial_1nb"] = {"what": "the same layer and data run as one nanobatch on one stream (no overlap engine at "
                                     "work), same warm-up and step count, timed right after the headline steps",
                             "value": tokens / serial_sec, "unit": "tokens/s", "ms_per_step": serial_sec * 1e3,
                             "mfma_util_end_to_end": flops / serial_sec / MFMA_PEAK_BF16}
    if "serial_1nb" in med:
        out["overlap"] = {
            "timing": "interleaved rounds after a 2 s pre-heat, median of 5 rounds per way",
            "nanobatched_ms": med["nanobatched"] * 1e3,
            "serial_1nb_ms": med["serial_1nb"] * 1e3,
            "speedup_vs_serial_1nb": med["serial_1nb"] / med["nanobatched"],
            "rounds_ms": {k: [round(t * 1e3, 4) for t in v] for k, v in samples.items()},
            # the plan file steers the nanobatched ways; one nanobatch has no slots to schedule
            "schedule_file_of_the_nanobatched_ways": os.path.relpath(schedule_path, ROOT) if schedule_path else None,
        }
        if "same_nb_one_stream" in med:
            out["overlap"]["same_nb_one_stream_ms"] = med["same_nb_one_stream"] * 1e3
            out["overlap"]["speedup_vs_one_stream"] = med["same_nb_one_stream"] / med["nanobatched"]

    if not args.no_extras:
        out.update(energy_per_iteration(runner, tokens, sec))
        out["host_enqueue_ms_per_step"] = {name: host_enqueue_ms(st) for name, st in ways.items()
                                           if name != "same_nb_one_stream"}
        flat = ways.get("same_nb_one_stream")
        if flat is not None:
            # per-partition times: the same nanobatches on one stream, an event pair around each partition
            parts = partition_times(flat)
            out["overlap"]["partition_ms"] = parts
            out["overlap"]["overlap_efficiency"] = sum(parts.values()) * 1e-3 / med["nanobatched"]

    ways.clear()
    del nano, runner, same_launches
    # roofline of the dominant kernel: its launches inside the K timed steps; the same kernel
    # launched back to back on its own (a hotter chip: nothing but the heaviest GEMM) beside it
    alone_main, alone_others = dominant_kernel_roofline(w, run_nnb, device)
    entries = []
    for alone in [alone_main] + alone_others:
        layout = alone["kernel"].split("<")[1][:2]
        acc = None
        s, n_launches = in_step.seconds(watched[layout], acc)
        if s is None:
            entries.append(dict(alone, measured="back to back on its own"))
            continue
        if alone_in_step is not None:
            s1, n1 = alone_in_step.seconds(watched[layout], acc)
            e = _roofline_entry(alone["kernel"], layout, *watched[layout][1:], s1)
            e["measured"] = (f"HIP events around its {n1} launches inside {args.steps} timed steps of the same "
                             f"{run_nnb} nanobatches on one stream ({one_stream_sec * 1e3:.3f} ms per step): there the "
                             "interval is the kernel's own duration")
            e["interval_on_concurrent_streams_us"] = s * 1e6
            e["interval_on_concurrent_streams_is"] = (
                f"the same {n_launches} launches inside {args.steps} further steps of the headline configuration, run "
                "right after the headline steps: the interval on the launch stream, which includes waiting for "
                "compute units held by the other nanobatch streams' kernels")
        else:
            e = _roofline_entry(alone["kernel"], layout, *watched[layout][1:], s)
            e["measured"] = f"HIP events around its {n_launches} launches inside the {args.steps} timed steps"
        e["back_to_back_alone_us"] = alone["avg_launch_us"]
        entries.append(e)
    out["roofline"], out["roofline_others"] = entries[0], entries[1:]
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
