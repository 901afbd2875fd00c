#!/usr/bin/env python3
"""Layer fwd+bwd throughput of the partition-overlap engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c4|c2|c3|c5|c1gpu]

A step = one forward+backward of the decoder-layer stack over one synthetic batch, inputs
resident in HBM.  Prints ONE JSON line (metric: layer fwd+bwd tokens/s) that also carries
  roofline      the dominant kernel (fc1 forward GEMM at nanobatch shape) timed live with HIP
                events on its stream, against the 2.5 PFLOP/s dense bf16 MFMA peak
  cpu_baseline  the CPU oracle (plain PyTorch fp32 layer) timed on the host cores on a bounded
                sample of the same layer shape
plus end-to-end MFMA utilisation, speed-up over the serial (1 nanobatch) run, overlap
efficiency (sum of serially timed partition times / overlapped wall time) and joules/token.
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
    "c1gpu": dict(h=512, nq=4, nkv=4, hd=128, ffn=1376, layers=1, b=2, s=256, nnb=2,
                  label="plumbing-sized layer (h512) in bf16"),
    "c2": dict(h=3072, nq=3, nkv=1, hd=128, ffn=1024, layers=1, b=8, s=4096, nnb=2,
               label="Llama-3.2-3B layer, TP=8 shard, MBS 8 x seq 4096, 2 nanobatches"),
    "c3": dict(h=3072, nq=24, nkv=8, hd=128, ffn=8192, layers=1, b=4, s=4096, nnb=2,
               label="Llama-3.2-3B full-width layer, MBS 4 x seq 4096"),
    "c4": dict(h=4096, nq=8, nkv=2, hd=128, ffn=3584, layers=1, b=4, s=4096, nnb=4,
               label="Llama-3.1-8B layer, TP=4 shard, MBS 4 x seq 4096, 4 nanobatches"),
    "c5": dict(h=4096, nq=32, nkv=8, hd=128, ffn=14336, layers=4, b=2, s=8192, nnb=2,
               label="4-layer full-width Llama-3.1-8B stack, MBS 2 x seq 8192, 2 nanobatches"),
}


def total_flops(w) -> float:
    t = w["b"] * w["s"]
    gemm_fwd = 2 * t * (w["h"] * (w["nq"] + 2 * w["nkv"]) * w["hd"] + w["nq"] * w["hd"] * w["h"]
                        + w["h"] * 2 * w["ffn"] + w["ffn"] * w["h"])
    attn_fwd = 2 * w["b"] * w["nq"] * w["s"] ** 2 * w["hd"]
    return w["layers"] * (3 * gemm_fwd + 3.5 * attn_fwd)


def make_model(w, nnb, device, use_streams=True, schedule=None):
    from kareus_amd import LayerConfig, LayerStack

    cfg = LayerConfig(hidden_size=w["h"], num_attention_heads=w["nq"], num_query_groups=w["nkv"],
                      kv_channels=w["hd"], ffn_hidden_size=w["ffn"], num_layers=w["layers"],
                      num_nanobatches=nnb, backend="hip", use_streams=use_streams)
    cfg.kareus_scheduler = schedule
    return LayerStack(cfg, device=device, seed=1234)


def run_steps(model, x, go, steps):
    for _ in range(steps):
        for p in model.parameters():
            p.grad = None
        x.grad = None
        y = model(x)
        y.backward(go)


def time_steps(model, x, go, steps, warmup):
    run_steps(model, x, go, warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run_steps(model, x, go, steps)
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


def partition_times(model, x, go, iters=3):
    from kareus_amd.partitions.partition_base import PartitionBase

    run_steps(model, x, go, 1)
    torch.cuda.synchronize()
    timer = EventTimer()
    PartitionBase.timer = timer
    try:
        run_steps(model, x, go, iters)
        torch.cuda.synchronize()
    finally:
        PartitionBase.timer = None
    return {k: v / iters for k, v in timer.totals().items()}


# HBM-side bytes per launch of the TN GEMM, from hardware counters (FETCH_SIZE and WRITE_SIZE of
# two profiler runs of `bench.py --roofline-only`, each scaled by what the same counter reads for
# `bench.py --copy-calibration`: x2.000 and x1.000).  Keyed by (M, N, K); shapes that were not
# profiled report null.
MEASURED_TRAFFIC_BYTES = {
    (4096, 7168, 4096): 369.7e6 + 58.7e6,
}


def dominant_kernel_roofline(w, nnb, device, launches=30):
    """fc1 forward GEMM, y[T_nb, 2F] = x[T_nb, h] . W[2F, h]^T, timed with HIP events on the
    stream it is launched on (torch's current stream)."""
    from kareus_amd.backend import get_backend

    be = get_backend("hip")
    m, n, k = (w["b"] // nnb) * w["s"], 2 * w["ffn"], w["h"]
    a = torch.randn(m, k, device=device).bfloat16()
    wt = (torch.randn(n, k, device=device) * 0.02).bfloat16()
    for _ in range(5):
        be.linear_fwd(a, wt)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(launches):
        be.linear_fwd(a, wt)
    e1.record()
    torch.cuda.synchronize()
    sec = e0.elapsed_time(e1) * 1e-3 / launches
    flops = 2.0 * m * n * k
    achieved = flops / sec / 1e12
    return {
        "bound": "mfma", "kernel": "gemm_kernel<TN> (fc1 forward)", "shape": [m, n, k],
        "flops_per_launch": flops, "avg_launch_us": sec * 1e6,
        "achieved": achieved, "peak": MFMA_PEAK_BF16 / 1e12, "unit": "TFLOP/s",
        "frac": achieved * 1e12 / MFMA_PEAK_BF16,
        "traffic": MEASURED_TRAFFIC_BYTES.get((m, n, k)),
    }


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c4", choices=sorted(WORKLOADS))
    ap.add_argument("--nanobatches", type=int, default=0, help="override the workload's nanobatch count")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip serial/partition/energy legs")
    ap.add_argument("--one-stream", action="store_true",
                    help="run every nanobatch on the caller's stream (no overlap; for profiling)")
    ap.add_argument("--roofline-only", action="store_true",
                    help="run only the dominant-kernel leg (the command profiled under profiles/)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run only a residual-add kernel of known size (calibrates FETCH_SIZE/WRITE_SIZE)")
    ap.add_argument("--attention-kernels", action="store_true",
                    help="run only the attention forward/backward stand-alone (TFLOP/s against the MFMA peak)")
    ap.add_argument("--hbm-kernels", action="store_true",
                    help="run only the HBM-bound kernels stand-alone (achieved TB/s against 8 TB/s)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs one GPU's shard of the layer; --gpus must be 1 "
                 "(no collective path exists to run on more)")
    if not torch.cuda.is_available():
        sys.exit("bench.py: needs a HIP device")

    w = dict(WORKLOADS[args.workload])
    if args.nanobatches:
        w["nnb"] = args.nanobatches
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.roofline_only:
        print(json.dumps({"roofline": dominant_kernel_roofline(w, w["nnb"], device)}))
        return
    if args.copy_calibration:
        print(json.dumps({"copy_calibration": copy_calibration(device)}))
        return
    if args.attention_kernels:
        print(json.dumps({"attention_kernels": attention_kernels(w, w["nnb"], device)}))
        return
    if args.hbm_kernels:
        print(json.dumps({"hbm_kernels": hbm_kernels(w, w["nnb"], device)}))
        return
    gen = torch.Generator().manual_seed(42)
    x = torch.randn(w["s"], w["b"], w["h"], generator=gen).to(device, torch.bfloat16).requires_grad_(True)
    go = torch.randn(w["s"], w["b"], w["h"], generator=gen).to(device, torch.bfloat16)
    tokens = w["b"] * w["s"]
    flops = total_flops(w)

    model = make_model(w, w["nnb"], device, use_streams=not args.one_stream)
    sec = time_steps(model, x, go, args.steps, args.warmup)

    out = {
        "metric": "layer fwd+bwd tokens/sec on 1 MI355X",
        "value": tokens / sec, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": sec * 1e3, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{args.workload}: {w['label']}", "hidden": w["h"], "q_heads": w["nq"],
                   "kv_heads": w["nkv"], "head_dim": w["hd"], "ffn": w["ffn"], "layers": w["layers"],
                   "batch": w["b"], "seq_len": w["s"], "nanobatches": w["nnb"]},
        "mfma_util_end_to_end": flops / sec / MFMA_PEAK_BF16,
        "tflops_end_to_end": flops / sec / 1e12,
    }

    if not args.no_extras:
        # energy: keep the layer running for >= 2 s under the power sampler
        from kareus_amd.energy import PowerSampler

        sampler = PowerSampler(0, hz=100.0)
        if sampler.available:
            n_e = max(args.steps, int(2.0 / sec) + 1)
            sampler.start()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            run_steps(model, x, go, n_e)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            sampler.stop()
            joules = sampler.energy_joules(t0, t1)
            if joules is not None:
                out["joules_per_token"] = joules / (n_e * tokens)
                out["mean_watts"] = joules / (t1 - t0)
        else:
            out["joules_per_token"] = None

        # serial baseline: one nanobatch, one stream
        del model
        serial = make_model(w, 1, device, use_streams=False)
        sec_serial = time_steps(serial, x, go, max(3, args.steps // 2), 2)
        del serial
        # same nanobatch count, all on one stream (no overlap), with per-partition events
        flat = make_model(w, w["nnb"], device, use_streams=False)
        sec_flat = time_steps(flat, x, go, max(3, args.steps // 2), 2)
        parts = partition_times(flat, x, go)
        del flat
        out["overlap"] = {
            "serial_1nb_ms": sec_serial * 1e3,
            "same_nb_one_stream_ms": sec_flat * 1e3,
            "speedup_vs_serial_1nb": sec_serial / sec,
            "speedup_vs_one_stream": sec_flat / sec,
            "partition_ms": parts,
            "overlap_efficiency": sum(parts.values()) * 1e-3 / sec,
        }

    out["roofline"] = dominant_kernel_roofline(w, w["nnb"], device)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
