"""``python -m kareus_amd.profiling --partition fwd_attn [...]`` — sweep one partition's release
points (and, where the user may set them, shader clocks) and append eval-log rows (JSON lines:
freq, overlap_start, overlap_end, sm, block, time_s, energy_j) to ``--out``.

Defaults are the 8B TP=4 shard, 4 nanobatches of one 4096-token sequence each.
"""

from __future__ import annotations

import argparse
import json
import sys

import torch

from ..block import LayerConfig
from ..energy import PowerSampler
from . import PARTITION_KEYS, PartitionTest, all_configurations, append_eval_log, measure_batch
from .hardware import nominal_frequency_mhz


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m kareus_amd.profiling")
    ap.add_argument("--partition", choices=PARTITION_KEYS + ("nonpartition",), required=True,
                    help="one of the four partitions, or the work outside them (embedding, output layer, loss)")
    ap.add_argument("--vocab-rows", type=int, default=32064, help="vocabulary shard size (nonpartition)")
    ap.add_argument("--out-dir", default=".", help="directory for the nonpartition CSV files")
    ap.add_argument("--hidden", type=int, default=4096)
    ap.add_argument("--q-heads", type=int, default=8)
    ap.add_argument("--kv-heads", type=int, default=2)
    ap.add_argument("--head-dim", type=int, default=128)
    ap.add_argument("--ffn", type=int, default=3584)
    ap.add_argument("--batch", type=int, default=4)
    ap.add_argument("--seq-len", type=int, default=4096)
    ap.add_argument("--nanobatches", type=int, default=4)
    ap.add_argument("--freq", type=int, nargs="*", default=None, help="shader clocks in MHz (default: leave alone)")
    ap.add_argument("--sm", type=int, nargs="*", default=[16], help="CU budgets handed to the collective")
    ap.add_argument("--duration", type=float, default=2.0)
    ap.add_argument("--cooldown", type=float, default=1.0)
    ap.add_argument("--backend", default="hip")
    ap.add_argument("--out", default=None, help="JSONL file to append to (default: stdout only)")
    args = ap.parse_args(argv)

    device = "cuda:0" if args.backend == "hip" else "cpu"
    if args.backend == "hip" and not torch.cuda.is_available():
        sys.exit("python -m kareus_amd.profiling: the hip backend needs a GPU")
    cfg = LayerConfig(hidden_size=args.hidden, num_attention_heads=args.q_heads, num_query_groups=args.kv_heads,
                      kv_channels=args.head_dim, ffn_hidden_size=args.ffn, num_nanobatches=args.nanobatches,
                      backend=args.backend,
                      params_dtype=torch.bfloat16 if args.backend == "hip" else torch.float32)
    if args.partition == "nonpartition":
        from .nonpartition import NonPartitionProfiler

        prof = NonPartitionProfiler(cfg, args.vocab_rows, args.batch, args.seq_len, device=device)
        freq = (args.freq or [nominal_frequency_mhz()])[0]
        trials = prof.run(args.out_dir, freq, sampler=PowerSampler(), measurement_duration=args.duration,
                          cooldown_duration=args.cooldown)
        for name, t in trials.items():
            print(json.dumps({"step": name, "freq": freq, "time_s": t.time_per_iter, "energy_j": t.energy_per_iter}),
                  flush=True)
        return 0
    test = PartitionTest(args.partition, cfg, args.batch, args.seq_len, device=device)
    freqs = args.freq or [nominal_frequency_mhz()]
    configs = all_configurations(freqs, args.sm, test.overlap_windows)
    sampler = PowerSampler()
    for rec in measure_batch(test, configs, sampler, args.duration, args.cooldown):
        print(json.dumps(rec), flush=True)
        if args.out:
            append_eval_log(args.out, [rec])
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
