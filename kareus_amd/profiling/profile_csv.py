"""Eval logs of the four partitions -> the per-stage candidate table the schedule solver reads.

Does for this build's logs what the reference's generator does for its own
(tests/kareus/generate_profile_csv.py, non-context-parallel branch ``_main_non_cp`` :268-446):

* read ``fwd_attn / fwd_mlp / bwd_attn / bwd_mlp`` eval logs (JSON lines with ``freq,
  overlap_start, overlap_end, sm, block, time_s, energy_j`` — rows missing a field or with no
  energy are skipped) and group them by frequency (:116-179);
* for every frequency present in all four, combine one attention and one MLP configuration
  (with activation recompute a backward candidate also carries the recompute-forward pair),
  sum time and energy, optionally scale by 1.15, multiply by ``layers of the stage x
  nanobatches`` and add the stage's embedding / output-layer / loss figures when given
  (:318-401);
* keep, per stage and direction, the points that are Pareto-optimal in (time, energy minus
  idle power x time) (:182-205) and write them as
  ``stage,instruction,frequency,[recompute_attention_configs,recompute_mlp_configs,]
  attention_configs,mlp_configs,time,energy`` with each configuration spelled
  ``<start>-<end>-<sm>-<block>`` — the string the schedule parser accepts (:403-442).

The embedding / output / loss ("non-partition") figures are optional here: this build has no
such operators, so they default to zero.
"""

from __future__ import annotations

import itertools
import json
import os
import warnings
from typing import Dict, List, Optional, Sequence, Tuple

Config = Tuple[object, object, int, int]          # (overlap_start, overlap_end, sm, block)
Measured = Tuple[float, float]                    # (time_s, energy_j)
Point = Tuple[tuple, Measured]

_FIELDS = ("freq", "overlap_start", "overlap_end", "sm", "block", "time_s", "energy_j")
NONPARTITION_KEYS = ("forward-embedding", "forward-output", "loss-func", "backward-embedding", "backward-output")

# Power a GPU draws while it waits on a pipeline neighbour (W); subtracted from energy when
# ranking candidates.  The reference lists its GPUs in tests/bayesian/common/model_config.py:13-16;
# the MI355X figure is the board power read from its hwmon sensor over 4 s with a HIP context open
# and no kernel running (261-294 W, mean 286 W).
P2P_POWER_W = {"A40": 70.0, "A100": 85.0, "MI355X": 286.0}


def read_eval_log(path: str) -> Dict[int, List[Tuple[Config, Measured]]]:
    """frequency -> [((start, end, sm, block), (time_s, energy_j)), ...]"""
    if not os.path.exists(path):
        raise FileNotFoundError(path)
    by_freq: Dict[int, List[Tuple[Config, Measured]]] = {}
    with open(path) as f:
        for line in f:
            line = line.strip()
            if not line:
                continue
            try:
                row = json.loads(line)
            except ValueError:
                continue
            if not all(k in row for k in _FIELDS) or row["energy_j"] is None:
                continue
            cfg = (row["overlap_start"], row["overlap_end"], int(row["sm"]), int(row["block"]))
            by_freq.setdefault(int(row["freq"]), []).append((cfg, (float(row["time_s"]), float(row["energy_j"]))))
    return by_freq


def pareto_optimal(points: Sequence[Point], p2p_power: float, min_improvement: float = 1e-4) -> List[Point]:
    """Walk the points by increasing time; keep one only if its effective energy
    (energy - p2p_power * time) beats the best kept so far by more than ``min_improvement``."""
    kept: List[Point] = []
    best = float("inf")
    for cfg, (t, e) in sorted(points, key=lambda p: (p[1][0], p[1][1])):
        effective = e - p2p_power * t
        if effective + min_improvement < best:
            kept.append((cfg, (t, e)))
            best = effective
    return kept


def layers_per_stage(num_layers: int, pipeline_parallel_size: int, first: int = 0, last: int = 0) -> List[int]:
    """Layers of each pipeline stage; ``first`` / ``last`` fix the outer stages' counts, the
    middle stages share the rest as evenly as possible, earlier ones taking the remainder."""
    if pipeline_parallel_size <= 0:
        raise ValueError("pipeline_parallel_size must be positive")
    if pipeline_parallel_size == 1:
        return [num_layers]
    first, last = max(0, int(first)), max(0, int(last))
    if pipeline_parallel_size == 2:
        if first + last != num_layers:
            if first > num_layers:
                warnings.warn(f"First stage layers ({first}) exceed total layers ({num_layers}); clamping to total.")
                first = num_layers
            last = max(0, num_layers - first)
        return [first, last]
    rest = num_layers - first - last
    if rest < 0:
        warnings.warn(f"first({first}) + last({last}) exceed total layers ({num_layers}); reducing last to fit.")
        last = max(0, num_layers - first)
        rest = num_layers - first - last
    middle = pipeline_parallel_size - 2
    shares = [rest // middle + (1 if i < rest % middle else 0) for i in range(middle)]
    out = [first] + shares + [last]
    out[-1] = max(0, out[-1] + num_layers - sum(out))
    return out


def _cfg_str(cfg: Config) -> str:
    return "-".join(str(x) for x in cfg)


def candidate_points(
    logs: Dict[str, Dict[int, List[Tuple[Config, Measured]]]],
    stage_layers: Sequence[int],
    nanobatches: int = 2,
    use_activation_checkpointing: bool = True,
    scale_time_energy: bool = True,
    nonpartition: Optional[Dict[int, Dict[str, Measured]]] = None,
) -> Tuple[Dict[int, List[Point]], Dict[int, List[Point]]]:
    """(forward points per stage, backward points per stage); a point's key is
    ``(frequency, attn_cfg, mlp_cfg)`` or, for backward with recompute,
    ``(frequency, rec_attn_cfg, rec_mlp_cfg, attn_cfg, mlp_cfg)``."""
    freqs = sorted(set.intersection(*(set(logs[k]) for k in ("fwd_attn", "fwd_mlp", "bwd_attn", "bwd_mlp"))))
    if not freqs:
        raise RuntimeError("No overlapping frequencies found across the four partitions' eval logs.")
    stages = len(stage_layers)
    scale = 1.15 if scale_time_energy else 1.0
    zero = {k: (0.0, 0.0) for k in NONPARTITION_KEYS}
    fwd: Dict[int, List[Point]] = {s: [] for s in range(stages)}
    bwd: Dict[int, List[Point]] = {s: [] for s in range(stages)}

    def add(table, key, parts, extras_of_stage):
        t = sum(p[0] for p in parts) * scale
        e = sum(p[1] for p in parts) * scale
        for s in range(stages):
            ts, es = t * stage_layers[s] * nanobatches, e * stage_layers[s] * nanobatches
            for (xt, xe), times in extras_of_stage(s):
                ts, es = ts + xt * times, es + xe * times
            table[s].append((key, (ts, es)))

    for f in freqs:
        extra = dict(zero, **((nonpartition or {}).get(f, {})))

        def fwd_extras(s, extra=extra):
            if s == 0:
                return [(extra["forward-embedding"], 1)]
            if s == stages - 1:
                return [(extra["forward-output"], 1), (extra["loss-func"], 1)]
            return []

        def bwd_extras(s, extra=extra):
            if s == 0:
                return [(extra["backward-embedding"], 2)]
            if s == stages - 1:
                return [(extra["backward-output"], 1)]
            return []

        for (ac, ar), (mc, mr) in itertools.product(logs["fwd_attn"][f], logs["fwd_mlp"][f]):
            add(fwd, (f, ac, mc), [ar, mr], fwd_extras)
        if use_activation_checkpointing:
            for (rac, rar), (rmc, rmr), (ac, ar), (mc, mr) in itertools.product(
                    logs["fwd_attn"][f], logs["fwd_mlp"][f], logs["bwd_attn"][f], logs["bwd_mlp"][f]):
                add(bwd, (f, rac, rmc, ac, mc), [rar, rmr, ar, mr], bwd_extras)
        else:
            for (ac, ar), (mc, mr) in itertools.product(logs["bwd_attn"][f], logs["bwd_mlp"][f]):
                add(bwd, (f, ac, mc), [ar, mr], bwd_extras)
    return fwd, bwd


def write_profile_csv(
    path: str,
    forward: Dict[int, List[Point]],
    backward: Dict[int, List[Point]],
    p2p_power: float,
    use_activation_checkpointing: bool = True,
) -> Dict[str, int]:
    """Write the Pareto-optimal candidates of every stage; returns how many were kept."""
    kept = {"forward": 0, "backward": 0}
    with open(path, "w") as f:
        if use_activation_checkpointing:
            f.write("stage,instruction,frequency,recompute_attention_configs,recompute_mlp_configs,"
                    "attention_configs,mlp_configs,time,energy\n")
        else:
            f.write("stage,instruction,frequency,attention_configs,mlp_configs,time,energy\n")
        for stage in sorted(forward):
            for name, table in (("forward", forward), ("backward", backward)):
                for key, (t, e) in pareto_optimal(table[stage], p2p_power):
                    freq, cfgs = key[0], [_cfg_str(c) for c in key[1:]]
                    if use_activation_checkpointing and len(cfgs) == 2:
                        cfgs = ["", ""] + cfgs
                    f.write(f"{stage},{name},{freq},{','.join(cfgs)},{t},{e}\n")
                    kept[name] += 1
    return kept


def generate_profile_csv(
    log_dir: str,
    output_path: str,
    num_layers: int,
    pipeline_parallel_size: int = 1,
    num_layers_in_first_pipeline_stage: int = 0,
    num_layers_in_last_pipeline_stage: int = 0,
    nanobatches: int = 2,
    gpu_type: str = "MI355X",
    use_activation_checkpointing: bool = True,
    scale_time_energy: bool = True,
    nonpartition: Optional[Dict[int, Dict[str, Measured]]] = None,
) -> Dict[str, int]:
    """``log_dir`` holds ``<partition>.jsonl`` (what ``python -m kareus_amd.profiling --out``
    writes) or the reference's ``<partition>/eval_results.jsonl`` for the four partitions."""
    if gpu_type not in P2P_POWER_W:
        raise ValueError(f"Unknown GPU type {gpu_type!r}. Available: {list(P2P_POWER_W)}")
    logs = {}
    for key in ("fwd_attn", "fwd_mlp", "bwd_attn", "bwd_mlp"):
        flat, nested = os.path.join(log_dir, f"{key}.jsonl"), os.path.join(log_dir, key, "eval_results.jsonl")
        logs[key] = read_eval_log(flat if os.path.exists(flat) else nested)
    stage_layers = layers_per_stage(num_layers, pipeline_parallel_size,
                                    num_layers_in_first_pipeline_stage, num_layers_in_last_pipeline_stage)
    fwd, bwd = candidate_points(logs, stage_layers, nanobatches, use_activation_checkpointing,
                                scale_time_energy, nonpartition)
    return write_profile_csv(output_path, fwd, bwd, P2P_POWER_W[gpu_type], use_activation_checkpointing)


def main(argv=None) -> int:
    """``python -m kareus_amd.profiling.profile_csv --log-dir logs --output profile.csv --num-layers 1``"""
    import argparse

    ap = argparse.ArgumentParser(prog="python -m kareus_amd.profiling.profile_csv")
    ap.add_argument("--log-dir", required=True, help="directory with the four partitions' eval logs")
    ap.add_argument("--output", required=True)
    ap.add_argument("--num-layers", type=int, required=True)
    ap.add_argument("--pipeline-parallel-size", type=int, default=1)
    ap.add_argument("--num-layers-in-first-pipeline-stage", type=int, default=0)
    ap.add_argument("--num-layers-in-last-pipeline-stage", type=int, default=0)
    ap.add_argument("--nanobatches", type=int, default=2)
    ap.add_argument("--gpu-type", default="MI355X")
    ap.add_argument("--no-activation-checkpointing", action="store_true")
    ap.add_argument("--no-scale", action="store_true", help="do not multiply time and energy by 1.15")
    args = ap.parse_args(argv)
    kept = generate_profile_csv(args.log_dir, args.output, args.num_layers, args.pipeline_parallel_size,
                                args.num_layers_in_first_pipeline_stage, args.num_layers_in_last_pipeline_stage,
                                args.nanobatches, args.gpu_type, not args.no_activation_checkpointing,
                                not args.no_scale)
    print(f"{args.output}: {kept['forward']} forward and {kept['backward']} backward candidates")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
