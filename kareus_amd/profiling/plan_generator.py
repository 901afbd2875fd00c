"""Per-stage candidate table (``profile_*.csv``) -> the plan files the schedulers step through.

The reference hands its candidate table to a driver (tests/kareus/run_optimization.py) around the
third-party ``lowtime`` package (not part of the reference tree, no version pinned there): it
builds one ``ExecutionOption`` per CSV row (:79-115), lays the instructions of every stage out in
synchronous 1F1B order (:381-402), lets the solver walk from the cheapest plan towards the fastest
one unit of time per iteration (:455-477) and writes, for every iteration,
``freqs_pipeline_<iteration>.py`` and ``scheds_pipeline_<iteration>.py`` (:198-262) followed by
three comment lines with the iteration's cost.

This module is the part of that which one GPU needs: **one pipeline stage**.  With one stage the
dependency graph is a chain, the iteration time is the sum of the instructions' times, and the
cheapest plan for a time budget is a multiple-choice knapsack, which a dynamic programme over the
quantised time solves exactly (no curve fitting, no min-cut).  Times are quantised to
``unit_time`` and the power a GPU draws anyway (``p2p_power``) is taken out of every option's
energy for the length of its quantised time, as the driver does (:374-375); the figure reported
as "total cost with P2P" adds it back for the whole iteration (:467).  More than one stage needs
the min-cut solver and is refused.

The written files have the reference's layout, so ``kareus_amd.scheduler.parse_schedule_file`` /
``parse_frequency_file`` and the two schedulers read them like a shipped plan.
"""

from __future__ import annotations

import argparse
import csv
import math
import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

from .profile_csv import P2P_POWER_W

__all__ = ["Option", "Plan", "read_profile_csv", "instruction_order", "plan_frontier", "write_plan_files",
           "generate_plans"]

_AC_COLUMNS = ("recompute_attention_configs", "recompute_mlp_configs", "attention_configs", "mlp_configs")
_PLAIN_COLUMNS = ("attention_configs", "mlp_configs")


@dataclass(frozen=True)
class Option:
    """One row of the candidate table: what an instruction costs when run with ``knob`` =
    ``(frequency, config strings...)`` (run_optimization.py:88-113)."""
    time: float
    energy: float
    knob: tuple


@dataclass(frozen=True)
class Plan:
    """One point of the stage's time/energy frontier.  ``assignment[i]`` is the option of the
    i-th instruction in 1F1B order."""
    iteration: int
    quant_time: int
    time: float            # sum of the chosen options' measured times
    cost: float            # energy with p2p_power taken out for the quantised times
    energy: float          # cost + p2p_power * quant_time * unit_time
    instructions: Tuple[Tuple[str, int], ...]
    assignment: Tuple[Option, ...]


def _text(value) -> str:
    """Missing configuration fields read as empty strings (run_optimization.py:69-75)."""
    if value is None:
        return ""
    s = str(value)
    return "" if s == "nan" else s


def read_profile_csv(path: str, use_activation_checkpointing: Optional[bool] = None
                     ) -> Tuple[Dict[int, Dict[str, List[Option]]], bool]:
    """``{stage: {"forward": [Option...], "backward": [...]}}`` and whether backward options carry
    the recompute pair.  A context-parallel table (column ``fwd_qkv_ar``) is refused: this build
    has no context-parallel partitions."""
    with open(path, newline="") as f:
        reader = csv.DictReader(f)
        header = reader.fieldnames or []
        if "fwd_qkv_ar" in header:
            raise ValueError("context-parallel candidate tables are not supported")
        for col in ("stage", "instruction", "frequency", "time", "energy") + _PLAIN_COLUMNS:
            if col not in header:
                raise ValueError(f"{path}: column {col!r} is missing")
        has_recompute = all(c in header for c in _AC_COLUMNS)
        ac = has_recompute if use_activation_checkpointing is None else bool(use_activation_checkpointing)
        if ac and not has_recompute:
            raise ValueError(f"{path}: activation checkpointing asked for, but the table has no recompute columns")
        table: Dict[int, Dict[str, List[Option]]] = {}
        for row in reader:
            name = row["instruction"].strip().lower()
            if name not in ("forward", "backward"):
                raise ValueError(f"Unknown instruction name: {row['instruction']}")
            cols = _AC_COLUMNS if (ac and name == "backward") else _PLAIN_COLUMNS
            knob = (int(float(row["frequency"])),) + tuple(_text(row.get(c)) for c in cols)
            opt = Option(float(row["time"]), float(row["energy"]), knob)
            table.setdefault(int(row["stage"]), {"forward": [], "backward": []})[name].append(opt)
    return table, ac


def instruction_order(num_stages: int, num_mbs: int, stage_id: int) -> List[Tuple[str, int]]:
    """Synchronous 1F1B: ``num_stages - stage_id - 1`` warm-up forwards, then one forward and one
    backward in turn, then the remaining backwards (the order of the shipped plans: stage 0 of 2
    with 8 microbatches is F F B F B ... F B B)."""
    if not 0 <= stage_id < num_stages:
        raise ValueError("stage_id out of range")
    warm = min(num_stages - stage_id - 1, num_mbs)
    order = [("forward", m) for m in range(warm)]
    fwd, bwd = warm, 0
    while bwd < num_mbs:
        if fwd < num_mbs:
            order.append(("forward", fwd))
            fwd += 1
        order.append(("backward", bwd))
        bwd += 1
    return order


def _quantise(t: float, unit_time: float) -> int:
    return max(1, int(round(t / unit_time)))


def plan_frontier(forward: Sequence[Option], backward: Sequence[Option], num_mbs: int,
                  unit_time: float = 1e-3, p2p_power: float = 0.0, num_stages: int = 1,
                  stage_id: int = 0) -> List[Plan]:
    """Every plan of one stage that is the cheapest for its time, from the cheapest (iteration 0)
    to the fastest, each strictly faster and strictly dearer than the one before."""
    if num_stages != 1:
        raise NotImplementedError("plans for more than one pipeline stage need the min-cut solver of the "
                                  "reference's optimisation driver; this generator covers one stage")
    if not forward or not backward:
        raise ValueError("the candidate table has no forward or no backward options for this stage")
    if num_mbs <= 0 or unit_time <= 0:
        raise ValueError("num_mbs and unit_time must be positive")
    order = instruction_order(num_stages, num_mbs, stage_id)
    choices = {"forward": list(forward), "backward": list(backward)}
    quant = {k: [_quantise(o.time, unit_time) for o in v] for k, v in choices.items()}
    cost = {k: [o.energy - p2p_power * q * unit_time for o, q in zip(v, quant[k])]
            for k, v in choices.items()}
    total_max = sum(max(quant[name]) for name, _ in order)
    inf = math.inf
    # best[i][t]: cheapest way to run the first i instructions in exactly t units; pick[i][t]: the
    # option of instruction i - 1 on that way
    best = [[inf] * (total_max + 1) for _ in range(len(order) + 1)]
    pick = [[-1] * (total_max + 1) for _ in range(len(order) + 1)]
    best[0][0] = 0.0
    reach = 0
    for i, (name, _mb) in enumerate(order):
        row, nxt, choose = best[i], best[i + 1], pick[i + 1]
        for t in range(reach + 1):
            c0 = row[t]
            if c0 == inf:
                continue
            for j, (q, c) in enumerate(zip(quant[name], cost[name])):
                if c0 + c < nxt[t + q]:
                    nxt[t + q] = c0 + c
                    choose[t + q] = j
        reach += max(quant[name])
    final = best[len(order)]
    # a time stays only if it is cheaper than every shorter one; iteration 0 is the cheapest plan
    plans: List[Plan] = []
    frontier, floor = [], inf
    for tt, c in enumerate(final):
        if c < floor:
            frontier.append((tt, c))
            floor = c
    frontier.reverse()
    for it, (tt, c) in enumerate(frontier):
        assignment = []
        rem = tt
        for i in range(len(order), 0, -1):
            j = pick[i][rem]
            name = order[i - 1][0]
            assignment.append(choices[name][j])
            rem -= quant[name][j]
        assignment.reverse()
        plans.append(Plan(iteration=it, quant_time=tt, time=sum(o.time for o in assignment), cost=c,
                          energy=c + p2p_power * tt * unit_time, instructions=tuple(order),
                          assignment=tuple(assignment)))
    return plans


def write_plan_files(output_dir: str, plans_by_stage: Sequence[Sequence[Plan]],
                     use_activation_checkpointing: bool, num_mbs: int) -> List[Tuple[str, str]]:
    """``freqs_pipeline_<i>.py`` / ``scheds_pipeline_<i>.py`` for every iteration, one inner list
    per stage (run_optimization.py:198-262): with recompute one tuple per instruction in 1F1B order,
    otherwise one ``(forward tuple, backward tuple)`` pair per microbatch.  Returns the paths."""
    os.makedirs(output_dir, exist_ok=True)
    iterations = min(len(p) for p in plans_by_stage)
    written = []
    for it in range(iterations):
        freq_lines, cfg_lines = [], []
        for plans in plans_by_stage:
            plan = plans[it]
            stage_freq, per_inst, by_mb = [], [], {}
            for (name, mb), opt in zip(plan.instructions, plan.assignment):
                stage_freq.append((name, opt.knob[0]))
                tup = (name,) + tuple(opt.knob[1:])
                per_inst.append(tup)
                by_mb.setdefault(mb, {})[name] = tup
            freq_lines.append(f"{stage_freq},\n")
            if use_activation_checkpointing:
                cfg_lines.append(f"{per_inst},\n")
            else:
                pairs = [(by_mb.get(m, {}).get("forward", ("forward", "", "")),
                          by_mb.get(m, {}).get("backward", ("backward", "", ""))) for m in range(num_mbs)]
                cfg_lines.append(f"{pairs},\n")
        first = plans_by_stage[0][it]
        prev = plans_by_stage[0][it - 1] if it else None
        change = sum(p[it].cost for p in plans_by_stage) - (sum(p[it - 1].cost for p in plans_by_stage) if prev else 0.0)
        total = sum(p[it].cost for p in plans_by_stage)
        with_p2p = sum(p[it].energy for p in plans_by_stage)
        tail = (f"# Iteration {it} cost change: {change if prev else 0.0}\n"
                f"# Iteration {it} total cost: {total}\n"
                f"# Iteration {it} total cost with P2P: {with_p2p}\n"
                f"# Iteration {it} time: {first.time}\n")
        paths = []
        for stem, lines in (("freqs", freq_lines), ("scheds", cfg_lines)):
            path = os.path.join(output_dir, f"{stem}_pipeline_{it:05d}.py")
            with open(path, "w") as f:
                f.write("[\n" + "".join(lines) + "]\n" + tail)
            paths.append(path)
        written.append((paths[0], paths[1]))
    return written


def generate_plans(inst_profile: str, output_dir: str, num_mbs: int = 8, num_stages: int = 1,
                   gpu_type: str = "MI355X", unit_time: float = 1e-3,
                   use_activation_checkpointing: Optional[bool] = None) -> List[Plan]:
    """Candidate table -> plan files under ``output_dir``; returns the frontier of stage 0."""
    if gpu_type not in P2P_POWER_W:
        raise ValueError(f"Unknown GPU type {gpu_type!r}. Available: {list(P2P_POWER_W)}")
    table, ac = read_profile_csv(inst_profile, use_activation_checkpointing)
    if sorted(table) != list(range(num_stages)):
        raise ValueError(f"the table has stages {sorted(table)}, the plan wants {num_stages}")
    stages = [plan_frontier(table[s]["forward"], table[s]["backward"], num_mbs, unit_time,
                            P2P_POWER_W[gpu_type], num_stages, s) for s in range(num_stages)]
    write_plan_files(output_dir, stages, ac, num_mbs)
    return stages[0]


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m kareus_amd.profiling.plan_generator")
    ap.add_argument("--inst-profile", required=True, help="candidate table (profile_*.csv)")
    ap.add_argument("--output-dir", required=True)
    ap.add_argument("--num-mbs", type=int, default=8)
    ap.add_argument("--num-stages", type=int, default=1)
    ap.add_argument("--gpu-type", default="MI355X")
    ap.add_argument("--unit-time", type=float, default=1e-3, help="time quantum in seconds")
    ap.add_argument("--no-activation-checkpointing", action="store_true")
    args = ap.parse_args(argv)
    plans = generate_plans(args.inst_profile, args.output_dir, args.num_mbs, args.num_stages, args.gpu_type,
                           args.unit_time, False if args.no_activation_checkpointing else None)
    for p in plans:
        print(f"iteration {p.iteration:5d}: {p.time * 1e3:10.3f} ms  {p.energy:10.3f} J")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
