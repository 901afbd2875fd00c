"""Per-stage candidate table (``profile_*.csv``) -> the plan files the schedulers step through.

The reference hands its candidate table to a driver (tests/kareus/run_optimization.py) around the
third-party ``lowtime`` package (not part of the reference tree, no version pinned there): it
builds one ``ExecutionOption`` per CSV row (:79-115), lays the instructions of every stage out in
synchronous 1F1B order (:381-402), lets the solver walk from the cheapest plan towards the fastest
one unit of time per iteration (:455-477) and writes, for every iteration,
``freqs_pipeline_<iteration>.py`` and ``scheds_pipeline_<iteration>.py`` (:198-262) followed by
three comment lines with the iteration's cost.

**One pipeline stage** (what one GPU runs): the dependency graph is a chain, the iteration time is
the sum of the instructions' times, and the cheapest plan for a time budget is a multiple-choice
knapsack, which a dynamic programme over the quantised time solves exactly (no curve fitting, no
min-cut).

**Several stages**: the instructions of all stages form the 1F1B dependency graph (a stage runs its
instructions in order; a microbatch's forward needs the previous stage's, its backward the next
stage's) and the iteration time is that graph's longest path.  ``pipeline_frontier`` walks it the way
the published algorithm behind the solver does (Phillips & Dessouky 1977, time-cost trade-off by
minimum cuts): every instruction starts at its cheapest duration, and each iteration finds, on the
sub-graph of critical instructions, the cheapest set of instructions to shorten by one unit (and
of instructions that may be lengthened again) so that every critical path loses one unit — a
minimum cut with lower bounds, here an integer Dinic max-flow.  An instruction's cost between two
measured options is the straight line between them (the lower convex hull of the options), where
the reference's driver fits an exponential to them; on the hull the walk is exact, which the tests
check by enumeration.  An instruction planned for ``d`` units is given the cheapest measured option
that is no slower than ``d``.

Times are quantised to ``unit_time`` and the power a GPU draws anyway (``p2p_power``) is taken out
of every option's energy for the length of its quantised time, as the driver does (:374-375); the
figure reported as "total cost with P2P" adds it back for the whole iteration on every stage (:467).

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

__all__ = ["Option", "Plan", "read_profile_csv", "instruction_order", "plan_frontier", "pipeline_frontier",
           "pipeline_dependencies", "write_plan_files", "generate_plans"]

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
        raise ValueError("plan_frontier plans one stage on its own; use pipeline_frontier for a pipeline")
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


_INF = 1 << 60
_COST_SCALE = 1e6   # costs enter the max-flow as integers of this many units per joule


class _FlowNetwork:
    """Integer max-flow (Dinic).  Edge ``e`` and its reverse ``e ^ 1`` sit next to each other."""

    def __init__(self, n: int):
        self.head: List[List[int]] = [[] for _ in range(n)]
        self.to: List[int] = []
        self.cap: List[int] = []

    def add_edge(self, u: int, v: int, cap: int) -> int:
        e = len(self.to)
        self.head[u].append(e)
        self.to.append(v)
        self.cap.append(cap)
        self.head[v].append(e + 1)
        self.to.append(u)
        self.cap.append(0)
        return e

    def _levels(self, s: int, t: int) -> Optional[List[int]]:
        level = [-1] * len(self.head)
        level[s] = 0
        queue = [s]
        for u in queue:
            for e in self.head[u]:
                v = self.to[e]
                if self.cap[e] > 0 and level[v] < 0:
                    level[v] = level[u] + 1
                    queue.append(v)
        return level if level[t] >= 0 else None

    def max_flow(self, s: int, t: int) -> int:
        total = 0
        while True:
            level = self._levels(s, t)
            if level is None:
                return total
            nxt = [0] * len(self.head)
            while True:  # one augmenting path of the level graph at a time, found without recursion
                path: List[int] = []
                u = s
                while u != t:
                    advanced = False
                    while nxt[u] < len(self.head[u]):
                        e = self.head[u][nxt[u]]
                        v = self.to[e]
                        if self.cap[e] > 0 and level[v] == level[u] + 1:
                            path.append(e)
                            u = v
                            advanced = True
                            break
                        nxt[u] += 1
                    if not advanced:
                        if not path:
                            break
                        e = path.pop()        # dead end: never try this edge again in this phase
                        u = self.to[e ^ 1]
                        nxt[u] += 1
                if u != t:
                    break
                push = min(self.cap[e] for e in path)
                for e in path:
                    self.cap[e] -= push
                    self.cap[e ^ 1] += push
                total += push

    def reachable(self, s: int) -> List[bool]:
        seen = [False] * len(self.head)
        seen[s] = True
        stack = [s]
        while stack:
            u = stack.pop()
            for e in self.head[u]:
                v = self.to[e]
                if self.cap[e] > 0 and not seen[v]:
                    seen[v] = True
                    stack.append(v)
        return seen


@dataclass(frozen=True)
class _Curve:
    """Cost of one kind of instruction as a function of its planned duration, in time units."""
    dmin: int
    dmax: int
    marginal: Dict[int, int]              # marginal[d]: integer cost of going from d to d - 1 units
    pareto: Tuple[Tuple[int, float, Option], ...]   # (quantised time, cost, option), faster first

    def option_for(self, d: int) -> Tuple[int, float, Option]:
        """The cheapest measured option that is no slower than ``d`` units."""
        best = self.pareto[0]
        for entry in self.pareto:
            if entry[0] <= d:
                best = entry
        return best


def _cost_curve(options: Sequence[Option], unit_time: float, p2p_power: float) -> _Curve:
    pts = sorted(((_quantise(o.time, unit_time), o.energy - p2p_power * _quantise(o.time, unit_time) * unit_time, i)
                  for i, o in enumerate(options)), key=lambda p: (p[0], p[1]))
    pareto: List[Tuple[int, float, Option]] = []
    for q, c, i in pts:                    # slower options stay only if they are strictly cheaper
        if not pareto or (q > pareto[-1][0] and c < pareto[-1][1]):
            pareto.append((q, c, options[i]))
    hull: List[Tuple[int, float]] = []
    for q, c, _ in pareto:                 # lower convex hull, left to right
        while len(hull) >= 2 and ((hull[-1][1] - hull[-2][1]) * (q - hull[-2][0])
                                  >= (c - hull[-2][1]) * (hull[-1][0] - hull[-2][0])):
            hull.pop()
        hull.append((q, c))
    marginal: Dict[int, int] = {}
    for (q0, c0), (q1, c1) in zip(hull, hull[1:]):
        step = max(0, int(round((c0 - c1) / (q1 - q0) * _COST_SCALE)))
        for d in range(q0 + 1, q1 + 1):
            marginal[d] = step
    return _Curve(dmin=hull[0][0], dmax=hull[-1][0], marginal=marginal, pareto=tuple(pareto))


def pipeline_dependencies(num_stages: int, num_mbs: int
                          ) -> Tuple[List[Tuple[int, str, int]], List[Tuple[int, int]]]:
    """The instructions of a synchronous 1F1B iteration as ``(stage, name, microbatch)`` — stage by
    stage, each in its own order — and the pairs ``(i, j)`` with j waiting for i: the next
    instruction of the same stage, the same microbatch's forward on the next stage, the same
    microbatch's backward on the previous stage."""
    ops: List[Tuple[int, str, int]] = []
    index: Dict[Tuple[int, str, int], int] = {}
    deps: List[Tuple[int, int]] = []
    for s in range(num_stages):
        prev = None
        for name, mb in instruction_order(num_stages, num_mbs, s):
            index[(s, name, mb)] = len(ops)
            if prev is not None:
                deps.append((prev, len(ops)))
            prev = len(ops)
            ops.append((s, name, mb))
    for s in range(num_stages - 1):
        for mb in range(num_mbs):
            deps.append((index[(s, "forward", mb)], index[(s + 1, "forward", mb)]))
            deps.append((index[(s + 1, "backward", mb)], index[(s, "backward", mb)]))
    return ops, deps


def _event_times(n: int, deps: Sequence[Tuple[int, int]], dur: Sequence) -> Tuple[list, list, float]:
    """Earliest start and latest start of every instruction and the length of the longest path
    (a pass in topological order and one back)."""
    succ: List[List[int]] = [[] for _ in range(n)]
    indeg = [0] * n
    for i, j in deps:
        succ[i].append(j)
        indeg[j] += 1
    order = [i for i in range(n) if indeg[i] == 0]
    for u in order:
        for v in succ[u]:
            indeg[v] -= 1
            if indeg[v] == 0:
                order.append(v)
    if len(order) != n:
        raise ValueError("the dependency graph has a cycle")
    early = [0] * n
    for u in order:
        for v in succ[u]:
            early[v] = max(early[v], early[u] + dur[u])
    total = max(early[i] + dur[i] for i in range(n))
    late = [total - dur[i] for i in range(n)]
    for u in reversed(order):
        for v in succ[u]:
            late[u] = min(late[u], late[v] - dur[u])
    return early, late, total


def _shorten_by_one(n: int, deps: Sequence[Tuple[int, int]], dur: List[int], curves: Sequence[_Curve]
                    ) -> Optional[int]:
    """One step of the walk: change ``dur`` so that the longest path loses one unit at the least
    cost, and return that cost (in integer units); ``None`` when no critical path can be shortened."""
    early, late, _total = _event_times(n, deps, dur)
    critical = [early[i] == late[i] for i in range(n)]
    # activity-on-arc: instruction i is the arc 2i+2 -> 2i+3; node 0 is the source, node 1 the sink
    lower_upper: List[Tuple[int, int, int, int, int]] = []   # (u, v, lb, ub, instruction or -1)
    has_pred, has_succ = [False] * n, [False] * n
    for i, j in deps:
        if critical[i] and critical[j] and early[i] + dur[i] == early[j]:
            lower_upper.append((2 * i + 3, 2 * j + 2, 0, _INF, -1))
            has_succ[i] = True
            has_pred[j] = True
    for i in range(n):
        if not critical[i]:
            continue
        c, d = curves[i], dur[i]
        ub = c.marginal[d] if d > c.dmin else _INF
        lb = c.marginal[d + 1] if d < c.dmax else 0
        lower_upper.append((2 * i + 2, 2 * i + 3, min(lb, ub), ub, i))
        if not has_pred[i]:
            lower_upper.append((0, 2 * i + 2, 0, _INF, -1))
        if not has_succ[i]:
            lower_upper.append((2 * i + 3, 1, 0, _INF, -1))
    nodes = 2 * n + 4
    ss, tt = nodes - 2, nodes - 1
    net = _FlowNetwork(nodes)
    excess = [0] * nodes
    edge_of: List[int] = []
    for u, v, lb, ub, _i in lower_upper:
        edge_of.append(net.add_edge(u, v, ub - lb if ub < _INF else _INF))
        excess[v] += lb
        excess[u] -= lb
    back = net.add_edge(1, 0, _INF)
    need = 0
    for v in range(nodes - 2):
        if excess[v] > 0:
            net.add_edge(ss, v, excess[v])
            need += excess[v]
        elif excess[v] < 0:
            net.add_edge(v, tt, -excess[v])
    if net.max_flow(ss, tt) != need:
        raise RuntimeError("no flow meets the lower bounds of the critical graph")
    flow = net.cap[back ^ 1]               # what already runs from the source to the sink
    net.cap[back] = net.cap[back ^ 1] = 0
    flow += net.max_flow(0, 1)
    if flow >= _INF // 2:
        return None
    side = net.reachable(0)
    for (u, v, lb, _ub, i) in lower_upper:
        if i < 0:
            continue
        if side[u] and not side[v]:
            dur[i] -= 1
        elif side[v] and not side[u] and lb > 0:
            dur[i] += 1
    return flow


def pipeline_frontier(table: Dict[int, Dict[str, List[Option]]], num_stages: int, num_mbs: int,
                      unit_time: float = 1e-3, p2p_power: float = 0.0,
                      max_iterations: Optional[int] = None) -> List[List[Plan]]:
    """Plans of a whole pipeline, cheapest first, each one time unit shorter than the one before:
    ``result[stage][iteration]``.  A plan's ``quant_time`` is the iteration time of the pipeline
    (the same for every stage), ``cost`` / ``energy`` are the stage's own."""
    if num_stages < 1 or num_mbs <= 0 or unit_time <= 0:
        raise ValueError("num_stages, num_mbs and unit_time must be positive")
    for s in range(num_stages):
        if s not in table or not table[s]["forward"] or not table[s]["backward"]:
            raise ValueError(f"the candidate table has no forward or no backward options for stage {s}")
    ops, deps = pipeline_dependencies(num_stages, num_mbs)
    kind = {(s, name): _cost_curve(table[s][name], unit_time, p2p_power)
            for s in range(num_stages) for name in ("forward", "backward")}
    curves = [kind[(s, name)] for s, name, _mb in ops]
    dur = [c.dmax for c in curves]
    result: List[List[Plan]] = [[] for _ in range(num_stages)]
    iteration = 0
    while True:
        chosen = [c.option_for(d) for c, d in zip(curves, dur)]
        _e, _l, planned = _event_times(len(ops), deps, dur)
        _e, _l, real = _event_times(len(ops), deps, [entry[2].time for entry in chosen])
        for s in range(num_stages):
            mine = [k for k, op in enumerate(ops) if op[0] == s]
            cost = sum(chosen[k][1] for k in mine)
            result[s].append(Plan(iteration=iteration, quant_time=int(planned), time=real, cost=cost,
                                  energy=cost + p2p_power * planned * unit_time,
                                  instructions=tuple((ops[k][1], ops[k][2]) for k in mine),
                                  assignment=tuple(chosen[k][2] for k in mine)))
        iteration += 1
        if max_iterations is not None and iteration >= max_iterations:
            break
        if _shorten_by_one(len(ops), deps, dur, curves) is None:
            break
    return result



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
    if num_stages == 1:
        stages = [plan_frontier(table[0]["forward"], table[0]["backward"], num_mbs, unit_time,
                                P2P_POWER_W[gpu_type])]
    else:
        stages = pipeline_frontier(table, num_stages, num_mbs, unit_time, P2P_POWER_W[gpu_type])
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
