"""Candidate table -> plan files: the one-stage dynamic programme and the pipeline's min-cut walk
against brute force and closed forms, the written files against the reference's own plan layout
(read back by the schedule / frequency parsers and stepped through by the schedulers)."""

import itertools
import os
import random

import pytest

from kareus_amd.profiling import plan_generator as pg
from kareus_amd.profiling.profile_csv import P2P_POWER_W
from kareus_amd.scheduler import (CommConfig, PipelineCommScheduler, PipelineFrequencyScheduler,
                                  parse_frequency_file, parse_schedule_file)


def _opt(t, e, freq, *cfgs):
    return pg.Option(t, e, (freq,) + cfgs)


def test_instruction_order_is_synchronous_1f1b(fixtures_dir):
    assert "".join(n[0].upper() for n, _ in pg.instruction_order(2, 8, 0)) == "FFBFBFBFBFBFBFBB"
    assert "".join(n[0].upper() for n, _ in pg.instruction_order(2, 8, 1)) == "FB" * 8
    assert pg.instruction_order(1, 3, 0) == [("forward", 0), ("backward", 0), ("forward", 1), ("backward", 1),
                                             ("forward", 2), ("backward", 2)]
    assert "".join(n[0] for n, _ in pg.instruction_order(4, 2, 0)) == "ffbb"      # fewer microbatches than stages
    # the shipped plans have this order
    for stage_id, stage in enumerate(parse_frequency_file(os.path.join(fixtures_dir, "freqs_pipeline_00324.py"))):
        assert [n for n, _ in stage] == [n for n, _ in pg.instruction_order(2, 8, stage_id)]
    for s in range(3):
        order = pg.instruction_order(3, 5, s)
        for name in ("forward", "backward"):
            assert [m for n, m in order if n == name] == list(range(5))
        for m in range(5):                                   # a microbatch's backward follows its forward
            assert order.index(("backward", m)) > order.index(("forward", m))


def _brute_force(fwd, bwd, num_mbs, unit, p2p):
    """Cheapest cost for every exact quantised time, by enumeration."""
    order = pg.instruction_order(1, num_mbs, 0)
    best = {}
    for combo in itertools.product(*[(fwd if n == "forward" else bwd) for n, _ in order]):
        q = sum(max(1, int(round(o.time / unit))) for o in combo)
        c = sum(o.energy - p2p * max(1, int(round(o.time / unit))) * unit for o in combo)
        if c < best.get(q, float("inf")) - 1e-12:
            best[q] = c
    return best


@pytest.mark.parametrize("seed", range(6))
def test_frontier_is_the_brute_force_optimum(seed):
    rng = random.Random(seed)
    unit = 1e-3
    fwd = [_opt(rng.uniform(2e-3, 9e-3), rng.uniform(1.0, 5.0), 1000 + 100 * i, f"a{i}", f"m{i}") for i in range(3)]
    bwd = [_opt(rng.uniform(4e-3, 15e-3), rng.uniform(2.0, 9.0), 1000 + 100 * i, f"ra{i}", f"rm{i}", f"a{i}", f"m{i}")
           for i in range(4)]
    p2p = rng.choice([0.0, 70.0, 286.0])
    plans = pg.plan_frontier(fwd, bwd, 3, unit, p2p)
    exact = _brute_force(fwd, bwd, 3, unit, p2p)
    assert plans[0].iteration == 0 and plans[0].cost == pytest.approx(min(exact.values()))
    assert plans[-1].quant_time == min(exact)                        # ends at the fastest plan there is
    for a, b in zip(plans, plans[1:]):
        assert b.quant_time < a.quant_time and b.cost > a.cost       # strictly faster, strictly dearer
    for p in plans:
        assert p.cost == pytest.approx(min(c for q, c in exact.items() if q <= p.quant_time))
        # the assignment is what the plan says it costs
        qs = [max(1, int(round(o.time / unit))) for o in p.assignment]
        assert sum(qs) == p.quant_time
        assert sum(o.energy - p2p * q * unit for o, q in zip(p.assignment, qs)) == pytest.approx(p.cost)
        assert p.energy == pytest.approx(sum(o.energy for o in p.assignment))
        assert p.time == pytest.approx(sum(o.time for o in p.assignment))
        for (name, _), o in zip(p.instructions, p.assignment):
            assert o in (fwd if name == "forward" else bwd)
    # every non-dominated exact time is on the frontier
    for q, c in exact.items():
        if all(c2 > c for q2, c2 in exact.items() if q2 < q) and all(c2 >= c for q2, c2 in exact.items() if q2 == q):
            if c <= min(c2 for q2, c2 in exact.items() if q2 <= q) + 1e-12:
                assert any(p.quant_time == q for p in plans)


def test_closed_forms():
    # one option each: one plan, its time and energy are the sums
    plans = pg.plan_frontier([_opt(2e-3, 3.0, 1500, "a", "m")], [_opt(5e-3, 7.0, 1500, "a", "m")], 4, 1e-3, 100.0)
    assert len(plans) == 1 and plans[0].quant_time == 28
    assert plans[0].energy == pytest.approx(40.0) and plans[0].cost == pytest.approx(40.0 - 100.0 * 28e-3)
    # two forward options, slow-cheap and fast-dear, k of n microbatches switched: n + 1 plans,
    # the i-th has i fast forwards
    slow, fast = _opt(6e-3, 1.0, 900, "s", "s"), _opt(4e-3, 2.0, 1400, "f", "f")
    plans = pg.plan_frontier([slow, fast], [_opt(5e-3, 7.0, 1400, "b", "b")], 5, 1e-3, 0.0)
    assert [p.quant_time for p in plans] == [55 - 2 * i for i in range(6)]
    for i, p in enumerate(plans):
        assert sum(o is fast for o in p.assignment) == i
        assert p.energy == pytest.approx(5 * 7.0 + 5 * 1.0 + i)
    # a dominated option (slower and dearer) is never chosen
    plans = pg.plan_frontier([slow, fast, _opt(7e-3, 2.5, 800, "x", "x")], [_opt(5e-3, 7.0, 1400, "b", "b")], 2, 1e-3, 0.0)
    assert all(o.knob[0] != 800 for p in plans for o in p.assignment)
    # the power a GPU draws anyway is taken out for an option's own time (a stage that is not on
    # the critical path would wait at that power instead): at 0 W the option that is slower and
    # 0.5 J dearer is dominated, at 300 W its 2 ms more are worth 0.6 J and it opens the frontier
    a, b = _opt(6e-3, 2.0, 900, "s", "s"), _opt(4e-3, 1.5, 1400, "f", "f")
    back = _opt(5e-3, 7.0, 1400, "b", "b")
    plans = pg.plan_frontier([a, b], [back], 1, 1e-3, 0.0)
    assert len(plans) == 1 and plans[0].assignment[0] is b
    plans = pg.plan_frontier([a, b], [back], 1, 1e-3, 300.0)
    assert [p.assignment[0] for p in plans] == [a, b]
    assert plans[0].cost == pytest.approx(2.0 - 1.8 + 7.0 - 1.5) and plans[0].energy == pytest.approx(9.0)
    with pytest.raises(ValueError, match="pipeline_frontier"):
        pg.plan_frontier([a], [b], 2, num_stages=2)
    with pytest.raises(ValueError):
        pg.plan_frontier([], [b], 2)


def _write_table(path, ac=True):
    with open(path, "w") as f:
        if ac:
            f.write("stage,instruction,frequency,recompute_attention_configs,recompute_mlp_configs,"
                    "attention_configs,mlp_configs,time,energy\n")
            f.write("0,forward,2400,,,norm_0-none-12-1024,norm_0-none-18-1024,0.0021,2.9\n")
            f.write("0,forward,1800,,,rope_0-none-8-1024,linear_1-none-16-1024,0.0026,2.5\n")
            f.write("0,backward,2400,attn_0-none-21-1024,norm_0-none-15-1024,rope_0-none-30-1024,activation_0-none-15-1024,0.0052,7.0\n")
            f.write("0,backward,1800,norm_0-none-27-1024,norm_0-none-27-1024,rope_0-none-21-1024,activation_0-none-15-1024,0.0063,6.2\n")
        else:
            f.write("stage,instruction,frequency,attention_configs,mlp_configs,time,energy\n")
            f.write("0,forward,2400,norm_0-none-12-1024,norm_0-none-18-1024,0.0021,2.9\n")
            f.write("0,forward,1800,rope_0-none-8-1024,linear_1-none-16-1024,0.0026,2.5\n")
            f.write("0,backward,2400,rope_0-none-30-1024,activation_0-none-15-1024,0.0032,4.0\n")
            f.write("0,backward,1800,rope_0-none-21-1024,activation_0-none-15-1024,0.0040,3.5\n")


def test_written_plans_are_read_like_shipped_ones(tmp_path, fixtures_dir):
    table = str(tmp_path / "profile.csv")
    _write_table(table, ac=True)
    out = str(tmp_path / "plans")
    plans = pg.generate_plans(table, out, num_mbs=4, unit_time=1e-4, gpu_type="MI355X")
    assert len(plans) >= 3 and plans[0].iteration == 0
    names = sorted(os.listdir(out))
    assert names == sorted([f"freqs_pipeline_{i:05d}.py" for i in range(len(plans))] +
                           [f"scheds_pipeline_{i:05d}.py" for i in range(len(plans))])
    for p in plans:
        freqs = parse_frequency_file(os.path.join(out, f"freqs_pipeline_{p.iteration:05d}.py"))
        scheds = parse_schedule_file(os.path.join(out, f"scheds_pipeline_{p.iteration:05d}.py"), True, False)
        assert len(freqs) == len(scheds) == 1 and len(freqs[0]) == len(scheds[0]) == 8
        assert freqs[0] == [(n, o.knob[0]) for (n, _), o in zip(p.instructions, p.assignment)]
        for item, (name, _), o in zip(scheds[0], p.instructions, p.assignment):
            if name == "forward":
                assert item.bwd_attn is None and item.bwd_mlp is None
                assert item.fwd_attn == _cfg(o.knob[1]) and item.fwd_mlp == _cfg(o.knob[2])
            else:   # recompute pair lands in fwd_*, as in a shipped plan
                assert (item.fwd_attn, item.fwd_mlp, item.bwd_attn, item.bwd_mlp) == tuple(_cfg(c) for c in o.knob[1:])
    # same text layout as a shipped plan: a list literal, one line per stage, comment lines after
    text = open(os.path.join(out, "scheds_pipeline_00000.py")).read().splitlines()
    shipped = open(os.path.join(fixtures_dir, "scheds_pipeline_00324.py")).read().splitlines()
    assert text[0] == shipped[0] == "[" and text[2] == "]" and shipped[3] == "]"
    assert text[1].startswith("[('forward', '") and text[1].endswith("],") and shipped[1].endswith("],")
    assert text[3].startswith("# Iteration 0 cost change:") and text[5].startswith("# Iteration 0 total cost with P2P:")
    # the fastest plan is all-2400 MHz, the cheapest (idle power taken out) is not all-fast
    last = parse_frequency_file(os.path.join(out, f"freqs_pipeline_{plans[-1].iteration:05d}.py"))[0]
    assert all(mhz == 2400 for _, mhz in last)
    assert plans[-1].time == pytest.approx(4 * (0.0021 + 0.0052))
    # the schedulers step through a written plan like through a shipped one
    path_s = os.path.join(out, "scheds_pipeline_00001.py")
    path_f = os.path.join(out, "freqs_pipeline_00001.py")
    sch = PipelineCommScheduler(path_s, pp_rank=0, num_microbatches=4, use_activation_checkpointing=True)
    clocks = []
    fsch = PipelineFrequencyScheduler(path_f, pp_rank=0, num_instructions=8,
                                      set_frequency=lambda mhz: (clocks.append(mhz), True)[1], reset_frequency=lambda: True)
    sch.on_step_begin(); fsch.on_step_begin()
    for (name, _), o in zip(plans[1].instructions, plans[1].assignment):
        sch.on_instruction_begin(name); fsch.on_instruction_begin(name)
        cur = sch.current_schedule
        assert (cur.bwd_mlp if name == "backward" else cur.fwd_mlp) == _cfg(o.knob[-1])
        assert fsch.current_frequency == o.knob[0]
        sch.on_instruction_end(name); fsch.on_instruction_end(name)
    sch.on_step_end(); fsch.on_step_end()
    assert set(clocks) <= {1800, 2400}


def _cfg(text):
    from kareus_amd.scheduler.parser import _parse_config_string
    return _parse_config_string(text)


def test_per_microbatch_pairs_without_recompute(tmp_path):
    table = str(tmp_path / "profile.csv")
    _write_table(table, ac=False)
    out = str(tmp_path / "plans")
    plans = pg.generate_plans(table, out, num_mbs=3, unit_time=1e-4, gpu_type="A100")
    for p in plans:
        stages = parse_schedule_file(os.path.join(out, f"scheds_pipeline_{p.iteration:05d}.py"), False, False)
        assert len(stages) == 1 and len(stages[0]) == 3          # one (forward, backward) pair per microbatch
        chosen = {(n, m): o for (n, m), o in zip(p.instructions, p.assignment)}
        for m, item in enumerate(stages[0]):                     # a pair reads as one item with both halves
            assert item.fwd_attn == _cfg(chosen[("forward", m)].knob[1])
            assert item.fwd_mlp == _cfg(chosen[("forward", m)].knob[2])
            assert item.bwd_attn == _cfg(chosen[("backward", m)].knob[1])
            assert item.bwd_mlp == _cfg(chosen[("backward", m)].knob[2])


def test_table_errors(tmp_path):
    path = str(tmp_path / "t.csv")
    open(path, "w").write("stage,instruction,frequency,fwd_qkv_ar,time,energy\n")
    with pytest.raises(ValueError, match="context-parallel"):
        pg.read_profile_csv(path)
    open(path, "w").write("stage,instruction,frequency,attention_configs,time,energy\n")
    with pytest.raises(ValueError, match="mlp_configs"):
        pg.read_profile_csv(path)
    _write_table(path, ac=False)
    with pytest.raises(ValueError, match="recompute"):
        pg.read_profile_csv(path, use_activation_checkpointing=True)
    with pytest.raises(ValueError, match="Unknown GPU type"):
        pg.generate_plans(path, str(tmp_path / "o"), gpu_type="H100")
    with pytest.raises(ValueError, match="stages"):
        pg.generate_plans(path, str(tmp_path / "o"), num_stages=2)
    assert "MI355X" in P2P_POWER_W


def test_profile_csv_round_trip(tmp_path):
    """What the table writer emits, the plan generator reads: eval logs -> CSV -> plans."""
    import json
    from kareus_amd.profiling.profile_csv import generate_profile_csv

    logs = tmp_path / "logs"
    logs.mkdir()
    rng = random.Random(3)
    for key, base in (("fwd_attn", 0.5e-3), ("fwd_mlp", 0.8e-3), ("bwd_attn", 1.0e-3), ("bwd_mlp", 1.6e-3)):
        with open(logs / f"{key}.jsonl", "w") as f:
            for freq in (1800, 2400):
                for start in ("norm_0", "linear_0"):
                    t = base * (2400 / freq) * rng.uniform(0.95, 1.05)
                    f.write(json.dumps({"freq": freq, "overlap_start": start, "overlap_end": "none", "sm": 16,
                                        "block": 1024, "time_s": t, "energy_j": t * (500 + 0.3 * freq)}) + "\n")
    csv_path = str(tmp_path / "profile.csv")
    kept = generate_profile_csv(str(logs), csv_path, num_layers=2, nanobatches=2, gpu_type="MI355X")
    assert kept["forward"] >= 1 and kept["backward"] >= 1
    table, ac = pg.read_profile_csv(csv_path)
    assert ac and len(table[0]["forward"]) == kept["forward"] and len(table[0]["backward"]) == kept["backward"]
    plans = pg.generate_plans(csv_path, str(tmp_path / "plans"), num_mbs=2, unit_time=1e-5)
    assert plans and all(len(p.assignment) == 4 for p in plans)


# ------------------------------------------------------------------------------------------------
# several stages: the 1F1B dependency graph and the walk by minimum cuts
# ------------------------------------------------------------------------------------------------

def test_pipeline_dependencies():
    ops, deps = pg.pipeline_dependencies(2, 3)
    assert len(ops) == 12 and [o[0] for o in ops] == [0] * 6 + [1] * 6
    at = {op: i for i, op in enumerate(ops)}
    dep = set(deps)
    # inside a stage: its 1F1B order; across stages: forwards flow down, backwards flow up
    assert len(dep) == 2 * 5 + 2 * 3
    for s in range(2):
        order = pg.instruction_order(2, 3, s)
        for (n0, m0), (n1, m1) in zip(order, order[1:]):
            assert (at[(s, n0, m0)], at[(s, n1, m1)]) in dep
    for m in range(3):
        assert (at[(0, "forward", m)], at[(1, "forward", m)]) in dep
        assert (at[(1, "backward", m)], at[(0, "backward", m)]) in dep
    # one stage is a chain
    ops1, deps1 = pg.pipeline_dependencies(1, 4)
    assert deps1 == [(i, i + 1) for i in range(7)]
    # closed form of the longest path with every forward f and every backward b long (f <= b):
    # (S - 1) f to fill the pipe, M (f + b) on the last stage, (S - 1) b to drain it
    for S, M, f, b in [(2, 8, 3, 5), (4, 6, 2, 7), (3, 3, 4, 4)]:
        ops, deps = pg.pipeline_dependencies(S, M)
        dur = [f if name == "forward" else b for _s, name, _m in ops]
        assert pg._event_times(len(ops), deps, dur)[2] == (S - 1) * f + M * (f + b) + (S - 1) * b


def test_max_flow_known_answers():
    # the textbook six-node network with maximum flow 23
    net = pg._FlowNetwork(6)
    for u, v, c in [(0, 1, 16), (0, 2, 13), (1, 2, 10), (2, 1, 4), (1, 3, 12), (3, 2, 9), (2, 4, 14), (4, 3, 7),
                    (3, 5, 20), (4, 5, 4)]:
        net.add_edge(u, v, c)
    assert net.max_flow(0, 5) == 23
    side = net.reachable(0)
    assert side[0] and not side[5]
    # two disjoint paths and a bottleneck
    net = pg._FlowNetwork(4)
    net.add_edge(0, 1, 5); net.add_edge(1, 3, 3); net.add_edge(0, 2, 2); net.add_edge(2, 3, 9)
    assert net.max_flow(0, 3) == 5
    assert pg._FlowNetwork(2).max_flow(0, 1) == 0


def test_cost_curve_is_the_lower_convex_hull():
    unit = 1e-3
    opts = [_opt(2e-3, 10.0, 2400, "a", "m"), _opt(4e-3, 4.0, 1800, "a", "m"), _opt(3e-3, 9.0, 2100, "a", "m"),
            _opt(6e-3, 3.0, 1200, "a", "m"), _opt(5e-3, 5.0, 1500, "a", "m"),      # dominated: slower and dearer
            _opt(7e-3, 3.0, 900, "a", "m")]                                         # slower, not cheaper
    c = pg._cost_curve(opts, unit, 0.0)
    assert (c.dmin, c.dmax) == (2, 6)
    assert [q for q, _c, _o in c.pareto] == [2, 3, 4, 6]
    # (3, 9.0) lies above the chord from (2, 10) to (4, 4): the hull skips it
    assert c.marginal == {3: 3_000_000, 4: 3_000_000, 5: 500_000, 6: 500_000}
    # a planned duration gets the cheapest measured option that is fast enough
    assert [c.option_for(d)[2].knob[0] for d in range(2, 8)] == [2400, 2100, 1800, 1800, 1200, 1200]
    # idle power comes out of an option's cost for its own quantised time
    c2 = pg._cost_curve(opts[:2], unit, 1000.0)
    assert [round(cost, 9) for _q, cost, _o in c2.pareto] == [8.0, 0.0]


def _model_cost(curve, d):
    return sum(curve.marginal[x] for x in range(d + 1, curve.dmax + 1))


@pytest.mark.parametrize("stages,mbs,seed", [(2, 2, 0), (2, 2, 1), (2, 2, 2), (3, 1, 3), (3, 1, 4), (1, 3, 5)])
def test_pipeline_walk_is_the_enumerated_optimum(stages, mbs, seed):
    """Every step of the walk lands on the cheapest assignment of integer durations whose longest
    path is that short (costs on the options' convex hull), found by trying them all."""
    rng = random.Random(seed)
    unit = 1e-3
    table = {s: {name: [_opt(rng.randint(2, 5) * unit, rng.uniform(1.0, 6.0), 1000 + i, "a", "m") for i in range(3)]
                 for name in ("forward", "backward")} for s in range(stages)}
    ops, deps = pg.pipeline_dependencies(stages, mbs)
    curves = [pg._cost_curve(table[s][name], unit, 0.0) for s, name, _m in ops]
    best = {}
    for combo in itertools.product(*[range(c.dmin, c.dmax + 1) for c in curves]):
        total = pg._event_times(len(ops), deps, combo)[2]
        cost = sum(_model_cost(c, d) for c, d in zip(curves, combo))
        best[total] = min(cost, best.get(total, cost))
    dur = [c.dmax for c in curves]
    total = pg._event_times(len(ops), deps, dur)[2]
    assert total == max(best) and best[total] == 0
    spent = 0
    while True:
        change = pg._shorten_by_one(len(ops), deps, dur, curves)
        if change is None:
            break
        spent += change
        total -= 1
        assert pg._event_times(len(ops), deps, dur)[2] == total
        assert all(c.dmin <= d <= c.dmax for c, d in zip(curves, dur))
        assert sum(_model_cost(c, d) for c, d in zip(curves, dur)) == spent
        assert spent == min(c for t, c in best.items() if t <= total)
    assert total == min(best)                                # it stops at the fastest plan there is


def test_pipeline_walk_closed_form():
    # two stages, one microbatch: F0 -> F1 -> B1 -> B0 is a chain of four, so the walk buys the
    # cheapest unit of time first: marginal costs 1 (stage-1 forward), 2, 3, 4 J per unit, one unit each
    def two(t_slow, e_fast_extra):
        return [_opt(t_slow * 1e-3, 5.0, 900, "s", "s"), _opt((t_slow - 1) * 1e-3, 5.0 + e_fast_extra, 1400, "f", "f")]
    table = {0: {"forward": two(4, 2.0), "backward": two(8, 4.0)},
             1: {"forward": two(5, 1.0), "backward": two(9, 3.0)}}
    stages = pg.pipeline_frontier(table, 2, 1, 1e-3, 0.0)
    assert [p.quant_time for p in stages[0]] == [26, 25, 24, 23, 22]
    total = [stages[0][i].cost + stages[1][i].cost for i in range(5)]
    assert total == pytest.approx([20.0, 21.0, 23.0, 26.0, 30.0])
    fast = [[o.knob[0] == 1400 for o in stages[s][i].assignment] for i in range(5) for s in range(2)]
    assert fast[2:4] == [[False, False], [True, False]]      # iteration 1: only stage 1's forward
    assert fast[8:10] == [[True, True], [True, True]]
    # an instruction off the critical path is never sped up: stage 0 has slack while stage 1 works
    table = {0: {"forward": two(4, 2.0), "backward": two(4, 2.0)},
             1: {"forward": two(9, 1.0), "backward": two(9, 1.0)}}
    stages = pg.pipeline_frontier(table, 2, 2, 1e-3, 0.0)
    # critical path: F0(0) F1(0) B1(0) F1(1) B1(1) B0(1); stage 0's F(1) and B(0) wait
    last = stages[0][-1]
    chosen = {(n, m): o.knob[0] for (n, m), o in zip(last.instructions, last.assignment)}
    assert chosen[("forward", 0)] == 1400 and chosen[("backward", 1)] == 1400
    assert chosen[("forward", 1)] == 900 and chosen[("backward", 0)] == 900
    assert all(o.knob[0] == 1400 for o in stages[1][-1].assignment)
    assert stages[0][-1].quant_time == 3 + 4 * 8 + 3


def _write_pipeline_table(path):
    with open(path, "w") as f:
        f.write("stage,instruction,frequency,recompute_attention_configs,recompute_mlp_configs,"
                "attention_configs,mlp_configs,time,energy\n")
        for stage, scale in ((0, 1.0), (1, 1.1)):
            for mhz, t, e in ((2400, 0.0021, 2.9), (2100, 0.0023, 2.6), (1800, 0.0026, 2.5)):
                f.write(f"{stage},forward,{mhz},,,norm_0-none-12-1024,norm_0-none-18-1024,{t * scale},{e * scale}\n")
            for mhz, t, e in ((2400, 0.0052, 7.0), (2100, 0.0057, 6.5), (1800, 0.0063, 6.2)):
                f.write(f"{stage},backward,{mhz},attn_0-none-21-1024,norm_0-none-15-1024,rope_0-none-30-1024,"
                        f"activation_0-none-15-1024,{t * scale},{e * scale}\n")


def test_pipeline_plans_are_read_like_shipped_ones(tmp_path, fixtures_dir):
    table = str(tmp_path / "profile.csv")
    _write_pipeline_table(table)
    out = str(tmp_path / "plans")
    unit = 1e-4
    first = pg.generate_plans(table, out, num_mbs=8, num_stages=2, unit_time=unit, gpu_type="MI355X")
    n = len(first)
    assert n > 10 and [p.quant_time for p in first] == [first[0].quant_time - i for i in range(n)]
    assert sorted(os.listdir(out)) == sorted([f"{stem}_pipeline_{i:05d}.py" for i in range(n) for stem in ("freqs", "scheds")])
    shipped = parse_frequency_file(os.path.join(fixtures_dir, "freqs_pipeline_00324.py"))
    options, _ac = pg.read_profile_csv(table)
    ops, deps = pg.pipeline_dependencies(2, 8)
    for i in (0, 1, n // 2, n - 1):
        freqs = parse_frequency_file(os.path.join(out, f"freqs_pipeline_{i:05d}.py"))
        scheds = parse_schedule_file(os.path.join(out, f"scheds_pipeline_{i:05d}.py"), True, False)
        assert len(freqs) == len(scheds) == 2
        for s in range(2):                                   # the instruction order of a shipped two-stage plan
            assert [name for name, _ in freqs[s]] == [name for name, _ in shipped[s]]
            assert len(scheds[s]) == 16
        # the clocks written are options of the table, and running them meets the plan's time
        dur = []
        for (s, name, _m), (_n, mhz) in zip(ops, freqs[0] + freqs[1]):
            opt = next(o for o in options[s][name] if o.knob[0] == mhz)
            dur.append(max(1, int(round(opt.time / unit))))
        assert pg._event_times(len(ops), deps, dur)[2] <= first[i].quant_time
    last = parse_frequency_file(os.path.join(out, f"freqs_pipeline_{n - 1:05d}.py"))
    # the fastest plan runs the slower stage flat out; the cheapest plan runs nothing at the top clock
    assert all(mhz == 2400 for _n, mhz in last[1])
    cheapest = parse_frequency_file(os.path.join(out, "freqs_pipeline_00000.py"))
    assert all(mhz != 2400 for stage in cheapest for _n, mhz in stage)
    text = open(os.path.join(out, f"scheds_pipeline_{n - 1:05d}.py")).read().splitlines()
    assert text[0] == "[" and text[3] == "]" and text[4].startswith(f"# Iteration {n - 1} cost change:")
    # both ranks step through a written plan
    for rank in range(2):
        sch = PipelineCommScheduler(os.path.join(out, "scheds_pipeline_00003.py"), pp_rank=rank, num_microbatches=8,
                                    use_activation_checkpointing=True)
        sch.on_step_begin()
        for name, _m in pg.instruction_order(2, 8, rank):
            sch.on_instruction_begin(name)
            assert sch.current_schedule is not None
            sch.on_instruction_end(name)
        sch.on_step_end()
