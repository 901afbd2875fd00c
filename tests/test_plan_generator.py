"""Candidate table -> plan files for one pipeline stage: the dynamic programme against brute
force and closed forms, the written files against the reference's own plan layout (read back by
the schedule / frequency parsers and stepped through by the schedulers)."""

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
    with pytest.raises(NotImplementedError):
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
