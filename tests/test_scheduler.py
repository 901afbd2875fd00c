"""Schedule / frequency file parsing and the per-instruction scheduler state machine, against
the plans the reference ships (tests/golden/*.py, copied data files) and its error behaviour."""

import os

import pytest

from kareus_amd.scheduler import (CommConfig, PipelineCommScheduler, ScheduleItem, ScheduleItemCP,
                                  parse_frequency_file, parse_schedule_file)
from kareus_amd.scheduler.parser import _TRAIL_CONFIG, _parse_config_string


def test_config_string_formats():
    # the four documented forms (kareus/scheduler/parser.py:69-72)
    assert _parse_config_string("0-8-16-1024") == CommConfig((0, 8), (16, 1024))
    assert _parse_config_string("-1--1-16-1024") == CommConfig((-1, -1), (16, 1024))
    assert _parse_config_string("norm_0-linear_1-16-1024") == CommConfig(("norm_0", "linear_1"), (16, 1024))
    assert _parse_config_string("none-none-16-1024") == CommConfig(("none", "none"), (16, 1024))
    for bad in ("16-1024", "norm_0-16-1024", "a-b-c-d"):
        with pytest.raises(ValueError):
            _parse_config_string(bad)
    assert _TRAIL_CONFIG == CommConfig(("norm_0", "none"), (20, 1024))


def test_shipped_plan_00324(fixtures_dir):
    stages = parse_schedule_file(os.path.join(fixtures_dir, "scheds_pipeline_00324.py"), True, False)
    assert len(stages) == 2 and [len(s) for s in stages] == [16, 16]
    kinds = ["B" if it.bwd_mlp is not None else "F" for it in stages[0]]
    assert "".join(kinds) == "FFBFBFBFBFBFBFBB"  # stage 0 of a 2-stage 1F1B with 8 microbatches
    assert "".join("B" if it.bwd_mlp is not None else "F" for it in stages[1]) == "FB" * 8
    first = stages[0][0]
    assert first == ScheduleItem(fwd_attn=CommConfig(("norm_0", "none"), (12, 1024)),
                                 fwd_mlp=CommConfig(("norm_0", "none"), (18, 1024)), bwd_attn=None, bwd_mlp=None)
    assert first.fwd_trail == _TRAIL_CONFIG and first.bwd_trail == _TRAIL_CONFIG
    third = stages[0][2]  # ('backward', rec_attn, rec_mlp, attn, mlp): recompute configs land in fwd_*
    assert third.fwd_attn == CommConfig(("attn_0", "none"), (21, 1024))
    assert third.fwd_mlp == CommConfig(("norm_0", "none"), (15, 1024))
    assert third.bwd_attn == CommConfig(("rope_0", "none"), (30, 1024))
    assert third.bwd_mlp == CommConfig(("activation_0", "none"), (15, 1024))
    assert stages[1][1].fwd_attn == CommConfig(("rope_0", "none"), (6, 1024))
    # every window of the shipped plans ends with the "none" sentinel and uses a known slot
    for path in ("scheds_pipeline_00324.py", "scheds_pipeline_02328.py"):
        for stage in parse_schedule_file(os.path.join(fixtures_dir, path), True, False):
            for it in stage:
                for cfg in (it.fwd_attn, it.fwd_mlp, it.bwd_attn, it.bwd_mlp):
                    if cfg is not None:
                        assert cfg.overlap_window[1] == "none" and cfg.resource_shape[1] == 1024
                        assert cfg.overlap_window[0] in {"norm_0", "linear_0", "rope_0", "attn_0", "activation_0", "linear_1"}


def test_shipped_frequency_plan(fixtures_dir):
    stages = parse_frequency_file(os.path.join(fixtures_dir, "freqs_pipeline_02328.py"))
    assert [len(s) for s in stages] == [16, 16]
    assert stages[0][:3] == [("forward", 1410), ("forward", 900), ("backward", 1320)]
    assert stages[1][-1] == ("backward", 1410)
    assert all(900 <= mhz <= 1410 and mhz % 30 == 0 for st in stages for _, mhz in st)  # A100 sweep grid
    # same instruction order as the schedule of the same plan
    sched = parse_schedule_file(os.path.join(fixtures_dir, "scheds_pipeline_02328.py"), True, False)
    for st_f, st_s in zip(stages, sched):
        assert [n for n, _ in st_f] == ["backward" if it.bwd_mlp is not None else "forward" for it in st_s]


def test_frequency_plan_is_stepped_and_applied(fixtures_dir):
    """The frequency plan of a stage drives the same four hooks as the communication schedule:
    one (instruction, MHz) per instruction, the clock switched only when the value changes, the
    instruction kind checked, the plan drained at step end."""
    from kareus_amd.scheduler import PipelineFrequencyScheduler

    path = os.path.join(fixtures_dir, "freqs_pipeline_02328.py")
    plan = parse_frequency_file(path)[0]
    calls = []
    sch = PipelineFrequencyScheduler(path, pp_rank=0, num_instructions=16,
                                     set_frequency=lambda mhz: (calls.append(mhz), True)[1],
                                     reset_frequency=lambda: True)
    for _ in range(2):                       # two steps: the plan restarts, the clock is remembered
        sch.on_step_begin()
        for name, _mhz in plan:
            sch.on_instruction_begin(name)
            sch.on_instruction_end(name)
        sch.on_step_end()
        assert [(n, f) for n, f, _ in sch.history] == plan and all(a for _, _, a in sch.history)
    changes = [mhz for i, (_, mhz) in enumerate(plan + plan) if i == 0 or mhz != (plan + plan)[i - 1][1]]
    assert calls == changes and sch.current_frequency == plan[-1][1]
    assert sch.release() and sch.current_frequency is None
    # a setter that is refused (an ordinary user may not write the clock files) is recorded, not fatal
    denied = PipelineFrequencyScheduler(path, pp_rank=1, set_frequency=lambda mhz: False, reset_frequency=lambda: False)
    denied.on_step_begin()
    denied.on_instruction_begin("forward")
    assert denied.history == [("forward", parse_frequency_file(path)[1][0][1], False)] and not denied.applied
    # wrong instruction kind, plan overrun, plan not drained, bad arguments
    with pytest.raises(RuntimeError, match="mismatch"):
        denied.on_instruction_begin("forward" if parse_frequency_file(path)[1][1][0] == "backward" else "backward")
    sch.on_step_begin()
    sch.on_instruction_begin("forward")
    with pytest.raises(RuntimeError, match="more entries"):
        sch.on_step_end()
    sch.on_step_begin()
    for name, _ in plan:
        sch.on_instruction_begin(name)
    with pytest.raises(RuntimeError, match="No more planned"):
        sch.on_instruction_begin("forward")
    with pytest.raises(IndexError):
        PipelineFrequencyScheduler(path, pp_rank=2)
    with pytest.raises(ValueError, match="does not match"):
        PipelineFrequencyScheduler(path, pp_rank=0, num_instructions=8)
    with pytest.raises(FileNotFoundError):
        PipelineFrequencyScheduler(os.path.join(fixtures_dir, "missing.py"), pp_rank=0)
    # the default setter goes through sysfs; without a GPU (or without write access) it reports False
    default = PipelineFrequencyScheduler(path, pp_rank=0)
    default.on_step_begin()
    default.on_instruction_begin("forward")
    assert default.history[0][:2] == plan[0] and default.history[0][2] in (False, True)
    default.release()   # hands the clock back if the write was allowed


def test_other_grammars(fixtures_dir, tmp_path):
    ac = parse_schedule_file(os.path.join(fixtures_dir, "single_stage_ac.py"), True, False)
    assert len(ac) == 1 and len(ac[0]) == 4
    assert ac[0][2].fwd_mlp == CommConfig(("none", "none"), (27, 1024))
    assert ac[0][3].bwd_attn == CommConfig((0, -1), (30, 1024)) and ac[0][3].bwd_mlp == CommConfig((-1, -1), (15, 1024))
    pm = parse_schedule_file(os.path.join(fixtures_dir, "per_microbatch.py"), False, False)
    assert pm[0][1] == ScheduleItem(fwd_attn=CommConfig(("rope_0", "none"), (6, 512)),
                                    fwd_mlp=CommConfig(("none", "none"), (18, 1024)),
                                    bwd_attn=CommConfig(("attn_0", "none"), (30, 1024)),
                                    bwd_mlp=CommConfig(("norm_0", "none"), (15, 1024)))
    # context-parallel grammars parse into the CP item type
    cp = tmp_path / "cp.py"
    f = "'norm_0-none-8-1024'"
    cp.write_text(f"[[('forward', {', '.join([f] * 5)}), ('backward', {', '.join([f] * 12)})]]")
    items = parse_schedule_file(cp, True, True)[0]
    assert isinstance(items[0], ScheduleItemCP) and items[0].bwd_mlp is None and items[1].bwd_qkv_rs is not None
    cp.write_text(f"[[(('forward', {', '.join([f] * 5)}), ('backward', {', '.join([f] * 7)}))]]")
    assert parse_schedule_file(cp, False, True)[0][0].bwd_o_ar == CommConfig(("norm_0", "none"), (8, 1024))


@pytest.mark.parametrize("text,ac,err", [
    ("{'a': 1}", True, TypeError),                                  # top level must be a list
    ("[('forward', 'a', 'b')]", True, TypeError),                    # stage entry must be a list
    ("[[('forward', '0-0-1-1')]]", True, TypeError),                 # too few fields
    ("[[('forward', '0--1-1-1', '0--1-1-1', '0--1-1-1')]]", True, TypeError),
    ("[[('backward', '0--1-1-1', '0--1-1-1', '0--1-1-1')]]", True, TypeError),
    ("[[('sideways', '0--1-1-1', '0--1-1-1')]]", True, ValueError),
    ("[[('forward', '0--1-1-1', '0--1-1-1')]]", False, TypeError),   # pair grammar expected
    ("[[(('backward', '0--1-1-1', '0--1-1-1'), ('forward', '0--1-1-1', '0--1-1-1'))]]", False, ValueError),
    ("[[('forward', 'norm_0-1024', '0--1-1-1')]]", True, ValueError),
])
def test_malformed_files(tmp_path, text, ac, err):
    p = tmp_path / "bad.py"
    p.write_text(text)
    with pytest.raises(err):
        parse_schedule_file(p, ac, False)


def test_file_is_never_executed(tmp_path):
    marker = tmp_path / "pwned"
    p = tmp_path / "evil.py"
    p.write_text(f"[__import__('pathlib').Path({str(marker)!r}).write_text('x')]")
    with pytest.raises(Exception):
        parse_schedule_file(p, True, False)
    assert not marker.exists()


def test_scheduler_state_machine_ac(fixtures_dir):
    path = os.path.join(fixtures_dir, "scheds_pipeline_00324.py")
    sch = PipelineCommScheduler(path, pp_rank=1, num_microbatches=8, use_activation_checkpointing=True)
    assert sch.current_schedule is None
    sch.on_step_begin()
    for i in range(8):
        sch.on_instruction_begin("forward")
        assert sch.current_schedule.bwd_mlp is None
        sch.on_instruction_end("forward")
        sch.on_instruction_begin("backward")
        assert sch.current_schedule.bwd_attn is not None
    with pytest.raises(RuntimeError, match="No more scheduled instructions"):
        sch.on_instruction_begin("forward")
    sch.on_step_end()  # drained: resets
    assert sch.current_schedule is None
    sch.on_instruction_begin("forward")
    with pytest.raises(RuntimeError, match="expected 'backward', got 'forward'"):
        sch.on_instruction_begin("forward")  # stage 1 alternates F, B
    with pytest.raises(RuntimeError, match="more items than expected"):
        sch.on_step_end()


def test_scheduler_state_machine_per_microbatch(fixtures_dir):
    path = os.path.join(fixtures_dir, "per_microbatch.py")
    sch = PipelineCommScheduler(path, pp_rank=0, num_microbatches=2)
    sch.on_instruction_begin("forward")
    first = sch.current_schedule
    sch.on_instruction_begin("backward")  # does not advance
    assert sch.current_schedule is first
    sch.on_instruction_begin("forward")
    assert sch.current_schedule is not first
    with pytest.raises(RuntimeError, match="No more forward microbatches"):
        sch.on_instruction_begin("forward")
    sch.on_step_end()
    with pytest.raises(ValueError, match="does not match num_microbatches"):
        PipelineCommScheduler(path, pp_rank=0, num_microbatches=3)
    with pytest.raises(IndexError, match="out of range"):
        PipelineCommScheduler(path, pp_rank=1, num_microbatches=2)
    with pytest.raises(FileNotFoundError):
        PipelineCommScheduler(path + ".txt", pp_rank=0, num_microbatches=2)
    with pytest.raises(FileNotFoundError):
        PipelineCommScheduler(os.path.join(fixtures_dir, "missing.py"), pp_rank=0, num_microbatches=2)
    parsed = parse_schedule_file(path, False, False)
    again = PipelineCommScheduler.from_parsed(parsed, 0, 2)
    again.on_instruction_begin("forward")
    assert again.current_schedule == first


def test_a_failed_clock_write_is_retried_and_never_recorded_as_applied(fixtures_dir):
    from kareus_amd.scheduler import PipelineFrequencyScheduler

    path = os.path.join(fixtures_dir, "freqs_pipeline_02328.py")
    plan = parse_frequency_file(path)[0]
    outcomes = iter([False, True] + [True] * 64)
    calls = []
    sch = PipelineFrequencyScheduler(path, pp_rank=0, set_frequency=lambda mhz: (calls.append(mhz), next(outcomes))[1],
                                     reset_frequency=lambda: True)
    sch.on_step_begin()
    sch.on_instruction_begin(plan[0][0])
    assert sch.current_frequency is None and sch.history[-1][2] is False
    sch.on_instruction_begin(plan[1][0])          # tried again even if the planned value is the same
    assert len(calls) == 2 and sch.current_frequency == plan[1][1] and sch.history[-1][2] is True
    assert sch.history[0][2] is False             # the earlier row still says the truth


def test_sysfs_node_is_found_by_pci_bus_id_not_by_listing_order(tmp_path):
    """card10 sorts before card2 as text and a one-GPU lease may be any card: the node is matched by bus id."""
    from kareus_amd.energy import sysfs_device_dir

    root = tmp_path / "sys"
    for card, bdf in ((0, "0000:05:00.0"), (2, "0000:15:00.0"), (10, "0000:85:00.0")):
        real = root / "devices" / "pci0000:00" / bdf
        real.mkdir(parents=True)
        (root / "class" / "drm" / f"card{card}").mkdir(parents=True)
        os.symlink(real, root / "class" / "drm" / f"card{card}" / "device")
    got = sysfs_device_dir(0, sysfs_root=str(root), bus_id="0000:85:00.0")
    assert got is not None and os.path.realpath(got).endswith("0000:85:00.0")
    assert sysfs_device_dir(0, sysfs_root=str(root), bus_id="0000:99:00.0") is None   # no match: nothing is picked
    (root / "bus" / "pci" / "devices").mkdir(parents=True)
    os.symlink(root / "devices" / "pci0000:00" / "0000:15:00.0", root / "bus" / "pci" / "devices" / "0000:15:00.0")
    assert sysfs_device_dir(0, sysfs_root=str(root), bus_id="0000:15:00.0").endswith("bus/pci/devices/0000:15:00.0")
