"""Per-partition profiler: the stand-alone partitions must compute what the same operators compute
inside the layer (checked against the CPU oracle), every release point must give the same numbers,
and the measuring loop / eval-log bookkeeping must behave as the reference's does
(tests/bayesian/common/{partition_executor,hardware,orchestration}.py)."""

import json

import pytest
import torch

from kareus_amd import LayerConfig
from kareus_amd.profiling import (
    PARTITION_KEYS, PartitionExecutor, PartitionTest, all_configurations, append_eval_log,
    build_eval_record, load_eval_log, measure, measure_batch,
)
from kareus_amd.partitions.tensor_graph import CommunicationType
from oracle import llama_layer_ref as R

DIMS = R.LayerDims(hidden=64, nq=4, nkv=2, hd=16, ffn=48)


def _cfg(backend="eager", dtype=torch.float32, nnb=2):
    return LayerConfig(hidden_size=DIMS.hidden, num_attention_heads=DIMS.nq, num_query_groups=DIMS.nkv,
                       kv_channels=DIMS.hd, ffn_hidden_size=DIMS.ffn, num_nanobatches=nnb,
                       params_dtype=dtype, backend=backend)


def _params(layer):
    return {"ln1": layer.input_layernorm.weight, "w_qkv": layer.linear_qkv.weight,
            "w_proj": layer.linear_proj.weight, "ln2": layer.pre_mlp_layernorm.weight,
            "w_fc1": layer.linear_fc1.weight, "w_fc2": layer.linear_fc2.weight}


def _attention(h, w_qkv):
    s, b, _ = h.shape
    q, k, v = R.split_qkv(R.linear(h, w_qkv), DIMS.nq, DIMS.nkv, DIMS.hd)
    freqs = R.rope_table(s, DIMS.hd, 500000.0)
    return R.causal_gqa_attention(R.rope(q, freqs), R.rope(k, freqs), v).reshape(s, b, DIMS.nq * DIMS.hd)


def _oracle_fwd_attn(t):
    p = {k: v.detach().float().cpu() for k, v in _params(t.layer).items()}
    x = t.forward_tensors["main"].detach().float().cpu()
    y = R.linear(_attention(R.rmsnorm(x, p["ln1"], DIMS.eps), p["w_qkv"]), p["w_proj"])
    # with the residual add folded into the projection's epilogue the partition's output already
    # holds what the BiasDropoutAddOp of the next partition would have added
    return x + y if t.layer.linear_proj.fuse_residual else y


def _oracle_fwd_mlp(t):
    p = {k: v.detach().float().cpu() for k, v in _params(t.layer).items()}
    x = t.forward_tensors["main"].detach().float().cpu() + t.forward_tensors["residual"].detach().float().cpu()
    y = R.linear(R.swiglu(R.linear(R.rmsnorm(x, p["ln2"], DIMS.eps), p["w_fc1"])), p["w_fc2"])
    return x + y if t.layer.linear_fc2.fuse_residual else y


@pytest.mark.parametrize("key", ["fwd_attn", "fwd_mlp"])
def test_forward_partitions_match_oracle_at_every_release_point(key):
    t = PartitionTest(key, _cfg(), batch_size=4, seq_len=32)
    want = (_oracle_fwd_attn if key == "fwd_attn" else _oracle_fwd_mlp)(t)
    assert t.overlap_windows[-1] == ("none", "none") and len(t.overlap_windows) >= 4
    for w in t.overlap_windows:
        t.test_config(w, (16, 1024))
        got = t.executor.output("main")
        assert (got - want).abs().max() <= 2e-4 * want.abs().max(), w
        # the other nanobatch's tensor went through the hand-over unchanged
        assert t.executor.pre_ctx.tensor_store.get("comm_out_main") is t.handover
    assert t.comm_op.calls == len(t.overlap_windows) and t.comm_op.last_resource_shape == (16, 1024)


@pytest.mark.parametrize("key", ["bwd_mlp", "bwd_attn"])
def test_backward_partitions_match_autograd_and_are_repeatable(key):
    t = PartitionTest(key, _cfg(), batch_size=4, seq_len=32)
    p = {k: v.detach().clone().requires_grad_(True) for k, v in _params(t.layer).items()}
    x = t.forward_tensors["main"].detach().clone().requires_grad_(True)
    res = t.forward_tensors["residual"].detach().clone().requires_grad_(True)
    if key == "bwd_mlp":
        y = R.linear(R.swiglu(R.linear(x, p["w_fc1"])), p["w_fc2"]) + res
        y.backward(t.grad_tensors["grad_main"])
        weights = {0: "w_fc1", 2: "w_fc2"}
    else:
        a = R.linear(_attention(x, p["w_qkv"]), p["w_proj"]) + res
        y = R.rmsnorm(a, p["ln2"], DIMS.eps)
        (y * t.grad_tensors["grad_main"]).sum().backward(retain_graph=True)
        (a * t.grad_tensors["grad_residual"]).sum().backward()
        weights = {0: "w_qkv", 4: "w_proj", 7: "ln2"}
    first = None
    for w in t.overlap_windows:   # profiling mode keeps the saved activations: every run is complete
        grads = t.test_config(w, (8, 512))
        dx = t.executor.output("grad_main")
        assert (dx - x.grad).abs().max() <= 2e-4 * x.grad.abs().max(), w
        for op_id, name in weights.items():
            g, rg = grads[op_id][0], p[name].grad
            assert (g - rg).abs().max() <= 2e-4 * rg.abs().max(), (w, name)
        first = first if first is not None else dx.clone()
        assert torch.equal(dx, first)


def test_executor_runs_the_partition_under_its_compute_unit_budget(monkeypatch):
    """The ``sm`` of a configuration is reserved while the partition runs (its device-filling
    launches take the rest), and only then."""
    from kareus_amd.backend import reserved_compute_units
    t = PartitionTest("fwd_mlp", _cfg(), batch_size=2, seq_len=16)
    seen = []
    inner = t.executor.partition.execute
    monkeypatch.setattr(t.executor.partition, "execute",
                        lambda **kw: (seen.append(reserved_compute_units()), inner(**kw))[1])
    for sm in (16, 64, 0):
        t.test_config(("linear_0", "none"), (sm, 1024))
    assert seen == [16, 64, 0] and reserved_compute_units() == 0


def test_executor_argument_errors():
    t = PartitionTest("fwd_mlp", _cfg(), batch_size=2, seq_len=16)
    with pytest.raises(ValueError, match="Invalid direction"):
        PartitionExecutor(t.comp_ops, t.comm_op, "sideways", "fwd_mlp")
    with pytest.raises(ValueError, match="fwd_initial_channel_names is required"):
        PartitionExecutor(t.comp_ops, t.comm_op, "backward", "bwd_mlp", initial_channel_names=["grad_main"])
    with pytest.raises(ValueError, match="No default comm channels"):
        PartitionExecutor(t.comp_ops, t.comm_op, "forward", "fwd_mlp", comm_type=CommunicationType.ALL_GATHER_KV)
    with pytest.raises(ValueError, match="Unknown channel name"):
        t.executor.setup_contexts({"nope": t.handover}, [t.handover])
    with pytest.raises(KeyError, match="Unknown overlap slot"):
        t.test_config(("attn_0", "none"), (16, 1024))      # the MLP partition has no attention slot
    with pytest.raises(ValueError, match="comm_end must be -1"):
        t.test_config(("norm_0", "linear_1"), (16, 1024))
    with pytest.raises(ValueError, match="unknown partition key"):
        PartitionTest("fwd_everything", _cfg(), 2, 16)
    assert set(PARTITION_KEYS) == {"fwd_attn", "fwd_mlp", "bwd_mlp", "bwd_attn"}


class _FakeClock:
    def __init__(self, per_call):
        self.now, self.per_call = 100.0, per_call

    def tick(self):
        self.now += self.per_call

    def __call__(self):
        return self.now


class _FakeSampler:
    available = True

    def __init__(self, watts):
        self.watts, self.started, self.stopped = watts, 0, 0

    def start(self):
        self.started += 1

    def stop(self):
        self.stopped += 1

    def energy_joules(self, t0, t1):
        return self.watts * (t1 - t0)


def test_measure_counts_iterations_and_integrates_power():
    clock = _FakeClock(per_call=0.01)
    sampler = _FakeSampler(watts=500.0)
    slept = []
    trial = measure(clock.tick, sampler, measurement_duration=1.0, cooldown_duration=2.5, warmup_iterations=3,
                    sync=lambda: None, clock=clock, sleep=slept.append, batch=8)
    assert slept == [2.5] and sampler.started == sampler.stopped == 1
    assert trial.iterations == 104          # first multiple of 8 calls whose 10 ms steps reach 1 s
    assert trial.time_per_iter == pytest.approx(0.01)
    assert trial.energy_per_iter == pytest.approx(5.0) and trial.mean_watts == pytest.approx(500.0)
    none = measure(clock.tick, None, 0.05, 0.0, sync=lambda: None, clock=clock, sleep=slept.append)
    assert none.energy_per_iter is None and none.mean_watts is None


def test_configuration_grid_and_eval_log(tmp_path):
    grid = all_configurations([2100, 1500], [8, 16], [("norm_0", "none"), ("none", "none")])
    assert len(grid) == 8 and grid[0] == {"freq": 2100, "sm": 8, "block": 1024, "overlap": ("norm_0", "none")}
    assert [c["freq"] for c in grid[:4]] == [2100] * 4 and grid[1]["overlap"] == ("none", "none")
    rec = build_eval_record(grid[0], 1.5e-3, 2.0)
    assert rec == {"freq": 2100, "overlap_start": "norm_0", "overlap_end": "none", "sm": 8, "block": 1024,
                   "time_s": 1.5e-3, "energy_j": 2.0}
    path = str(tmp_path / "eval.jsonl")
    assert load_eval_log(path) == []
    append_eval_log(path, [rec, build_eval_record(grid[2], 1e-3, None)])
    append_eval_log(path, [dict(rec, time_s=9.9)])                      # same configuration again
    rows = load_eval_log(path)
    assert len(rows) == 2 and rows[0]["time_s"] == 1.5e-3               # first occurrence wins
    with open(path, "a") as f:
        f.write("not json\n")
    assert load_eval_log(path) == []


def test_measure_batch_on_the_host():
    t = PartitionTest("fwd_mlp", _cfg(), batch_size=2, seq_len=16)
    configs = all_configurations([0], [4], t.overlap_windows[:2])
    recs = measure_batch(t, configs, None, measurement_duration=0.02, cooldown_duration=0.0,
                         warmup_iterations=1, batch=2)
    assert [r["overlap_start"] for r in recs] == [w[0] for w in t.overlap_windows[:2]]
    assert all(r["time_s"] > 0 and r["energy_j"] is None and r["freq_applied"] is False for r in recs)
    assert t.comm_op.last_resource_shape == (4, 1024)
    json.dumps(recs)


def _oracle_partition(key, t, dims):
    """What one partition computes, composed from the oracle's operator functions (fp32, autograd for the
    backward partitions) on the partition test's own tensors; operator lists as in
    tests/bayesian/common/partition_executor.py:74-318 of the reference / ``partition_tests._operators``."""
    from oracle import llama_layer_ref as R

    f32 = lambda x: x.detach().float().cpu()
    w = {n: f32(getattr(t.layer, a).weight) for a, n in (
        ("input_layernorm", "ln1"), ("linear_qkv", "w_qkv"), ("linear_proj", "w_proj"),
        ("pre_mlp_layernorm", "ln2"), ("linear_fc1", "w_fc1"), ("linear_fc2", "w_fc2"))}
    fw = {n: f32(v) for n, v in t.forward_tensors.items()}
    s, b = t.seq_length, t.nano_batch_size

    def attention_block(x):      # qkv -> split -> rope -> attention -> proj
        q, k, v = R.split_qkv(R.linear(x, w["w_qkv"]), dims.nq, dims.nkv, dims.hd)
        fr = fw["rotary_pos_emb"]
        a = R.causal_gqa_attention(R.rope(q, fr), R.rope(k, fr), v).reshape(s, b, dims.nq * dims.hd)
        return R.linear(a, w["w_proj"])

    def mlp_block(x):            # fc1 -> swiglu -> fc2
        return R.linear(R.swiglu(R.linear(x, w["w_fc1"])), w["w_fc2"])

    fused = t.layer.linear_proj.fuse_residual   # the projections add the residual in their epilogue
    if key == "fwd_attn":
        y = attention_block(R.rmsnorm(fw["main"], w["ln1"], dims.eps))
        return fw["main"] + y if fused else y
    if key == "fwd_mlp":
        x2 = fw["residual"] + fw["main"]
        y = mlp_block(R.rmsnorm(x2, w["ln2"], dims.eps))
        return x2 + y if fused else y
    g = {n: f32(v) for n, v in t.grad_tensors.items()}
    x = fw["main"].clone().requires_grad_(True)
    if key == "bwd_mlp":         # forward: residual + mlp(main); upstream gradient on that sum
        (fw["residual"] + mlp_block(x)).backward(g["grad_main"])
        return x.grad
    x2 = fw["residual"] + attention_block(x)   # bwd_attn: ... then the fork and the second norm
    (R.rmsnorm(x2, w["ln2"], dims.eps) * g["grad_main"]).sum().add((x2 * g["grad_residual"]).sum()).backward()
    return x.grad


@pytest.mark.gpu
@pytest.mark.parametrize("key", PARTITION_KEYS)
def test_partitions_on_the_gpu_match_the_oracle(key):
    """Each stand-alone partition on the HIP kernels (bf16) against the same operators composed from the CPU
    oracle's functions in fp32 on the same tensors, for the earliest and the latest release point; bf16
    tolerance 2e-2 max-relative."""
    from oracle import llama_layer_ref as R

    dims = R.LayerDims(512, 4, 2, 128, 640)
    cfg = LayerConfig(hidden_size=512, num_attention_heads=4, num_query_groups=2, kv_channels=128,
                      ffn_hidden_size=640, num_nanobatches=2, backend="hip")
    dev = PartitionTest(key, cfg, batch_size=4, seq_len=256, device="cuda:0")
    want = _oracle_partition(key, dev, dims)
    out = "grad_main" if key.startswith("bwd") else "main"
    for w in (dev.overlap_windows[0], dev.overlap_windows[-1]):
        dev.test_config(w, (16, 1024))
        torch.cuda.synchronize()
        got = dev.executor.output(out).float().cpu()
        err = (got - want).abs().max()
        print(f"{key} {w}: max-rel {err / want.abs().max():.3e} max-abs {err:.3e}")
        assert err <= 2e-2 * want.abs().max(), (key, w)


# ---- eval logs -> solver input ---------------------------------------------------------------------
from kareus_amd.profiling.profile_csv import (  # noqa: E402
    candidate_points, generate_profile_csv, layers_per_stage, pareto_optimal, read_eval_log,
)
from kareus_amd.scheduler.parser import _parse_config_string  # noqa: E402


def test_listed_clock_levels_and_the_label_without_a_device(tmp_path, monkeypatch):
    """``pp_dpm_sclk`` lines ``"<n>: <MHz>Mhz [*]"`` are the levels (a line ``S: ...`` is the clock in
    force, not a level); without a device to ask, a sweep that pins no clock is labelled with the
    highest of them, and with 0 when there is no such file."""
    from kareus_amd.profiling import hardware
    dev = tmp_path / "dev"
    dev.mkdir()
    (dev / "pp_dpm_sclk").write_text("0: 132Mhz\n1: 2105Mhz *\n2: 2400Mhz\nS: 2105Mhz *\n")
    monkeypatch.setattr(hardware, "sysfs_device_dir", lambda i=0: str(dev))
    assert hardware.available_frequencies_mhz() == [132, 2105, 2400]
    assert hardware.nominal_frequency_mhz() == 2400          # no GPU here: the listed maximum
    (dev / "pp_dpm_sclk").unlink()
    assert hardware.available_frequencies_mhz() == [] and hardware.nominal_frequency_mhz() == 0


@pytest.mark.gpu
def test_nominal_clock_is_the_devices_rated_clock():
    """The label of a sweep that pins no clock comes from the device's properties, so two reads
    (and the four partitions' logs of one sweep) agree."""
    from kareus_amd.profiling import nominal_frequency_mhz
    a, b = nominal_frequency_mhz(), nominal_frequency_mhz()
    assert a == b and 1000 <= a <= 4000


def test_pareto_filter_uses_effective_energy():
    pts = [("a", (1.0, 100.0)), ("b", (2.0, 90.0)), ("c", (3.0, 95.0)), ("d", (1.0, 120.0)), ("e", (4.0, 150.0))]
    # no idle power: keep strictly improving energy along increasing time
    assert [k for k, _ in pareto_optimal(pts, 0.0)] == ["a", "b"]
    # 20 W idle: effective energies 80, 50, 35, 100, 70 -> c now improves on b
    assert [k for k, _ in pareto_optimal(pts, 20.0)] == ["a", "b", "c"]
    # an improvement below the tolerance does not count
    assert [k for k, _ in pareto_optimal([("a", (1.0, 10.0)), ("b", (2.0, 10.0 - 5e-5))], 0.0)] == ["a"]
    assert pareto_optimal([], 85.0) == []


def test_layers_per_stage():
    assert layers_per_stage(32, 1) == [32]
    assert layers_per_stage(32, 2, 15, 17) == [15, 17]
    assert layers_per_stage(32, 2, 20, 20) == [20, 12]            # inconsistent pair: last is what is left
    assert layers_per_stage(28, 4, 6, 6) == [6, 8, 8, 6]
    assert layers_per_stage(29, 5, 5, 5) == [5, 7, 6, 6, 5]       # remainder goes to the earlier middle stages
    with pytest.warns(UserWarning):
        assert layers_per_stage(8, 3, 6, 6) == [6, 0, 2]
    with pytest.raises(ValueError):
        layers_per_stage(8, 0)


def _write_logs(tmp_path, nested=False):
    rows = {
        "fwd_attn": [(1500, "norm_0", 1.0, 10.0), (1500, "attn_0", 0.9, 10.5), (2100, "norm_0", 0.7, 12.0)],
        "fwd_mlp": [(1500, "linear_0", 2.0, 20.0), (2100, "linear_0", 1.5, 25.0)],
        "bwd_attn": [(1500, "linear_1", 3.0, 30.0), (2100, "linear_1", 2.0, 36.0)],
        "bwd_mlp": [(1500, "none", 4.0, 40.0), (2100, "none", 3.0, 50.0), (900, "none", 9.0, 30.0)],
    }
    for key, items in rows.items():
        path = tmp_path / key / "eval_results.jsonl" if nested else tmp_path / f"{key}.jsonl"
        path.parent.mkdir(parents=True, exist_ok=True)
        with open(path, "w") as f:
            for freq, start, t, e in items:
                f.write(json.dumps(build_eval_record({"freq": freq, "sm": 16, "block": 1024, "overlap": (start, "none")}, t, e)) + "\n")
            f.write("garbage\n")
            f.write(json.dumps({"freq": 1500, "time_s": 1.0}) + "\n")                       # fields missing
            f.write(json.dumps(build_eval_record({"freq": 1500, "sm": 8, "block": 1024, "overlap": ("x", "none")}, 1.0, None)) + "\n")
    return rows


def test_candidate_table_closed_form(tmp_path):
    _write_logs(tmp_path)
    logs = {k: read_eval_log(str(tmp_path / f"{k}.jsonl")) for k in ("fwd_attn", "fwd_mlp", "bwd_attn", "bwd_mlp")}
    assert sorted(logs["fwd_attn"]) == [1500, 2100] and len(logs["fwd_attn"][1500]) == 2     # bad rows dropped
    extra = {1500: {"forward-embedding": (0.5, 5.0), "forward-output": (0.25, 2.5), "loss-func": (0.125, 1.25),
                    "backward-embedding": (1.0, 10.0), "backward-output": (2.0, 20.0)}}
    fwd, bwd = candidate_points(logs, [3, 5], nanobatches=2, use_activation_checkpointing=True,
                                scale_time_energy=False, nonpartition=extra)
    # frequency 900 exists for one partition only and is left out
    assert {k[0] for k, _ in fwd[0]} == {1500, 2100} and len(fwd[0]) == 3 and len(bwd[1]) == 3
    f0 = dict(fwd[0])[(1500, ("norm_0", "none", 16, 1024), ("linear_0", "none", 16, 1024))]
    assert f0 == (pytest.approx((1.0 + 2.0) * 3 * 2 + 0.5), pytest.approx((10.0 + 20.0) * 3 * 2 + 5.0))
    f1 = dict(fwd[1])[(1500, ("norm_0", "none", 16, 1024), ("linear_0", "none", 16, 1024))]
    assert f1 == (pytest.approx(3.0 * 5 * 2 + 0.25 + 0.125), pytest.approx(30.0 * 5 * 2 + 2.5 + 1.25))
    key = (1500, ("attn_0", "none", 16, 1024), ("linear_0", "none", 16, 1024),
           ("linear_1", "none", 16, 1024), ("none", "none", 16, 1024))
    assert dict(bwd[0])[key] == (pytest.approx((0.9 + 2 + 3 + 4) * 3 * 2 + 2 * 1.0), pytest.approx((10.5 + 20 + 30 + 40) * 6 + 20.0))
    assert dict(bwd[1])[key] == (pytest.approx(9.9 * 10 + 2.0), pytest.approx(100.5 * 10 + 20.0))
    # 2100 MHz has no non-partition figures: zeros; scaling multiplies both by 1.15
    fwd_s, _ = candidate_points(logs, [1], nanobatches=4, use_activation_checkpointing=False, scale_time_energy=True)
    k2 = (2100, ("norm_0", "none", 16, 1024), ("linear_0", "none", 16, 1024))
    assert dict(fwd_s[0])[k2] == (pytest.approx(2.2 * 1.15 * 4), pytest.approx(37.0 * 1.15 * 4))
    with pytest.raises(RuntimeError, match="No overlapping frequencies"):
        candidate_points(dict(logs, fwd_mlp={900: logs["bwd_mlp"][900]}), [1])


@pytest.mark.parametrize("recompute", [True, False])
def test_profile_csv_rows_feed_the_schedule_parser(tmp_path, recompute):
    _write_logs(tmp_path, nested=True)
    out = str(tmp_path / "profile.csv")
    kept = generate_profile_csv(str(tmp_path), out, num_layers=8, pipeline_parallel_size=2,
                                num_layers_in_first_pipeline_stage=4, num_layers_in_last_pipeline_stage=4,
                                gpu_type="A100", use_activation_checkpointing=recompute, scale_time_energy=False)
    lines = open(out).read().strip().splitlines()
    header = lines[0].split(",")
    assert header == (["stage", "instruction", "frequency", "recompute_attention_configs", "recompute_mlp_configs",
                       "attention_configs", "mlp_configs", "time", "energy"] if recompute else
                      ["stage", "instruction", "frequency", "attention_configs", "mlp_configs", "time", "energy"])
    assert len(lines) - 1 == kept["forward"] + kept["backward"] and kept["forward"] >= 2 and kept["backward"] >= 2
    for line in lines[1:]:
        cells = line.split(",")
        assert len(cells) == len(header) and cells[1] in ("forward", "backward") and cells[0] in ("0", "1")
        cfg_cells = cells[3:-2]
        if recompute and cells[1] == "forward":
            assert cfg_cells[:2] == ["", ""]
            cfg_cells = cfg_cells[2:]
        for c in cfg_cells:                                   # every configuration is a schedule-file field
            parsed = _parse_config_string(c)
            assert parsed.resource_shape == (16, 1024) and parsed.overlap_window[1] in ("none", -1)
        assert float(cells[-2]) > 0 and float(cells[-1]) > 0
    # Pareto per stage and direction: times strictly increase, effective energy strictly decreases
    for stage in ("0", "1"):
        for inst in ("forward", "backward"):
            pts = [(float(l.split(",")[-2]), float(l.split(",")[-1])) for l in lines[1:]
                   if l.split(",")[0] == stage and l.split(",")[1] == inst]
            eff = [e - 85.0 * t for t, e in pts]
            assert pts == sorted(pts) and all(b < a for a, b in zip(eff, eff[1:]))
    with pytest.raises(ValueError, match="Unknown GPU type"):
        generate_profile_csv(str(tmp_path), out, 8, gpu_type="H100")
    with pytest.raises(FileNotFoundError):
        generate_profile_csv(str(tmp_path / "missing"), out, 8)


def test_nonpartition_profiler_files_round_trip(tmp_path):
    from kareus_amd.profiling.nonpartition import HEADER, STEP_NAMES, NonPartitionProfiler, read_nonpartition

    prof = NonPartitionProfiler(_cfg(), vocab_rows=96, batch_size=4, seq_len=16)
    sampler = _FakeSampler(watts=300.0)
    trials = prof.run(str(tmp_path), 1500, sampler=sampler, world_size=2, measurement_duration=0.02,
                      cooldown_duration=0.0, warmup_iterations=1, batch=2)
    assert set(trials) == set(STEP_NAMES)
    for name in STEP_NAMES:
        lines = open(tmp_path / "nonpartition" / "1500" / f"{name}_energy.csv").read().strip().splitlines()
        assert lines[0] == HEADER and len(lines) == 2
        t, e, e_rank = (float(v) for v in lines[1].split(","))
        assert t == pytest.approx(trials[name].time_per_iter) and e == pytest.approx(300.0 * t, rel=1e-6)
        assert e_rank == pytest.approx(e / 2)
    table = read_nonpartition(str(tmp_path), [1500])
    assert set(table[1500]) == {"forward-embedding", "forward-output", "loss-func", "backward-embedding", "backward-output"}
    assert table[1500]["loss-func"] == (pytest.approx(trials["loss"].time_per_iter),
                                        pytest.approx(trials["loss"].energy_per_iter / 2))
    # the steps compute what the model's ends compute: postprocess = final norm + output layer
    logits = prof.step("postprocess")()
    x = torch.cat(prof.hidden_parts, dim=1)
    want = R.linear(R.rmsnorm(x, prof.final_gamma.detach(), 1e-5), prof.w_out.detach())
    assert (logits - want).abs().max() <= 2e-4 * want.abs().max()
    prof.step("preprocess_backward")()
    assert prof.embedding.weight.grad is not None and prof.embedding.weight.grad.shape == (96, DIMS.hidden)
    # and the table plugs into the candidate generator
    _write_logs(tmp_path)
    logs = {k: read_eval_log(str(tmp_path / f"{k}.jsonl")) for k in ("fwd_attn", "fwd_mlp", "bwd_attn", "bwd_mlp")}
    fwd, _ = candidate_points(logs, [2, 2], scale_time_energy=False, nonpartition=table)
    k = (1500, ("norm_0", "none", 16, 1024), ("linear_0", "none", 16, 1024))
    assert dict(fwd[0])[k][0] == pytest.approx(3.0 * 2 * 2 + table[1500]["forward-embedding"][0])
    with pytest.raises(FileNotFoundError):
        read_nonpartition(str(tmp_path), [999])
    with pytest.raises(ValueError, match="unknown step"):
        prof.step("postprocess_sideways")
