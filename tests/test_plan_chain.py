"""The schedule-generation chain end to end, as one test: sweep the four partitions -> eval logs -> candidate
table -> plan files -> a step of the layer stack under a generated plan -> the frequency plan stepped
through on the device node.

The reference's chain is tests/bayesian/common/orchestration.py:65-147 (eval-log rows) ->
tests/kareus/generate_profile_csv.py:56-57,159-172,314-317 (table) -> tests/kareus/run_optimization.py:1-40
(plans) -> kareus/scheduler/parser.py:122-165 (``parse_schedule_file``) and
kareus/scheduler/pipeline_comm_scheduler.py:97-144 (the four hooks of a step).

The same body runs on the host (eager backend, fp32, a constant-power stand-in for the board sensor) and, marked
``gpu``, on the device through the HIP kernels with the real board-power sensor.
"""

import os

import pytest
import torch

from kareus_amd import LayerConfig, LayerStack
from kareus_amd.energy import PowerSampler
from kareus_amd.profiling import (
    PARTITION_KEYS, PartitionTest, all_configurations, append_eval_log, measure_batch,
)
from kareus_amd.profiling.plan_generator import generate_plans, read_profile_csv
from kareus_amd.profiling.profile_csv import generate_profile_csv
from kareus_amd.scheduler import PipelineCommScheduler
from kareus_amd.scheduler.parser import parse_frequency_file, parse_schedule_file
from kareus_amd.scheduler.pipeline_frequency_scheduler import PipelineFrequencyScheduler
from oracle import llama_layer_ref as R

DIMS = R.LayerDims(512, 4, 2, 128, 640)
LAYERS, NNB, SEQ, BATCH, MICROBATCHES = 2, 2, 256, 4, 2
PARAMS = [("input_layernorm", "ln1"), ("linear_qkv", "w_qkv"), ("linear_proj", "w_proj"),
          ("pre_mlp_layernorm", "ln2"), ("linear_fc1", "w_fc1"), ("linear_fc2", "w_fc2")]


class _ConstantPower:
    """Stands in for the board sensor where there is none (the host runs)."""
    available = True

    def start(self):
        pass

    def stop(self):
        pass

    def energy_joules(self, t0, t1):
        return 100.0 * (t1 - t0)


def _config(backend, layers=LAYERS, **kw):
    return LayerConfig(hidden_size=DIMS.hidden, num_attention_heads=DIMS.nq, num_query_groups=DIMS.nkv,
                       kv_channels=DIMS.hd, ffn_hidden_size=DIMS.ffn, num_layers=layers, num_nanobatches=NNB,
                       backend=backend, params_dtype=torch.bfloat16 if backend == "hip" else torch.float32, **kw)


def _stack(backend, device, **kw):
    model = LayerStack(_config(backend, **kw), device=device, seed=1234)
    for layer in model.layers:     # bit-exact comparisons across modes: no GEMM cuts its contraction
        for op in (layer.linear_qkv, layer.linear_proj, layer.linear_fc1, layer.linear_fc2):
            op.split_k = None
    return model


def _step(model, sch, x, go):
    """One microbatch: a forward and a backward instruction (both announced to the scheduler)."""
    for p in model.parameters():
        p.grad = None
    dtype = next(model.parameters()).dtype
    xd = x.to(next(model.parameters()).device, dtype, copy=True).requires_grad_(True)
    if sch is not None:
        sch.on_instruction_begin("forward")
    y = model(xd)
    if sch is not None:
        sch.on_instruction_end("forward")
        sch.on_instruction_begin("backward")
    y.backward(go.to(xd.device, dtype))
    if sch is not None:
        sch.on_instruction_end("backward")
    if xd.is_cuda:
        torch.cuda.synchronize()
    grads = [[getattr(layer, a).weight.grad.clone() for a, _ in PARAMS] for layer in model.layers]
    return y.detach(), xd.grad, grads


def _rel(got, want):
    got, want = got.float().cpu(), want.float().cpu()
    return ((got - want).abs().max() / want.abs().max()).item()


def _chain(tmp_path, backend, device, sampler, recompute, tol):
    # 1. sweep: earliest and latest release slot x two reservations of compute units, short windows
    logs = tmp_path / "logs"
    logs.mkdir()
    freq = 2400
    for key in PARTITION_KEYS:
        test = PartitionTest(key, _config(backend, layers=1), batch_size=BATCH, seq_len=SEQ, device=device)
        windows = [test.overlap_windows[0], test.overlap_windows[-1]]
        configs = all_configurations([freq], [0, 16], windows)
        recs = measure_batch(test, configs, sampler, measurement_duration=0.03, cooldown_duration=0.0,
                             warmup_iterations=2, batch=4)
        assert len(recs) == 4 and all(r["time_s"] > 0 and r["energy_j"] is not None and r["energy_j"] > 0 for r in recs)
        assert {(r["overlap_start"], r["sm"]) for r in recs} == {(w[0], sm) for w in windows for sm in (0, 16)}
        append_eval_log(str(logs / f"{key}.jsonl"), recs)

    # 2. eval logs -> candidate table, in the reference's column layout
    table_path = str(tmp_path / "profile.csv")
    kept = generate_profile_csv(str(logs), table_path, num_layers=LAYERS, nanobatches=NNB,
                                use_activation_checkpointing=recompute, scale_time_energy=False)
    assert kept["forward"] >= 1 and kept["backward"] >= 1
    header = open(table_path).readline().strip().split(",")
    assert header == (["stage", "instruction", "frequency", "recompute_attention_configs", "recompute_mlp_configs",
                       "attention_configs", "mlp_configs", "time", "energy"] if recompute else
                      ["stage", "instruction", "frequency", "attention_configs", "mlp_configs", "time", "energy"])
    table, ac = read_profile_csv(table_path)
    assert ac == recompute and sorted(table) == [0]

    # 3. candidate table -> plans; every emitted file is read back by the parsers of the reference's grammar
    plans_dir = str(tmp_path / "plans")
    frontier = generate_plans(table_path, plans_dir, num_mbs=MICROBATCHES, unit_time=1e-6)
    assert frontier and all(a.quant_time > b.quant_time for a, b in zip(frontier, frontier[1:]))   # cheapest first, fastest last
    names = sorted(os.listdir(plans_dir))
    assert len(names) == 2 * len(frontier)
    for name in names:
        path = os.path.join(plans_dir, name)
        if name.startswith("freqs_"):
            stages = parse_frequency_file(path)
            assert len(stages) == 1 and [k for k, _ in stages[0]] == ["forward", "backward"] * MICROBATCHES
            assert all(mhz == freq for _, mhz in stages[0])
        else:
            stages = parse_schedule_file(path, recompute, False)
            # recompute grammar: one item per instruction (F B F B on one stage); else one per microbatch
            assert len(stages) == 1 and len(stages[0]) == MICROBATCHES * (2 if recompute else 1)
            for item in stages[0]:                              # every field resolves to a window and a shape
                fields = [cc for cc in (item.fwd_attn, item.fwd_mlp, item.bwd_attn, item.bwd_mlp) if cc is not None]
                assert len(fields) in ((2, 4) if recompute else (4,))
                for cc in fields:
                    assert cc.resource_shape[0] in (0, 16) and cc.resource_shape[1] == 1024
                    assert cc.overlap_window[1] in ("none", -1)

    # 4. a step of the stack under the cheapest and under the fastest plan
    plain = _stack(backend, device)
    g = torch.Generator().manual_seed(42)
    data = [(torch.randn(SEQ, BATCH, DIMS.hidden, generator=g), torch.randn(SEQ, BATCH, DIMS.hidden, generator=g))
            for _ in range(MICROBATCHES)]
    want = [_step(plain, None, x, go) for x, go in data]
    params = [{n: getattr(layer, a).weight.detach().float().cpu() for a, n in PARAMS} for layer in plain.layers]
    for it in sorted({frontier[0].iteration, frontier[-1].iteration}):
        sched = os.path.join(plans_dir, f"scheds_pipeline_{it:05d}.py")
        model = _stack(backend, device, checkpoint_activations=recompute)
        sch = PipelineCommScheduler(sched, pp_rank=0, num_microbatches=MICROBATCHES,
                                    use_activation_checkpointing=recompute)
        model.config.kareus_scheduler = sch
        sch.on_step_begin()
        for (x, go), (py, pdx, pgrads) in zip(data, want):
            y, dx, grads = _step(model, sch, x, go)
            assert torch.equal(y, py) and torch.equal(dx, pdx)                   # a plan moves no bit
            assert all(torch.equal(a, c) for la, lb in zip(grads, pgrads) for a, c in zip(la, lb))
        sch.on_step_end()
    # ... and the step itself against the oracle: one layer at a time on the layer's own inputs would be the
    # bound for a stack; two small layers stay inside the one-layer bound, which is what is asserted
    for (x, go), (py, pdx, pgrads) in zip(data, want):
        cast = (lambda t: t.bfloat16().float()) if backend == "hip" else (lambda t: t)
        ry, rdx, rgrads = R.stack_forward_backward(cast(x), params, DIMS, cast(go))
        errs = [_rel(py, ry), _rel(pdx, rdx)]
        errs += [_rel(pgrads[li][pi], rgrads[li][n]) for li in range(LAYERS) for pi, (_, n) in enumerate(PARAMS)]
        assert max(errs) <= tol, errs
    return plans_dir, frontier


@pytest.mark.parametrize("recompute", [False, True])
def test_chain_on_the_host(tmp_path, recompute):
    _chain(tmp_path, "eager", "cpu", _ConstantPower(), recompute, tol=2e-4)


@pytest.mark.gpu
@pytest.mark.skipif(not torch.cuda.is_available(), reason="needs a HIP device")
@pytest.mark.parametrize("recompute", [False, True])
def test_chain_on_the_gpu(tmp_path, recompute):
    """Sweep -> table -> plans -> scheduled step on the HIP kernels, board power from the device's own sensor
    (the constant-power stand-in only where the box exposes no sensor; the log rows then still carry energy)."""
    sampler = PowerSampler()
    if not sampler.available:
        print("no board-power sensor on this box: constant-power stand-in")
        sampler = _ConstantPower()
    _chain(tmp_path, "hip", "cuda:0", sampler, recompute, tol=2e-2)


def _performance_level(device_dir):
    try:
        with open(os.path.join(device_dir, "power_dpm_force_performance_level")) as f:
            return f.read().strip()
    except OSError:
        return None


@pytest.mark.gpu
@pytest.mark.skipif(not torch.cuda.is_available(), reason="needs a HIP device")
def test_frequency_plan_is_stepped_on_the_device_node(fixtures_dir):
    """``PipelineFrequencyScheduler`` over the reference's own ``freqs_pipeline_00324.py`` against the real
    sysfs node of the device, around real steps of the layer: one history row per instruction in the plan's
    order; each row either applied (the user may write the node) or a recorded refusal; the node's
    ``power_dpm_force_performance_level`` is left as it was found."""
    from kareus_amd.energy import sysfs_device_dir

    node = sysfs_device_dir(0)
    before = _performance_level(node) if node else None
    path = os.path.join(fixtures_dir, "freqs_pipeline_00324.py")
    plan = parse_frequency_file(path)[0]
    fs = PipelineFrequencyScheduler(path, pp_rank=0, num_instructions=len(plan))
    model = _stack("hip", "cuda:0", layers=1)
    g = torch.Generator().manual_seed(7)
    x = torch.randn(SEQ, BATCH, DIMS.hidden, generator=g).to("cuda", torch.bfloat16).requires_grad_(True)
    go = torch.randn(SEQ, BATCH, DIMS.hidden, generator=g).to("cuda", torch.bfloat16)
    first = None
    try:
        fs.on_step_begin()
        pending = []                                 # stage 0 runs F F B F B ... B B: outputs wait for their backward
        for name, _ in plan:
            fs.on_instruction_begin(name)
            if name == "forward":
                pending.append(model(x))
            else:
                x.grad = None
                pending.pop(0).backward(go)
                first = x.grad.clone() if first is None else first
                assert torch.equal(x.grad, first)                     # the clock plan moves no bit either
            fs.on_instruction_end(name)
        fs.on_step_end()
        torch.cuda.synchronize()
        assert not pending
        assert [(n, mhz) for n, mhz, _ in fs.history] == list(plan)
        applied = [a for _, _, a in fs.history]
        print(f"frequency plan: {sum(applied)} of {len(applied)} instructions applied; node {node}; "
              f"performance level before: {before}")
        if not fs.applied:
            # a refusal: nothing was applied, no clock is claimed, and later instructions kept trying
            assert not any(applied) and fs.current_frequency is None
        else:
            assert applied[-1] and fs.current_frequency == plan[-1][1]
        with pytest.raises(RuntimeError, match="No more planned frequencies"):
            fs.on_instruction_begin("forward")
    finally:
        released = fs.release()
        if fs.applied:
            assert released
    if node is not None and before is not None:
        # the node is handed back to the governor; a user who may not write it never changed it
        assert _performance_level(node) == (before if not any(a for _, _, a in fs.history) else "auto")
