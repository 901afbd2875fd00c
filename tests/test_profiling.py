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
    return R.linear(_attention(R.rmsnorm(x, p["ln1"], DIMS.eps), p["w_qkv"]), p["w_proj"])


def _oracle_fwd_mlp(t):
    p = {k: v.detach().float().cpu() for k, v in _params(t.layer).items()}
    x = t.forward_tensors["main"].detach().float().cpu() + t.forward_tensors["residual"].detach().float().cpu()
    return R.linear(R.swiglu(R.linear(R.rmsnorm(x, p["ln2"], DIMS.eps), p["w_fc1"])), p["w_fc2"])


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


@pytest.mark.gpu
@pytest.mark.parametrize("key", PARTITION_KEYS)
def test_partitions_on_the_gpu_match_the_host_engine(key):
    """Same partition, same seed: hand-written kernels (bf16) against the eager engine (fp32)."""
    dims = dict(hidden_size=512, num_attention_heads=4, num_query_groups=2, kv_channels=128, ffn_hidden_size=640)
    host = PartitionTest(key, LayerConfig(**dims, num_nanobatches=2, params_dtype=torch.float32, backend="eager"),
                         batch_size=4, seq_len=256)
    dev = PartitionTest(key, LayerConfig(**dims, num_nanobatches=2, backend="hip"), batch_size=4, seq_len=256,
                        device="cuda:0")
    out = "grad_main" if key.startswith("bwd") else "main"
    for w in (dev.overlap_windows[0], dev.overlap_windows[-1]):
        host.test_config(w, (16, 1024))
        dev.test_config(w, (16, 1024))
        torch.cuda.synchronize()
        a, b = dev.executor.output(out).float().cpu(), host.executor.output(out)
        assert (a - b).abs().max() <= 2e-2 * b.abs().max(), (key, w)   # bf16 vs fp32: 2e-2 max-relative
