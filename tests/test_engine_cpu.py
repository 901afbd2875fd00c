"""The partition engine end to end on the host: benchmark configuration 1 (fp32 plumbing layer) through
graph -> partitions -> contexts -> single autograd node, with the eager backend, against the CPU
oracle; nanobatch counts 1, 2 and 4, with and without activation recompute, with and without a
schedule; host-forceable error paths; and the stream/event ordering rules replayed without a GPU."""

import os

import pytest
import torch

from kareus_amd import LayerConfig, LayerStack
from kareus_amd.operators import NoOpAllReduce, QKVPostProcessOp, RMSNorm
from kareus_amd.partitions import NanoBatchContext, TensorStore, TransformerBlockAutogradFunction
from kareus_amd.partitions.autograd_function import _flatten_grad_params
from kareus_amd.partitions.partition_base import PartitionBase
from kareus_amd.partitions.streams import use_stream_api
from kareus_amd.schedule_check import RecordingStreams
from kareus_amd.scheduler import CommConfig, PipelineCommScheduler, ScheduleItem
from oracle import llama_layer_ref as R

C1 = dict(hidden_size=512, num_attention_heads=8, num_query_groups=8, kv_channels=64, ffn_hidden_size=1376)
PARAMS = [("input_layernorm", "ln1"), ("linear_qkv", "w_qkv"), ("linear_proj", "w_proj"),
          ("pre_mlp_layernorm", "ln2"), ("linear_fc1", "w_fc1"), ("linear_fc2", "w_fc2")]


def _oracle(layers, s, b, seed=42, dims=None):
    dims = dims or R.LayerDims(512, 8, 8, 64, 1376)
    gen = torch.Generator().manual_seed(1234)
    params = [R.init_layer_params(dims, gen) for _ in range(layers)]
    gd = torch.Generator().manual_seed(seed)
    x, go = torch.randn(s, b, dims.hidden, generator=gd), torch.randn(s, b, dims.hidden, generator=gd)
    return x, go, R.stack_forward_backward(x, params, dims, go)


def _run(model, x, go):
    xx = x.clone().requires_grad_(True)
    y = model(xx)
    y.backward(go)
    return y.detach(), xx.grad


def _check(model, x, go, ref, tol=2e-4):
    y, dx = _run(model, x, go)
    ry, rdx, rgrads = ref
    assert (y - ry).abs().max() <= tol * ry.abs().max()
    assert (dx - rdx).abs().max() <= tol * rdx.abs().max()
    for li, layer in enumerate(model.layers):
        for attr, name in PARAMS:
            g, rg = getattr(layer, attr).weight.grad, rgrads[li][name]
            assert (g - rg).abs().max() <= tol * rg.abs().max(), (li, name)


@pytest.mark.parametrize("nnb", [1, 2, 4])
@pytest.mark.parametrize("recompute", [False, True])
def test_config1_matches_oracle(nnb, recompute):
    # benchmark configuration 1 is b=2, s=256, 2 nanobatches; b=4 here so that 4 nanobatches divide it
    x, go, ref = _oracle(layers=1, s=256, b=4)
    cfg = LayerConfig(**C1, num_layers=1, num_nanobatches=nnb, params_dtype=torch.float32,
                      backend="eager", checkpoint_activations=recompute)
    _check(LayerStack(cfg, seed=1234), x, go, ref)


@pytest.mark.parametrize("recompute", [False, True])
def test_fused_weight_gradient_accumulation_equals_autograd_sum(recompute):
    """With the fusion on, the first nanobatch's wgrad buffer receives the other nanobatches'
    products (later copies report None); with it off autograd sums N separate gradients.  Both
    must give the oracle's gradient."""
    x, go, ref = _oracle(layers=2, s=128, b=4)
    grads = {}
    for fuse in (True, False):
        cfg = LayerConfig(**C1, num_layers=2, num_nanobatches=4, params_dtype=torch.float32,
                          backend="eager", checkpoint_activations=recompute,
                          fuse_wgrad_accumulation=fuse)
        model = LayerStack(cfg, seed=1234)
        _check(model, x, go, ref)
        grads[fuse] = [p.grad.clone() for p in model.parameters()]
    for a, b in zip(grads[True], grads[False]):
        assert (a - b).abs().max() <= 1e-5 * b.abs().max()


@pytest.mark.parametrize("recompute", [False, True])
def test_weight_gradient_over_all_nanobatches_equals_per_nanobatch_accumulation(recompute):
    """One product per layer over the tokens of all nanobatches (launched by the last nanobatch to
    deliver its operands, which survive the engine's op-by-op release of saved tensors) against one
    accumulating product per nanobatch: the same gradient, and the oracle's."""
    x, go, ref = _oracle(layers=2, s=128, b=4)
    grads = {}
    for whole, at_end in ((True, True), (True, False), (False, None)):
        cfg = LayerConfig(**C1, num_layers=2, num_nanobatches=4, params_dtype=torch.float32,
                          backend="eager", checkpoint_activations=recompute,
                          wgrad_over_all_nanobatches=whole, wgrad_launches_at_end=at_end)
        model = LayerStack(cfg, seed=1234)
        _check(model, x, go, ref)
        grads[whole, at_end] = [p.grad.clone() for p in model.parameters()]
    for a, b, c in zip(grads[True, True], grads[True, False], grads[False, None]):
        assert torch.equal(a, b)                         # when the launch is issued does not change what it computes
        assert (a - c).abs().max() <= 1e-5 * c.abs().max()


@pytest.mark.parametrize("b,nnb", [(4, 4), (8, 4), (4, 2)])
@pytest.mark.parametrize("recompute", [False, True])
def test_nanobatches_joined_in_place_equal_concatenation(b, nnb, recompute, monkeypatch):
    """The last op of every nanobatch writes into its slice of one [s, b, h] tensor (and the first
    fork's backward into its slice of the input gradient): same numbers as concatenating, and
    no concatenation is run."""
    x, go, ref = _oracle(layers=2, s=64, b=b)
    results = {}
    for in_place in (False, True):
        cfg = LayerConfig(**C1, num_layers=2, num_nanobatches=nnb, params_dtype=torch.float32,
                          backend="eager", checkpoint_activations=recompute,
                          join_nanobatches_in_place=in_place)
        model = LayerStack(cfg, seed=1234)
        calls = []
        real_cat = torch.cat
        monkeypatch.setattr(torch, "cat", lambda *a, **k: (calls.append(1), real_cat(*a, **k))[1])
        y, dx = _run(model, x, go)
        monkeypatch.setattr(torch, "cat", real_cat)
        results[in_place] = (y, dx, [p.grad.clone() for p in model.parameters()], len(calls))
        assert y.is_contiguous() and dx.is_contiguous() and y.shape == x.shape
    (y0, dx0, g0, cats0), (y1, dx1, g1, cats1) = results[False], results[True]
    assert torch.equal(y0, y1) and torch.equal(dx0, dx1)
    assert all(torch.equal(a, c) for a, c in zip(g0, g1))
    # joining costs two concatenations (outputs, input gradients); the QKV merge in the attention
    # backward concatenates too and is there either way
    assert cats0 - cats1 == 2
    ry, rdx, _ = ref
    assert (y1 - ry).abs().max() <= 2e-4 * ry.abs().max() and (dx1 - rdx).abs().max() <= 2e-4 * rdx.abs().max()


@pytest.mark.parametrize("nnb", [1, 4])
def test_fused_norm_and_fork_backward_changes_nothing(nnb, monkeypatch):
    """RMSNorm backward and the residual fork's backward run as one call when adjacent (two pairs
    per layer); switching the fusion off, or putting the schedule's launch point between the
    two, gives the same bits."""
    from kareus_amd.operators.rmsnorm import RMSNorm
    from kareus_amd.partitions.backward_partition import BackwardPartition

    x, go, ref = _oracle(layers=2, s=64, b=4)
    fused_calls = []
    real = RMSNorm.fuser_backward

    def spy(self, ctxs, dy, **kw):
        fused_calls.append(len(ctxs))
        return real(self, ctxs, dy, **kw)

    monkeypatch.setattr(RMSNorm, "fuser_backward", spy)
    results = {}
    for fuse in (True, False):
        cfg = LayerConfig(**C1, num_layers=2, num_nanobatches=nnb, params_dtype=torch.float32, backend="eager")
        model = LayerStack(cfg, seed=1234)
        for part in model.backward_partitions:
            assert isinstance(part, BackwardPartition)
            part.fuse_backward_ops = fuse
        fused_calls.clear()
        y, dx = _run(model, x, go)
        results[fuse] = (y, dx, [p.grad.clone() for p in model.parameters()])
        assert fused_calls == [2 if fuse else 1] * (4 * nnb)   # 2 layers x 2 norms per nanobatch
    assert torch.equal(results[True][1], results[False][1])
    assert all(torch.equal(a, c) for a, c in zip(results[True][2], results[False][2]))
    for p in model.parameters():
        p.grad = None
    _check(model, x, go, ref)


@pytest.mark.parametrize("nnb", [1, 2, 4])
@pytest.mark.parametrize("recompute", [False, True])
def test_forward_epilogue_fusions_change_nothing(nnb, recompute, monkeypatch):
    """fc1 runs the SwiGLU activation behind it as part of its own call, the out-projection and fc2 add the
    residual themselves and the BiasDropoutAddOp behind the all-reduce slot passes the sum on; a schedule
    whose launch point falls between fc1 and the activation switches that pair off.  Same numbers either way."""
    from kareus_amd.operators.bias_dropout_add import BiasDropoutAddOp
    from kareus_amd.operators.linear import PartitionableLinear

    x, go, ref = _oracle(layers=2, s=64, b=4)
    calls = {"pairs": 0, "passed_on": 0, "bwd_pairs": 0}
    real_linear, real_bda = PartitionableLinear.fuser_forward, BiasDropoutAddOp.fuser_forward
    real_linear_bwd = PartitionableLinear.fuser_backward

    def spy_linear_bwd(self, ctxs, dy, **kw):
        calls["bwd_pairs"] += len(ctxs) == 2
        return real_linear_bwd(self, ctxs, dy, **kw)

    monkeypatch.setattr(PartitionableLinear, "fuser_backward", spy_linear_bwd)

    def spy_linear(self, ctxs, x_, **kw):
        calls["pairs"] += len(ctxs) == 2
        return real_linear(self, ctxs, x_, **kw)

    def spy_bda(self, ctxs, x_, **kw):
        out = real_bda(self, ctxs, x_, **kw)
        calls["passed_on"] += out[0] is x_
        return out

    monkeypatch.setattr(PartitionableLinear, "fuser_forward", spy_linear)
    monkeypatch.setattr(BiasDropoutAddOp, "fuser_forward", spy_bda)
    results = {}
    for fuse in (True, False):
        cfg = LayerConfig(**C1, num_layers=2, num_nanobatches=nnb, params_dtype=torch.float32, backend="eager",
                          checkpoint_activations=recompute, fuse_forward_epilogues=fuse)
        model = LayerStack(cfg, seed=1234)
        calls.update(pairs=0, passed_on=0, bwd_pairs=0)
        y, dx = _run(model, x, go)
        results[fuse] = (y, dx, [p.grad.clone() for p in model.parameters()])
        assert calls["bwd_pairs"] == (2 * nnb if fuse else 0)     # fc2's backward takes the activation's along
        passes = 2 if recompute else 1                       # the recompute runs the forward again
        assert calls["pairs"] == (2 * nnb * passes if fuse else 0)          # one fc1 per layer and nanobatch
        # two residual adds per layer; the last one of a nanobatch writes into the block's output, and a
        # nanobatch of more than one sequence is a slice of it that no single row stride addresses: that add
        # stays a separate call (the recompute pass has no output to write)
        kept = nnb if (nnb > 1 and x.shape[1] // nnb > 1) else 0
        assert calls["passed_on"] == (4 * nnb * passes - kept if fuse else 0)
    assert torch.allclose(results[True][0], results[False][0], atol=1e-6)
    assert torch.allclose(results[True][1], results[False][1], atol=1e-6)
    assert all(torch.allclose(a, c, atol=1e-5) for a, c in zip(results[True][2], results[False][2]))
    for p in model.parameters():
        p.grad = None
    cfg = LayerConfig(**C1, num_layers=2, num_nanobatches=nnb, params_dtype=torch.float32, backend="eager",
                      checkpoint_activations=recompute)
    _check(LayerStack(cfg, seed=1234), x, go, ref)
    # a launch point between fc1 (linear_0 of the MLP partition) and the activation: the pair runs as two calls
    cfg.kareus_scheduler = None
    model = LayerStack(cfg, seed=1234)
    for part in model.forward_partitions:
        if part.partition_key == "fwd_mlp":
            part._schedule_config = (("activation_0", "none"), (16, 1024))
    calls.update(pairs=0, passed_on=0, bwd_pairs=0)
    _check(model, x, go, ref)
    assert calls["pairs"] == (0 if nnb > 1 else 2 * (2 if recompute else 1))   # (one nanobatch: no launch points)


def _params_of(model):
    return [{name: getattr(layer, attr).weight.detach().clone() for attr, name in PARAMS} for layer in model.layers]


@pytest.mark.parametrize("recompute", [False, True])
def test_hidden_dropout_matches_oracle_given_the_masks(recompute):
    """Hidden dropout in front of the two residual adds (bias_dropout_add.py:24-45): with the masks the
    operators drew handed to the oracle, output and every gradient agree; with recomputation the backward
    pass draws the same masks again (the generator states are saved and replayed,
    autograd_function.py:143-146, 263-266)."""
    prob, dims = 0.25, R.LayerDims(512, 8, 8, 64, 1376)
    cfg = LayerConfig(**C1, num_layers=1, num_nanobatches=1, params_dtype=torch.float32, backend="eager",
                      hidden_dropout=prob, checkpoint_activations=recompute)
    model = LayerStack(cfg, seed=1234)
    gd = torch.Generator().manual_seed(5)
    x, go = torch.randn(64, 2, 512, generator=gd), torch.randn(64, 2, 512, generator=gd)
    torch.manual_seed(77)
    y, dx = _run(model, x, go)
    layer = model.layers[0]
    masks = (prob, layer.self_attn_bda.last_mask.clone(), layer.mlp_bda.last_mask.clone())
    for m in masks[1:]:
        assert m.shape == x.shape and 0.70 < m.float().mean() < 0.80      # about 1 - p of the elements kept
    assert not torch.equal(masks[1], masks[2])
    xx = x.clone().requires_grad_(True)
    leaves = {k: v.requires_grad_(True) for k, v in _params_of(model)[0].items()}
    freqs = R.rope_table(64, dims.hd, dims.rope_base)
    ry = R.layer_forward(xx, leaves, dims, freqs, dropout=masks)
    ry.backward(go)
    tol = 2e-4
    assert (y - ry.detach()).abs().max() <= tol * ry.abs().max()
    assert (dx - xx.grad).abs().max() <= tol * xx.grad.abs().max()
    for attr, name in PARAMS:
        g, rg = getattr(layer, attr).weight.grad, leaves[name].grad
        assert (g - rg).abs().max() <= tol * rg.abs().max(), name
    # without dropout the layer gives something else; the same seed gives the same step again
    assert (y - R.layer_forward(x, _params_of(model)[0], dims, freqs)).abs().max() > 1e-2
    for layer_param in model.parameters():
        layer_param.grad = None
    torch.manual_seed(77)
    y2, dx2 = _run(model, x, go)
    assert torch.equal(y, y2) and torch.equal(dx, dx2)


def test_hidden_dropout_with_nanobatches_and_in_evaluation():
    """Every nanobatch draws its own mask (so the result depends on the nanobatch count, as in the reference,
    where each nanobatch's native_dropout call advances the generator); recomputation changes nothing; a layer
    that is not training applies no dropout."""
    base = dict(**C1, num_layers=1, params_dtype=torch.float32, backend="eager", hidden_dropout=0.3)
    gd = torch.Generator().manual_seed(6)
    x, go = torch.randn(32, 4, 512, generator=gd), torch.randn(32, 4, 512, generator=gd)
    results = []
    for recompute in (False, True):
        model = LayerStack(LayerConfig(**base, num_nanobatches=2, checkpoint_activations=recompute), seed=1234)
        torch.manual_seed(3)
        y, dx = _run(model, x, go)
        results.append((y, dx, [p.grad.clone() for p in model.parameters()]))
    (y0, dx0, g0), (y1, dx1, g1) = results
    assert torch.equal(y0, y1) and torch.equal(dx0, dx1) and all(torch.equal(a, b) for a, b in zip(g0, g1))
    model = LayerStack(LayerConfig(**base, num_nanobatches=2), seed=1234)
    for layer in model.layers:
        layer.self_attn_bda.training = layer.mlp_bda.training = False
    plain = LayerStack(LayerConfig(**{**base, "hidden_dropout": 0.0}, num_nanobatches=2), seed=1234)
    ya, dxa = _run(model, x, go)
    yb, dxb = _run(plain, x, go)
    assert torch.equal(ya, yb) and torch.equal(dxa, dxb)


@pytest.mark.parametrize("nnb,recompute,grouped", [(1, False, True), (2, True, True), (2, False, False)])
def test_query_and_key_norms_match_oracle(nnb, recompute, grouped):
    """The q / k layernorm of the QKV split (Qwen3-style layers; qkv_postprocess.py:115-118 forward,
    :150-157 backward, weight gradients query first): output, input gradient and every parameter's gradient,
    the two head-norm weights included, against the oracle; the nanobatches' weight gradients add up."""
    dims = R.LayerDims(hidden=64, nq=6, nkv=2, hd=16, ffn=40)
    cfg = LayerConfig(hidden_size=64, num_attention_heads=6, num_query_groups=2, kv_channels=16, ffn_hidden_size=40,
                      num_layers=2, num_nanobatches=nnb, params_dtype=torch.float32, backend="eager",
                      qk_layernorm=True, checkpoint_activations=recompute)
    model = LayerStack(cfg, seed=1234)
    gd = torch.Generator().manual_seed(8)
    for layer in model.layers:
        layer.qkv_postprocess.grouped_query_view = grouped
        for norm in (layer.qkv_postprocess.q_layernorm, layer.qkv_postprocess.k_layernorm):
            with torch.no_grad():
                norm.weight.copy_(1 + 0.3 * torch.randn(16, generator=gd))
    names = [n for n, _ in model.named_parameters() if "qkv_postprocess" in n]
    assert [n.split("qkv_postprocess.")[1] for n in names[:2]] == ["q_layernorm.weight", "k_layernorm.weight"]
    x, go = torch.randn(24, 4, 64, generator=gd), torch.randn(24, 4, 64, generator=gd)
    y, dx = _run(model, x, go)
    params = []
    for layer, plain in zip(model.layers, _params_of(model)):
        post = layer.qkv_postprocess
        params.append({**plain, "q_norm": post.q_layernorm.weight.detach().clone(),
                       "k_norm": post.k_layernorm.weight.detach().clone()})
    ry, rdx, rgrads = R.stack_forward_backward(x, params, dims, go)
    tol = 2e-4
    assert (y - ry).abs().max() <= tol * ry.abs().max()
    assert (dx - rdx).abs().max() <= tol * rdx.abs().max()
    for layer, rg in zip(model.layers, rgrads):
        post = layer.qkv_postprocess
        got = {name: getattr(layer, attr).weight.grad for attr, name in PARAMS}
        got.update(q_norm=post.q_layernorm.weight.grad, k_norm=post.k_layernorm.weight.grad)
        for name, g in got.items():
            assert (g - rg[name]).abs().max() <= tol * rg[name].abs().max(), name
    # the norms matter: the oracle without them is somewhere else
    assert (R.stack_forward(x, _params_of(model), dims, R.rope_table(24, 16, dims.rope_base)) - ry).abs().max() > 1e-2


def test_config1_exact_shape_two_layers():
    x, go, ref = _oracle(layers=2, s=256, b=2)
    cfg = LayerConfig(**C1, num_layers=2, num_nanobatches=2, params_dtype=torch.float32, backend="eager")
    _check(LayerStack(cfg, seed=1234), x, go, ref)


def test_gqa_layer_and_dense_query_view():
    dims = R.LayerDims(hidden=64, nq=6, nkv=2, hd=16, ffn=40)
    x, go, ref = _oracle(layers=1, s=24, b=2, dims=dims)
    cfg = LayerConfig(hidden_size=64, num_attention_heads=6, num_query_groups=2, kv_channels=16, ffn_hidden_size=40,
                      num_layers=1, num_nanobatches=2, params_dtype=torch.float32, backend="eager")
    m = LayerStack(cfg, seed=1234)
    _check(m, x, go, ref)
    # the reference's dense [s, b, nq, hd] query layout gives the same numbers
    m.layers[0].qkv_postprocess.grouped_query_view = False
    for p in m.parameters():
        p.grad = None
    _check(m, x, go, ref)
    op = QKVPostProcessOp(2, 6, 16)
    mixed = torch.arange(2 * 3 * 160, dtype=torch.float32).reshape(2, 3, 160)
    q, k, v = op.split(mixed)
    rq, rk, rv = R.split_qkv(mixed, 6, 2, 16)
    assert torch.equal(q.flatten(2, 3), rq) and torch.equal(k, rk) and torch.equal(v, rv)
    assert q.data_ptr() == mixed.data_ptr()  # a view, not a copy
    assert torch.equal(op.merge(q.flatten(2, 3), k, v), mixed)  # merge inverts split


def test_schedule_driven_run_matches_and_records_shapes(fixtures_dir):
    x, go, ref = _oracle(layers=1, s=64, b=2)
    cfg = LayerConfig(**C1, num_layers=1, num_nanobatches=2, params_dtype=torch.float32,
                      backend="eager", checkpoint_activations=True)
    m = LayerStack(cfg, seed=1234)
    sch = PipelineCommScheduler(os.path.join(fixtures_dir, "scheds_pipeline_00324.py"), pp_rank=1,
                                num_microbatches=8, use_activation_checkpointing=True)
    cfg.kareus_scheduler = sch
    xx = x.clone().requires_grad_(True)
    sch.on_step_begin()
    sch.on_instruction_begin("forward")
    y = m(xx)
    assert m.allreduce_comm_ops[1].last_resource_shape == (18, 1024)  # NB1's last carrier: fwd_mlp of item 0
    assert m.allreduce_comm_ops[0].last_resource_shape == (20, 1024)  # fwd_trail default
    sch.on_instruction_begin("backward")
    y.backward(go)  # recompute pass reads rec_attn/rec_mlp, backward reads bwd_attn/bwd_mlp
    assert m.allreduce_comm_ops[1].last_resource_shape == (21, 1024)  # bwd_attn 'rope_0-none-21-1024'
    ry, rdx, _ = ref
    assert (y.detach() - ry).abs().max() <= 2e-4 * ry.abs().max()
    assert (xx.grad - rdx).abs().max() <= 2e-4 * rdx.abs().max()
    assert m.allreduce_comm_ops[0].calls > 0 and m.allreduce_comm_ops[1].calls > 0


def test_host_error_paths():
    cfg = LayerConfig(**C1, num_layers=1, num_nanobatches=2, params_dtype=torch.float32, backend="eager")
    m = LayerStack(cfg, seed=0)
    with pytest.raises(ValueError, match="multiple of 2 nanobatches"):
        m(torch.randn(8, 1, 512))
    with pytest.raises(ValueError, match="multiple of 2 nanobatches"):
        m(torch.randn(8, 3, 512))
    with pytest.raises(ValueError, match=r"\[s, b, 512\]"):
        m(torch.randn(8, 2, 256))
    with pytest.raises(NotImplementedError):
        m(torch.randn(8, 2, 512), attention_mask=torch.ones(1))
    with pytest.raises(NotImplementedError):
        m(torch.randn(8, 2, 512), packed_seq_params=object())
    with pytest.raises(ValueError, match="rotary table covers"):
        m(torch.randn(8, 2, 512), rotary_pos_emb=m.rotary_pos_emb(4))
    with pytest.raises(RuntimeError, match="executed by the partition engine"):
        m.layers[0](torch.randn(1))
    with pytest.raises(NotImplementedError):
        LayerStack(LayerConfig(**C1, attention_dropout=0.1, params_dtype=torch.float32, backend="eager"))
    with pytest.raises(ValueError, match="outside"):
        LayerStack(LayerConfig(**C1, hidden_dropout=1.5, params_dtype=torch.float32, backend="eager"))
    with pytest.raises(NotImplementedError):
        LayerStack(LayerConfig(**C1, add_bias_linear=True, params_dtype=torch.float32, backend="eager"))
    with pytest.raises(NotImplementedError, match="come as a pair"):
        QKVPostProcessOp(2, 6, 16, q_layernorm=torch.nn.LayerNorm(16))
    with pytest.raises(NotImplementedError, match="only an RMSNorm"):
        QKVPostProcessOp(2, 6, 16, q_layernorm=torch.nn.LayerNorm(16), k_layernorm=torch.nn.LayerNorm(16))
    with pytest.raises(ValueError, match="over the head dimension"):
        QKVPostProcessOp(2, 6, 16, q_layernorm=RMSNorm(32, backend="eager"), k_layernorm=RMSNorm(32, backend="eager"))
    with pytest.raises(NotImplementedError):
        NoOpAllReduce(world_size=2)
    with pytest.raises(ValueError, match="unknown backend"):
        LayerStack(LayerConfig(**C1, params_dtype=torch.float32, backend="triton"))(torch.randn(8, 2, 512))
    store = TensorStore()
    with pytest.raises(KeyError, match="tensor_id 't_9' not found"):
        store.get("t_9")
    with pytest.raises(AssertionError, match="Parameter gradient count mismatch"):
        _flatten_grad_params({0: [None], 1: [None]}, 3)
    with pytest.raises(AssertionError, match="parameter list repeated"):
        TransformerBlockAutogradFunction.apply(torch.randn(2, 1, 512), torch.randn(2, 1, 512), None, None, m.forward_partitions,
                                               m.backward_partitions, m.forward_tensor_graph, m.backward_tensor_graph,
                                               None, cfg, m.seed_config, True, False, *m._get_all_params()[:5])


def test_hip_backend_refuses_host_tensors_and_missing_library(monkeypatch):
    from kareus_amd.backend import hip

    if os.path.exists(hip.library_path()):
        be = hip.HipBackend()
        with pytest.raises(RuntimeError, match="HIP device"):
            be.add(torch.zeros(8, dtype=torch.bfloat16), torch.zeros(8, dtype=torch.bfloat16))
    monkeypatch.setattr(hip, "_LIB_NAME", "libdoes_not_exist.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        hip.load_library()


def test_saved_tensor_bookkeeping():
    ctx = NanoBatchContext(batch_idx=0)
    a, b, c = torch.ones(1), torch.ones(2), torch.ones(3)
    ctx.create_op_context(5).save_for_backward(c)
    ctx.create_op_context(2).save_for_backward(a, b)
    ctx.create_op_context(3)  # saves nothing
    flat = ctx.flatten_saved_tensors()
    assert [t.numel() for t in flat] == [1, 2, 3]  # op id order, not creation order
    assert ctx.get_op_context(2).to_save is None
    ctx.restore_saved_tensors(tuple(flat))
    assert ctx.get_op_context(5).saved_tensors[0] is c and ctx.get_op_context(3).saved_tensors is None
    ctx.clear_saved_tensors_except({id(a)})
    assert a.numel() == 1 and b.numel() == 0 and c.numel() == 0


def _replay(window, nnb=2, layers=1):
    rec = RecordingStreams()
    with use_stream_api(rec):
        cfg = LayerConfig(hidden_size=64, num_attention_heads=2, num_query_groups=1, kv_channels=32, ffn_hidden_size=64,
                          num_layers=layers, num_nanobatches=nnb, params_dtype=torch.float32, backend="eager")
        m = LayerStack(cfg, seed=1)
        if window is not None:
            cc = CommConfig(window, (20, 1024))

            class Sch:
                current_schedule = ScheduleItem(cc, cc, cc, cc)  # trail partitions keep the default window

            cfg.kareus_scheduler = Sch()
        PartitionBase.timer = rec
        try:
            x = torch.randn(16, 2 * nnb, 64, requires_grad=True)
            m(x).sum().backward()
        finally:
            PartitionBase.timer = None
    return rec


def test_stream_protocol_replay():
    # slot "none": a hand-over is released only after the carrying partition's compute, so from the
    # second segment on the two nanobatches strictly alternate
    rec = _replay(("none", "none"))
    assert rec.violations == []
    f = lambda key, nb: rec.find("ForwardPartition", key, nb)
    assert rec.ordered(f("fwd_attn", 1), f("fwd_mlp", 0))   # NB0 seg 1 waits for NB1 seg 0
    assert rec.ordered(f("fwd_mlp", 0), f("fwd_mlp", 1))    # NB1 seg 1 waits for NB0 seg 1
    assert rec.may_overlap(f("fwd_attn", 0), f("fwd_attn", 1))  # nothing to hand over yet
    # a nanobatch's own partitions are always ordered (same stream)
    assert rec.ordered(f("fwd_attn", 0), f("fwd_mlp", 0)) and rec.ordered(f("fwd_attn", 1), f("fwd_mlp", 1))
    b = lambda key, nb: rec.find("BackwardPartition", key, nb)
    assert rec.ordered(b("bwd_mlp", 1), b("bwd_attn", 0)) and rec.ordered(b("bwd_attn", 0), b("bwd_attn", 1))
    # forward finished on every stream before backward starts anywhere (join / fork)
    assert rec.ordered(f("fwd_trail", 0), b("bwd_mlp", 1)) and rec.ordered(f("-", 1), b("bwd_mlp", 0))

    # slot 0 (default window, or "norm_0"): released before the first op -> compute may overlap
    for window in (None, ("norm_0", "none")):
        rec = _replay(window)
        assert rec.violations == []
        f = lambda key, nb: rec.find("ForwardPartition", key, nb)
        assert rec.may_overlap(f("fwd_attn", 1), f("fwd_mlp", 0))
        assert rec.may_overlap(f("fwd_mlp", 0), f("fwd_mlp", 1))
        assert rec.ordered(f("fwd_attn", 0), f("fwd_mlp", 0))
        # the carrier still waits, at its end, until the owner has passed the hand-over
        assert not rec.ordered(f("fwd_mlp", 1), f("fwd_attn", 0))

    # a mid-partition slot: NB1's next segment may start once NB0's carrier passed that op
    rec = _replay(("linear_0", "none"))
    carrier, owner_next = rec.find("ForwardPartition", "fwd_mlp", 0), rec.find("ForwardPartition", "fwd_mlp", 1)
    slot = carrier_slot = 3  # bda, fork, ln | fc1  -> linear_0 is op 3
    assert rec.happens_before(carrier.op_done[slot - 1], owner_next.begin)
    assert not rec.happens_before(carrier.op_done[slot], owner_next.begin)
    assert rec.violations == []

    for nnb in (1, 4):
        rec = _replay(("norm_0", "none"), nnb=nnb, layers=2)
        assert rec.violations == [] and len(rec.spans) == 2 * nnb * 5


def test_resource_shape_reserves_compute_units_for_the_other_streams(monkeypatch):
    """A schedule's resource shape (sm_num, block_size) acts on the launches: while a partition that carries a
    hand-over runs on its nanobatch's stream, that many compute units are reserved (GEMM launches take the
    rest); partitions without a schedule entry, and runs without nanobatch streams, reserve nothing."""
    from kareus_amd.backend import reserved_compute_units
    from kareus_amd.backend.eager import EagerBackend

    seen = []
    real = EagerBackend.linear_fwd

    def spy(self, x, w, **kw):
        seen.append(reserved_compute_units())
        return real(self, x, w, **kw)

    monkeypatch.setattr(EagerBackend, "linear_fwd", spy)
    rec = RecordingStreams()
    cfg = LayerConfig(hidden_size=64, num_attention_heads=2, num_query_groups=1, kv_channels=32, ffn_hidden_size=64,
                      num_layers=1, num_nanobatches=2, params_dtype=torch.float32, backend="eager")
    attn, mlp = CommConfig(("norm_0", "none"), (24, 1024)), CommConfig(("linear_0", "none"), (40, 512))

    class Sch:
        current_schedule = ScheduleItem(attn, mlp, attn, mlp)

    with use_stream_api(rec):
        m = LayerStack(cfg, seed=1)
        cfg.kareus_scheduler = Sch()
        with torch.no_grad():
            m(torch.randn(16, 4, 64))
    # per nanobatch: qkv, proj (fwd_attn), fc1, fc2 (fwd_mlp); the first partition of all carries no hand-over
    assert sorted(seen) == sorted([0, 0, 24, 24, 40, 40, 40, 40])
    assert reserved_compute_units() == 0
    seen.clear()
    cfg2 = LayerConfig(hidden_size=64, num_attention_heads=2, num_query_groups=1, kv_channels=32, ffn_hidden_size=64,
                       num_layers=1, num_nanobatches=2, params_dtype=torch.float32, backend="eager", use_streams=False)
    m2 = LayerStack(cfg2, seed=1)
    cfg2.kareus_scheduler = Sch()
    with torch.no_grad():
        m2(torch.randn(16, 4, 64))
    assert seen == [0] * 8
