"""The whole layer on the device through the partition engine and the HIP kernels, against the CPU
oracle (bf16 tolerance 2e-2, max-abs also printed), plus size-independent properties at the full
benchmark shapes."""

import os

import pytest
import torch

from kareus_amd import LayerConfig, LayerStack
from kareus_amd.scheduler import PipelineCommScheduler
from oracle import llama_layer_ref as R

pytestmark = [pytest.mark.gpu, pytest.mark.skipif(not torch.cuda.is_available(), reason="needs a HIP device")]
TOL = 2e-2
PARAMS = [("input_layernorm", "ln1"), ("linear_qkv", "w_qkv"), ("linear_proj", "w_proj"),
          ("pre_mlp_layernorm", "ln2"), ("linear_fc1", "w_fc1"), ("linear_fc2", "w_fc2")]


def _inputs(s, b, h, seed=42):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(s, b, h, generator=g), torch.randn(s, b, h, generator=g)


def _build(dims, layers, nnb, **kw):
    cfg = LayerConfig(hidden_size=dims.hidden, num_attention_heads=dims.nq, num_query_groups=dims.nkv,
                      kv_channels=dims.hd, ffn_hidden_size=dims.ffn, num_layers=layers, num_nanobatches=nnb,
                      backend="hip", **kw)
    model = LayerStack(cfg, device="cuda", seed=1234)
    # split-K changes the order of the contraction sum, and which GEMMs split depends on the mode (alone on
    # the GPU, beside other nanobatch streams, with a fused epilogue — which never splits): for bit-exact
    # comparisons across modes no GEMM splits
    for layer in model.layers:
        for op in (layer.linear_qkv, layer.linear_proj, layer.linear_fc1, layer.linear_fc2):
            op.split_k = None
    return model


def _run(model, x, go):
    for p in model.parameters():
        p.grad = None
    xd = x.to("cuda", torch.bfloat16).requires_grad_(True)
    y = model(xd)
    y.backward(go.to("cuda", torch.bfloat16))
    torch.cuda.synchronize()
    grads = [[getattr(layer, a).weight.grad.clone() for a, _ in PARAMS] for layer in model.layers]
    return y.detach(), xd.grad, grads


def _oracle(model, dims, x, go):
    params = [{n: getattr(layer, a).weight.detach().float().cpu() for a, n in PARAMS} for layer in model.layers]
    return R.stack_forward_backward(x.bfloat16().float(), params, dims, go.bfloat16().float())


def _rel(got, want):
    got, want = got.float().cpu(), want.float().cpu()
    return ((got - want).abs().max() / want.abs().max()).item(), (got - want).abs().max().item()


@pytest.mark.parametrize("dims,s,b,layers", [
    (R.LayerDims(512, 8, 8, 64, 1376), 256, 4, 1),      # benchmark configuration 1's layer exactly (8 heads of 64), in bf16
    (R.LayerDims(512, 4, 4, 128, 1376), 200, 4, 1),     # the same widths with head_dim 128 and a ragged sequence length
    (R.LayerDims(3072, 3, 1, 128, 1024), 512, 4, 1),    # config 2 widths (3B TP=8 shard), short sequence
    (R.LayerDims(1024, 8, 2, 128, 896), 384, 4, 2),     # config 4 ratios (8 q / 2 kv heads), two layers
])
@pytest.mark.parametrize("nnb", [1, 2, 4])
def test_layer_matches_oracle(dims, s, b, layers, nnb):
    x, go = _inputs(s, b, dims.hidden)
    model = _build(dims, layers, nnb)
    y, dx, grads = _run(model, x, go)
    ry, rdx, rgrads = _oracle(model, dims, x, go)
    worst = [_rel(y, ry), _rel(dx, rdx)]
    for li in range(layers):
        for pi, (_, name) in enumerate(PARAMS):
            worst.append(_rel(grads[li][pi], rgrads[li][name]))
    print(f"nnb={nnb} max-rel={max(w[0] for w in worst):.3e} max-abs={max(w[1] for w in worst):.3e}")
    assert max(w[0] for w in worst) <= TOL


@pytest.mark.parametrize("dims,s,b", [(R.LayerDims(1024, 8, 2, 128, 896), 384, 4), (R.LayerDims(512, 8, 8, 64, 1376), 256, 2)])
def test_layer_with_hidden_dropout_matches_oracle_given_the_masks(dims, s, b):
    """Hidden dropout in front of the two residual adds (bias_dropout_add.py:24-45; the reference's training
    configuration uses 0.1): the masks the two operators drew go to the oracle, everything else as in
    test_layer_matches_oracle.  With recomputation the backward pass draws the same masks again (generator
    states saved and replayed, autograd_function.py:143-146, 263-266) and the step is bit-identical; with two
    nanobatches, each drawing its own masks, the same seed still gives the same step."""
    prob = 0.1
    x, go = _inputs(s, b, dims.hidden)
    model = _build(dims, 1, 1, hidden_dropout=prob)
    torch.manual_seed(21)
    y, dx, grads = _run(model, x, go)
    layer = model.layers[0]
    m1, m2 = layer.self_attn_bda.last_mask.float().cpu(), layer.mlp_bda.last_mask.float().cpu()
    assert m1.shape == (s, b, dims.hidden) and 0.88 < m1.mean() < 0.92 and 0.88 < m2.mean() < 0.92
    params = {n: getattr(layer, a).weight.detach().float().cpu().requires_grad_(True) for a, n in PARAMS}
    xx = x.bfloat16().float().requires_grad_(True)
    ry = R.layer_forward(xx, params, dims, R.rope_table(s, dims.hd, dims.rope_base), dropout=(prob, m1, m2))
    ry.backward(go.bfloat16().float())
    worst = [_rel(y, ry.detach()), _rel(dx, xx.grad)] + [_rel(grads[0][pi], params[n].grad) for pi, (_, n) in enumerate(PARAMS)]
    print(f"hidden dropout {prob}: max-rel={max(w[0] for w in worst):.3e}")
    assert max(w[0] for w in worst) <= TOL
    recomputing = _build(dims, 1, 1, hidden_dropout=prob, checkpoint_activations=True)
    torch.manual_seed(21)
    y2, dx2, grads2 = _run(recomputing, x, go)
    assert torch.equal(y, y2) and torch.equal(dx, dx2)
    assert all(torch.equal(a, c) for a, c in zip(grads[0], grads2[0]))
    two = _build(dims, 1, 2, hidden_dropout=prob)
    torch.manual_seed(22)
    ya, dxa, ga = _run(two, x, go)
    torch.manual_seed(22)
    yb, dxb, gb = _run(two, x, go)
    assert torch.equal(ya, yb) and torch.equal(dxa, dxb) and all(torch.equal(a, c) for a, c in zip(ga[0], gb[0]))
    assert not torch.equal(ya, y)


@pytest.mark.parametrize("dims,s,b,nnb", [
    (R.LayerDims(2048, 4, 2, 128, 1536), 384, 4, 1),   # Qwen3-1.7B widths (16 q / 8 kv heads of 128) at TP=4
    (R.LayerDims(2048, 4, 2, 128, 1536), 384, 4, 2),
    (R.LayerDims(512, 8, 8, 64, 1376), 200, 2, 2),     # one query head per group, 64 channels, ragged length
    (R.LayerDims(2048, 2, 1, 128, 768), 256, 8, 2),     # the TP=8 shard at MBS 8: nanobatches of four sequences, addressed in row runs
])
def test_layer_with_query_and_key_norms_matches_oracle(dims, s, b, nnb):
    """Qwen3-style layers (qk_layernorm): an RMSNorm over the head dimension of every query head and of every
    key head between the QKV split and the rotary embedding (qkv_postprocess.py:115-118, 150-157).  Output, input
    gradient and all gradients, the two head-norm weights' included, against the oracle; recomputation and the
    nanobatch streams change no bit."""
    x, go = _inputs(s, b, dims.hidden)
    model = _build(dims, 2, nnb, qk_layernorm=True)
    gen = torch.Generator().manual_seed(9)
    heads = [("q_layernorm", "q_norm"), ("k_layernorm", "k_norm")]
    for layer in model.layers:
        for attr, _ in heads:
            with torch.no_grad():
                getattr(layer.qkv_postprocess, attr).weight.copy_(1 + 0.3 * torch.randn(dims.hd, generator=gen))

    def run(m):
        y, dx, grads = _run(m, x, go)
        extra = [[getattr(layer.qkv_postprocess, a).weight.grad.clone() for a, _ in heads] for layer in m.layers]
        return y, dx, grads, extra

    y, dx, grads, extra = run(model)
    params = [{**{n: getattr(layer, a).weight.detach().float().cpu() for a, n in PARAMS},
               **{n: getattr(layer.qkv_postprocess, a).weight.detach().float().cpu() for a, n in heads}}
              for layer in model.layers]
    ry, rdx, rgrads = R.stack_forward_backward(x.bfloat16().float(), params, dims, go.bfloat16().float())
    worst = [_rel(y, ry), _rel(dx, rdx)]
    for li in range(2):
        worst += [_rel(grads[li][pi], rgrads[li][name]) for pi, (_, name) in enumerate(PARAMS)]
        worst += [_rel(extra[li][pi], rgrads[li][name]) for pi, (_, name) in enumerate(heads)]
    print(f"qk_layernorm nnb={nnb} max-rel={max(w[0] for w in worst):.3e} max-abs={max(w[1] for w in worst):.3e}")
    assert max(w[0] for w in worst) <= TOL
    plain = [{n: t for n, t in p.items() if n not in ("q_norm", "k_norm")} for p in params]
    without = R.stack_forward(x.bfloat16().float(), plain, dims, R.rope_table(s, dims.hd, dims.rope_base))
    assert _rel(without, ry)[0] > 2 * TOL       # the norms matter at this tolerance
    other = _build(dims, 2, nnb, qk_layernorm=True, checkpoint_activations=True, use_streams=False)
    other.load_state_dict(model.state_dict())
    y2, dx2, grads2, extra2 = run(other)
    assert torch.equal(y, y2) and torch.equal(dx, dx2)
    for la, lb in zip(grads + extra, grads2 + extra2):
        assert all(torch.equal(a, c) for a, c in zip(la, lb))


def test_streams_recompute_and_schedule_do_not_change_results(fixtures_dir):
    dims = R.LayerDims(1024, 8, 2, 128, 896)
    x, go = _inputs(256, 4, dims.hidden)
    base = _run(_build(dims, 2, 2, use_streams=False), x, go)

    def same(other):
        assert torch.equal(other[0], base[0]) and torch.equal(other[1], base[1])
        for la, lb in zip(other[2], base[2]):
            for ga, gb in zip(la, lb):
                assert torch.equal(ga, gb)

    same(_run(_build(dims, 2, 2, use_streams=True), x, go))            # concurrent streams: bit-identical
    same(_run(_build(dims, 2, 2, checkpoint_activations=True), x, go))  # recompute: bit-identical
    model = _build(dims, 2, 2, checkpoint_activations=True)
    sch = PipelineCommScheduler(os.path.join(fixtures_dir, "scheds_pipeline_02328.py"), pp_rank=0,
                                num_microbatches=8, use_activation_checkpointing=True)
    model.config.kareus_scheduler = sch
    for p in model.parameters():
        p.grad = None
    xd = x.to("cuda", torch.bfloat16).requires_grad_(True)
    sch.on_step_begin()
    sch.on_instruction_begin("forward")
    y = model(xd)
    sch.on_instruction_begin("forward")          # stage 0 of the shipped plan runs F F B ...
    sch.on_instruction_begin("backward")
    y.backward(go.to("cuda", torch.bfloat16))
    torch.cuda.synchronize()
    assert torch.equal(y.detach(), base[0]) and torch.equal(xd.grad, base[1])  # any legal schedule: same numbers
    # repeated steps are deterministic
    m2 = _build(dims, 2, 4)
    r1, r2 = _run(m2, x, go), _run(m2, x, go)
    assert torch.equal(r1[0], r2[0]) and torch.equal(r1[1], r2[1]) and torch.equal(r1[2][1][4], r2[2][1][4])


def test_fused_epilogues_do_not_change_results():
    """SwiGLU in fc1's epilogue, the residual adds in the epilogues of the out-projection and fc2, and the
    RMSNorm weight gradient summed over nanobatches in fp32: outputs, input gradients and the linear layers'
    weight gradients are bit-identical to the engine running every operator as its own kernel (the GEMMs never
    split the contraction here: a fused epilogue cannot, and splitting changes the order of the sum); only the
    norm weights' gradients differ, by the one rounding the fp32 sum saves."""
    dims = R.LayerDims(1024, 8, 2, 128, 896)
    x, go = _inputs(256, 4, dims.hidden)
    runs = {}
    for fuse in (True, False):
        for nnb in (1, 2, 4):
            model = _build(dims, 2, nnb, fuse_forward_epilogues=fuse)
            for layer in model.layers:
                for op in (layer.linear_qkv, layer.linear_proj, layer.linear_fc1, layer.linear_fc2):
                    op.split_k = None
            runs[fuse, nnb] = _run(model, x, go)
    for nnb in (1, 2, 4):
        a, b = runs[True, nnb], runs[False, nnb]
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
        for la, lb in zip(a[2], b[2]):
            for (attr, _), ga, gb in zip(PARAMS, la, lb):
                if "layernorm" in attr:
                    assert _rel(ga, gb)[0] <= 1e-2
                else:
                    assert torch.equal(ga, gb)


def test_full_size_properties_config4():
    """Benchmark configuration 4 at full size (h4096, 8q/2kv, ffn 3584, MBS 4 x seq 4096): too large for the CPU
    oracle in test time, so check properties that hold at any size."""
    dims = R.LayerDims(4096, 8, 2, 128, 3584)
    s, b = 4096, 4
    x, go = _inputs(s, b, dims.hidden)
    y4, dx4, g4 = _run(_build(dims, 1, 4), x, go)
    y1, dx1, g1 = _run(_build(dims, 1, 1), x, go)
    # per-sample ops: outputs and input gradients do not depend on the nanobatch count (the GEMMs may
    # cut the contraction differently for different row counts, so equal up to rounding, not bitwise)
    assert _rel(y4, y1)[0] <= TOL and _rel(dx4, dx1)[0] <= TOL
    # weight gradients: sum over nanobatches (bf16 accumulation order differs) within tolerance
    for a, c in zip(g4[0], g1[0]):
        assert _rel(a, c)[0] <= TOL
    # causality end to end: perturbing the last 1024 positions leaves the first 3072 outputs unchanged
    x2 = x.clone()
    x2[3072:] += 1.0
    y2, _, _ = _run(_build(dims, 1, 4), x2, go)
    assert torch.equal(y2[:3072], y4[:3072]) and not torch.equal(y2[3072:], y4[3072:])
    # linearity of backward in the upstream gradient: dx(2*go) == 2*dx(go) exactly in bf16 (power of two)
    _, dx_double, _ = _run(_build(dims, 1, 4), x, 2 * go)
    assert torch.equal(dx_double, 2 * dx4)
    assert torch.isfinite(y4).all() and torch.isfinite(dx4).all()


# ---- benchmark configurations 3 and 5: full widths ------------------------------------------------
C3 = R.LayerDims(3072, 24, 8, 128, 8192)     # Llama-3.2-3B layer, TP=1 (tests/bayesian/common/model_config.py:88-96)
C5 = R.LayerDims(4096, 32, 8, 128, 14336)    # Llama-3.1-8B layer, full width


@pytest.mark.parametrize("nnb", [1, 2, 4])
def test_config3_widths_match_oracle(nnb):
    """Configuration 3 at its full widths (24 query / 8 KV heads, ffn 8192), MBS 4, with the sequence cut to
    256 so the CPU oracle finishes in seconds; nanobatch counts 1 (serial), 2 and 4."""
    s, b = 256, 4
    x, go = _inputs(s, b, C3.hidden)
    model = _build(C3, 1, nnb)
    y, dx, grads = _run(model, x, go)
    ry, rdx, rgrads = _oracle(model, C3, x, go)
    worst = [_rel(y, ry), _rel(dx, rdx)] + [_rel(grads[0][pi], rgrads[0][n]) for pi, (_, n) in enumerate(PARAMS)]
    print(f"c3 nnb={nnb} max-rel={max(w[0] for w in worst):.3e} max-abs={max(w[1] for w in worst):.3e}")
    assert max(w[0] for w in worst) <= TOL


def _scheduled_step(model, sch, x, go):
    """One microbatch under the activation-checkpointing plan: a forward and a backward instruction."""
    for p in model.parameters():
        p.grad = None
    xd = x.to("cuda", torch.bfloat16).requires_grad_(True)
    sch.on_instruction_begin("forward")
    y = model(xd)
    sch.on_instruction_end("forward")
    sch.on_instruction_begin("backward")
    y.backward(go.to("cuda", torch.bfloat16))
    sch.on_instruction_end("backward")
    torch.cuda.synchronize()
    grads = [[getattr(layer, a).weight.grad.clone() for a, _ in PARAMS] for layer in model.layers]
    return y.detach(), xd.grad, grads


def test_config5_widths_match_oracle():
    """One layer of configuration 5's widths (32 query / 8 KV heads, ffn 14336), MBS 2, two nanobatches, at the
    single-layer tolerance."""
    x, go = _inputs(256, 2, C5.hidden)
    model = _build(C5, 1, 2)
    y, dx, grads = _run(model, x, go)
    ry, rdx, rgrads = _oracle(model, C5, x, go)
    worst = [_rel(y, ry), _rel(dx, rdx)] + [_rel(grads[0][pi], rgrads[0][n]) for pi, (_, n) in enumerate(PARAMS)]
    print(f"c5 one layer max-rel={max(w[0] for w in worst):.3e} max-abs={max(w[1] for w in worst):.3e}")
    assert max(w[0] for w in worst) <= TOL


def _one_layer_models(stack, dims, nnb):
    """One single-layer model per layer of ``stack``, holding that layer's weights."""
    singles = []
    for layer in stack.layers:
        one = _build(dims, 1, nnb)
        with torch.no_grad():
            for attr, _ in PARAMS:
                getattr(one.layers[0], attr).weight.copy_(getattr(layer, attr).weight)
        singles.append(one)
    return singles


def test_config5_stack_under_a_schedule_file_matches_oracle(fixtures_dir):
    """Configuration 5 at its full widths, four layers, MBS 2, two nanobatches, activations recomputed, every
    partition's launch slot taken from a schedule file (two microbatches: both steps of the plan are run and
    checked); sequence cut to 256 for the oracle.

    The stated tolerance, 2e-2, is the bf16 bound for one layer against fp32 on the same inputs, so the stack
    is checked layer by layer (operator order of a layer: transformer_layer.py:148-174): layer l alone, on
    the device, is given the bf16 input that layer l-1 produced and — backward — the bf16 gradient that layer
    l+1 handed down; its output, input gradient and six weight gradients are compared at 2e-2 with ONE oracle
    layer in fp32 fed exactly those tensors; and the stack's output, input gradient and all weight gradients
    must equal that chain's bit for bit, so every layer of the stack is pinned at the stated bound with
    nothing widened for depth.  The scheduled, recomputing run must also equal the plain run of the same
    stack bit for bit."""
    s, b, layers = 256, 2, 4
    model = _build(C5, layers, 2, checkpoint_activations=True)
    plain = _build(C5, layers, 2)
    singles = _one_layer_models(model, C5, 2)
    sch = PipelineCommScheduler(os.path.join(fixtures_dir, "single_stage_ac.py"), pp_rank=0,
                                num_microbatches=2, use_activation_checkpointing=True)
    model.config.kareus_scheduler = sch
    sch.on_step_begin()
    for mb in range(2):
        x, go = _inputs(s, b, C5.hidden, seed=42 + mb)
        y, dx, grads = _scheduled_step(model, sch, x, go)
        py, pdx, pgrads = _run(plain, x, go)
        assert torch.equal(y, py) and torch.equal(dx, pdx)
        assert all(torch.equal(a, c) for la, lb in zip(grads, pgrads) for a, c in zip(la, lb))

        # the chain of single layers: forward inputs first, then the gradients from the top down
        xs = [x.bfloat16()]
        for one in singles:
            with torch.no_grad():
                xs.append(one(xs[-1].to("cuda")).cpu())
        gos = [None] * layers + [go.bfloat16()]
        worst = []
        for li in reversed(range(layers)):
            cy, cdx, cgrads = _run(singles[li], xs[li].float(), gos[li + 1].float())
            gos[li] = cdx.cpu()
            assert torch.equal(cy.cpu(), xs[li + 1])
            assert all(torch.equal(a, c) for a, c in zip(cgrads[0], grads[li]))      # the stack's layer li
            ry, rdx, rgrads = _oracle(singles[li], C5, xs[li].float(), gos[li + 1].float())
            errs = [_rel(cy, ry), _rel(cdx, rdx)] + [_rel(cgrads[0][pi], rgrads[0][n]) for pi, (_, n) in enumerate(PARAMS)]
            print(f"c5 microbatch {mb} layer {li} max-rel={max(e[0] for e in errs):.3e} "
                  f"max-abs={max(e[1] for e in errs):.3e}")
            worst += errs
        assert torch.equal(xs[layers], y.cpu()) and torch.equal(gos[0], dx.cpu())    # chain == stack
        assert max(w[0] for w in worst) <= TOL
    sch.on_step_end()


def _size_independent_properties(dims, layers, s, b, counts, cut, **kw):
    """Properties that hold at any size: results do not depend on the nanobatch count, the layer is
    causal end to end, the backward is linear in the upstream gradient, everything is finite."""
    x, go = _inputs(s, b, dims.hidden)
    runs = {n: _run(_build(dims, layers, n, **kw), x, go) for n in counts}
    base = runs[counts[0]]
    for n in counts[1:]:
        y, dx, g = runs[n]
        assert _rel(y, base[0])[0] <= TOL and _rel(dx, base[1])[0] <= TOL
        for la, lb in zip(g, base[2]):
            for ga, gb in zip(la, lb):
                assert _rel(ga, gb)[0] <= TOL
    n = counts[-1]
    x2 = x.clone()
    x2[cut:] += 1.0
    y2, _, _ = _run(_build(dims, layers, n, **kw), x2, go)
    assert torch.equal(y2[:cut], runs[n][0][:cut]) and not torch.equal(y2[cut:], runs[n][0][cut:])
    _, dx_double, _ = _run(_build(dims, layers, n, **kw), x, 2 * go)
    assert torch.equal(dx_double, 2 * runs[n][1])
    for y, dx, g in runs.values():
        assert torch.isfinite(y).all() and torch.isfinite(dx).all()
        assert all(torch.isfinite(t).all() for layer in g for t in layer)


def test_full_size_properties_config3():
    """Configuration 3 at full size (h3072, 24q/8kv, ffn 8192, MBS 4 x seq 4096), nanobatch counts 1, 2, 4."""
    _size_independent_properties(C3, 1, 4096, 4, [1, 2, 4], cut=3072)


def test_full_size_properties_config5():
    """Configuration 5 at full size (4 layers, h4096, 32q/8kv, ffn 14336, MBS 2 x seq 8192, 2 nanobatches)."""
    _size_independent_properties(C5, 4, 8192, 2, [1, 2], cut=6144)


def test_full_size_properties_qwen3_shard_with_head_norms():
    """The reference's Qwen3-1.7B configuration (h2048, 16q/8kv heads of 128, ffn 6144, qk_layernorm; seq 4096)
    as a TP=4 shard at MBS 4, nanobatch counts 1, 2, 4."""
    _size_independent_properties(R.LayerDims(2048, 4, 2, 128, 1536), 1, 4096, 4, [1, 2, 4], cut=3072,
                                 qk_layernorm=True)


def test_nanobatch_streams_do_not_share_a_hardware_queue():
    """Streams handed to the nanobatches must overlap for real: a short kernel on one finishes
    while a spinning kernel occupies the other."""
    from kareus_amd.partitions.streams import _run_concurrently, stream_api

    two = stream_api().new_streams(2)
    assert len(two) == 2 and two[0] != two[1]
    assert _run_concurrently(two[0], two[1]) and _run_concurrently(two[1], two[0])
    four = stream_api().new_streams(4)
    assert len({s.cuda_stream for s in four}) == 4
    # one stream cannot overtake itself: the probe must say so
    assert not _run_concurrently(two[0], two[0])
