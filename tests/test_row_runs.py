"""Nanobatches of several sequences addressed in place ("row runs").

A nanobatch of r sequences cut out of a [s, b, h] tensor along the batch axis
(kareus/megatron/core/transformer/transformer_block.py:483-485) has its rows in runs of r whose starts are
b*h apart.  The reference copies such a slice into a dense tensor in every linear layer
(kareus/transformer_engine/pytorch/ops/basic/basic_linear.py:565-569); the kernels here read and write it
where it lies.  Addressing moves no arithmetic, so every check is bit-exact against the same kernel fed a
dense copy of the slice; the copy-based path is itself checked against the oracle elsewhere.
"""

import pytest
import torch

from kareus_amd.backend.hip import HipBackend

DEV = "cuda"


def gpu(test):
    """Marks a test that needs the device."""
    return pytest.mark.gpu(pytest.mark.skipif(not torch.cuda.is_available(), reason="needs a HIP device")(test))


# ---- host logic: which tensors the kernels can address as they lie ---------------------------------
def test_operand_classification():
    op = HipBackend._operand
    whole = torch.empty(40, 8, 64, dtype=torch.bfloat16)            # [s, b, h]
    assert op(whole[:, 0:1]) == (40, 8 * 64, 1, 0)                   # one sequence: a matrix with row stride b*h
    assert op(whole[:, 2:4]) == (80, 64, 2, 8 * 64)                  # two sequences: runs of 2 rows, b*h apart
    assert op(whole[:, 4:8]) == (160, 64, 4, 8 * 64)
    assert op(whole[:, 0:8]) == (320, 64, 1, 0)                      # all of them: dense again
    assert op(whole[:, 1:4]) is None                                 # 3 sequences: not a power of two -> copy
    assert op(torch.empty(40, 32, 64, dtype=torch.bfloat16)[:, :17]) is None
    assert op(torch.empty(4, 64, 64, dtype=torch.bfloat16)[:, :32]) is None          # more than 16 rows per run
    assert op(torch.empty(40, 8, 60, dtype=torch.bfloat16)[:, 0:2]) is None          # row stride not a multiple of 8
    assert op(torch.empty(16, 128, dtype=torch.bfloat16)[:, :64]) == (16, 128, 1, 0)  # a plain row-strided matrix
    assert op(torch.empty(16, 128, dtype=torch.bfloat16).t()) is None                # column stride not 1
    be = HipBackend.__new__(HipBackend)                              # the view helpers need no library
    assert be.rows_view(whole[:, 2:4]) is not None and be.rows_view(whole[:, 2:4]).dim() == 3
    assert be.rows_view(whole[:, 0:1]).shape == (40, 64)
    assert be.rows_view(whole[:, 1:4]) is None
    dense = be.rows_in_place(whole[:, 1:4])
    assert dense.shape == (120, 64) and dense.is_contiguous()


def test_entry_points_reject_bad_runs_without_a_device():
    from kareus_amd.backend import hip

    lib = hip.load_library()
    # rows per run: a power of two, at most 16 for the GEMM, dividing the row count; run starts a multiple of 8 apart
    g = lambda a_rows, a_ld, c_rows=1, c_ld=0, acc=0, epi=0: lib.kr_gemm_bf16_runs(
        0, 64, 64, 64, 16, 64, a_rows, a_ld, 16, 64, 16, 64, c_rows, c_ld, acc, epi, None, 0, 1, 0, None, 0, 0, None, 0, None)
    assert g(3, 512) == -1 and g(32, 4096) == -2 and g(2, 500) == -2 and g(2, 0) == -1
    assert g(1, 0, 2, 512, acc=1) == -2                                  # an output in runs cannot accumulate
    assert lib.kr_rmsnorm_fwd_runs(16, 16, 16, 16, 6, 64, 64, 4, 512, 1e-5, None) == -2    # 6 rows, runs of 4
    assert lib.kr_rmsnorm_fwd_runs(16, 16, 16, 16, 8, 64, 64, 3, 512, 1e-5, None) == -1
    assert lib.kr_rmsnorm_bwd_add_runs(16, 16, 16, 16, None, 16, 16, 16, 8, 64, 64, 64, 2, 100, 0, 1, 0, 64, 1, 0, None) == -2


# ---- kernels ------------------------------------------------------------------------------------------
def _rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(DEV, torch.bfloat16)


@pytest.fixture(scope="module")
def be():
    from kareus_amd.backend import get_backend

    return get_backend("hip")


def _slice(s, b, cols, lo, r, seed):
    """A [s, r, cols] nanobatch slice of a [s, b, cols] tensor, and the tensor."""
    whole = _rnd(s, b, cols, seed=seed)
    return whole[:, lo:lo + r], whole


@gpu
@pytest.mark.parametrize("s,b,r,cols", [(256, 8, 4, 3072), (300, 4, 2, 512), (64, 16, 8, 4096), (130, 32, 16, 1024)])
def test_rmsnorm_reads_and_writes_runs_in_place(be, s, b, r, cols):
    x, _ = _slice(s, b, cols, r, r, seed=1)
    gamma = (1 + 0.1 * _rnd(cols, seed=2).float()).bfloat16()
    assert be.rows_view(x).dim() == 3                                    # addressed as it lies
    y, rstd = be.rmsnorm_fwd(x, gamma, 1e-5)
    y0, rstd0 = be.rmsnorm_fwd(x.reshape(-1, cols).contiguous(), gamma, 1e-5)
    assert torch.equal(y, y0) and torch.equal(rstd, rstd0)
    # backward: saved input, residual gradient and result each in runs, alone and together
    dy = _rnd(s * r, cols, seed=3)
    dres, _ = _slice(s, b, cols, 0, r, seed=4)
    dx_whole = torch.zeros(s, b, cols, device=DEV, dtype=torch.bfloat16)
    sink = dx_whole[:, b - r:]
    want_dx, want_dg = be.rmsnorm_bwd(dy, x.reshape(-1, cols).contiguous(), rstd, gamma,
                                      residual_grad=dres.reshape(-1, cols).contiguous())
    got_dx, got_dg = be.rmsnorm_bwd(dy, x, rstd, gamma, residual_grad=dres, out=sink)
    assert got_dx is sink and torch.equal(sink.reshape(-1, cols), want_dx) and torch.equal(got_dg, want_dg)
    assert not dx_whole[:, :b - r].any()                                 # nothing outside the slice was touched
    only_x, _ = be.rmsnorm_bwd(dy, x, rstd, gamma, residual_grad=dres.reshape(-1, cols).contiguous())
    only_res, _ = be.rmsnorm_bwd(dy, x.reshape(-1, cols).contiguous(), rstd, gamma, residual_grad=dres)
    assert torch.equal(only_x, want_dx) and torch.equal(only_res, want_dx)
    plain, _ = be.rmsnorm_bwd(dy, x, rstd, gamma)                        # no residual gradient
    plain0, _ = be.rmsnorm_bwd(dy, x.reshape(-1, cols).contiguous(), rstd, gamma)
    assert torch.equal(plain, plain0)


@gpu
@pytest.mark.parametrize("s,b,r,n,k", [(256, 8, 4, 768, 512), (300, 4, 2, 520, 200), (64, 16, 8, 4096, 1024),
                                       (136, 32, 16, 640, 384), (1024, 4, 2, 3072, 1024)])
def test_gemm_operands_and_output_in_runs(be, s, b, r, n, k):
    m = s * r
    w = _rnd(n, k, seed=11, scale=0.05)
    # forward with the residual add: residual in runs, output in runs (the two ends of a layer stack)
    x = _rnd(m, k, seed=12)
    res, _ = _slice(s, b, n, r, r, seed=13)
    want = be.linear_fwd(x, w, split_k=None, residual=res.reshape(-1, n).contiguous())
    assert torch.equal(be.linear_fwd(x, w, split_k=None, residual=res), want)
    out_whole = torch.zeros(s, b, n, device=DEV, dtype=torch.bfloat16)
    sink = out_whole[:, 0:r]
    got = be.linear_fwd(x, w, split_k=None, residual=res.reshape(-1, n).contiguous(), out=sink)
    assert got is sink and torch.equal(sink.reshape(-1, n), want) and not out_whole[:, r:].any()
    both = torch.zeros(s, b, n, device=DEV, dtype=torch.bfloat16)
    be.linear_fwd(x, w, split_k=None, residual=res, out=both[:, b - r:])
    assert torch.equal(both[:, b - r:].reshape(-1, n), want)
    with pytest.raises(RuntimeError, match="not supported"):            # no forward instance without the residual add
        be.linear_fwd(x, w, split_k=None, out=torch.zeros(s, b, n, device=DEV, dtype=torch.bfloat16)[:, 0:r])
    # backward: the incoming gradient in runs feeds the input gradient (A of layout NN) and the weight
    # gradient (layout NT: its rows are the contraction), also cut along K and accumulated
    dy, _ = _slice(s, b, n, b - r, r, seed=14)
    dyc = dy.reshape(-1, n).contiguous()
    assert torch.equal(be.linear_dgrad(dy, w, split_k=None), be.linear_dgrad(dyc, w, split_k=None))
    for split in (None, True, False):
        assert torch.equal(be.linear_wgrad(dy, x, split_k=split), be.linear_wgrad(dyc, x, split_k=split))
    acc0 = _rnd(n, k, seed=15)
    a, c = acc0.clone(), acc0.clone()
    be.linear_wgrad(dy, x, out=a, accumulate=True, split_k=None)
    be.linear_wgrad(dyc, x, out=c, accumulate=True, split_k=None)
    assert torch.equal(a, c)


@gpu
@pytest.mark.parametrize("s,b,r,f,h", [(256, 8, 4, 1024, 768), (200, 4, 2, 448, 512)])
def test_input_gradient_with_swiglu_backward_reads_runs(be, s, b, r, f, h):
    """fc2's input gradient with the SwiGLU backward in its epilogue, fed the block's incoming gradient as it lies."""
    m = s * r
    w2 = _rnd(h, f, seed=21, scale=0.05)
    act_in = _rnd(m, 2 * f, seed=22)
    dy, _ = _slice(s, b, h, 0, r, seed=23)
    want = be.linear_dgrad(dy.reshape(-1, h).contiguous(), w2, split_k=None, swiglu_bwd_x=act_in)
    assert torch.equal(be.linear_dgrad(dy, w2, split_k=None, swiglu_bwd_x=act_in), want)


# ---- the whole layer: several sequences per nanobatch, no copy at either end -------------------------------
@gpu
@pytest.mark.parametrize("b,nnb", [(8, 2), (4, 2), (16, 2), (8, 4)])
def test_layer_with_wide_nanobatches_equals_the_copying_run(monkeypatch, b, nnb):
    """Configuration 2's widths (3072 hidden, 3 query / 1 KV head, ffn 1024), 4 / 2 / 8 / 2 sequences per
    nanobatch: the run that addresses the nanobatch slices in place gives the bits of the run that copies
    them into dense tensors first (the reference's way), for outputs, input gradients and every weight
    gradient; and the nanobatch tensors it hands the engine are views of the caller's tensor."""
    from kareus_amd import LayerConfig, LayerStack
    from kareus_amd import block as blk

    s, h = 256, 3072
    cfg = dict(hidden_size=h, num_attention_heads=3, num_query_groups=1, kv_channels=128, ffn_hidden_size=1024,
               num_layers=2, num_nanobatches=nnb, backend="hip")

    def run():
        model = LayerStack(LayerConfig(**cfg), device=DEV, seed=1234)
        for layer in model.layers:
            for op in (layer.linear_qkv, layer.linear_proj, layer.linear_fc1, layer.linear_fc2):
                op.split_k = None
        g = torch.Generator().manual_seed(5)
        x = torch.randn(s, b, h, generator=g).to(DEV, torch.bfloat16).requires_grad_(True)
        go = torch.randn(s, b, h, generator=g).to(DEV, torch.bfloat16)
        y = model(x)
        y.backward(go)
        torch.cuda.synchronize()
        return [y.detach(), x.grad] + [p.grad for p in model.parameters()]

    seen = []
    split = blk._SplitNanobatches.forward

    def watch(ctx, hidden_states, n, backend="eager"):
        parts = split(ctx, hidden_states, n, backend)
        seen.append(all(p.untyped_storage().data_ptr() == hidden_states.untyped_storage().data_ptr() for p in parts))
        return parts

    monkeypatch.setattr(blk._SplitNanobatches, "forward", staticmethod(watch))
    in_place = run()
    assert seen == [True]                                    # the nanobatches are views of the caller's tensor
    monkeypatch.setattr(HipBackend, "MAX_RUN_ROWS", 1)       # no runs: wide nanobatches are copied, as before
    copying = run()
    assert seen == [True, False]
    assert len(in_place) == len(copying) and all(torch.equal(a, c) for a, c in zip(in_place, copying))

